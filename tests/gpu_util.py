"""Helpers shared by the GPU parity tests."""
import numpy as np


def to_dev(torch, a, kind=None):
    """numpy -> device tensor.  `kind` = 'bf16' / 'f16' reinterprets uint16 bit patterns."""
    a = np.ascontiguousarray(a)
    if kind == "bf16":
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    if kind == "f16":
        return torch.from_numpy(a.view(np.float16)).cuda()
    return torch.from_numpy(a).cuda()


def bits(torch, t):
    """device 16-bit tensor -> numpy uint16 bit patterns."""
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def error_bound_16(ref64, S, K, kind, c=2.0):
    """|gpu - ref64| <= u_out*|ref64| + c*K*2^-24*S (+ half the smallest subnormal).
    u_out: unit roundoff of the single output narrowing (2^-11 fp16, 2^-8 bf16); the second
    term bounds fp32 accumulation of K exact products in any order (first-order gamma_K,
    with slack factor c)."""
    u_out = 2.0 ** -11 if kind == "f16" else 2.0 ** -8
    tiny = 2.0 ** -25 if kind == "f16" else 0.0
    return u_out * np.abs(ref64) + c * K * 2.0 ** -24 * S * (1 + u_out) + tiny

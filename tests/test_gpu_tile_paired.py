"""The paired form of the tile kernel (libcigemm_probe.so, cigemm_probe_gemm_*_paired): 128-row
tiles and two workgroups resident per compute unit.  Same arithmetic as the one-per-unit kernel: int8 bit-exact against the oracle,
16-bit bit-exact on exact-arithmetic inputs and within the K-scaled bound on N(0,1) inputs;
ragged edges, partly filled last stages of K, guard rows and columns untouched."""
import numpy as np
import pytest

import cudaintro_amd as ci
from cudaintro_amd import probe
from gpu_util import bits, error_bound_16, to_dev

pytestmark = pytest.mark.gpu

VALS = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
SHAPES = [(128, 256, 64), (128, 256, 128), (128, 256, 192), (256, 512, 256), (100, 264, 1000),
          (513, 1032, 328), (64, 2048, 2048 + 16), (1000, 520, 72), (300, 256, 8), (1, 8, 8),
          (2048, 2048, 2048), (4096, 1024, 512)]


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_paired_16bit_exact_inputs(handle, torch_gpu, oracle, rng, kind, M, N, K):
    torch = torch_gpu
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    widen = oracle.bf16_to_f32 if kind == "bf16" else oracle.f16_to_f32
    Ab, Bb = narrow(rng.choice(VALS, size=(M, K))), narrow(rng.choice(VALS, size=(K, N)))
    out = torch.full((M + 1, N + 8), 3.0, dtype=torch.bfloat16 if kind == "bf16" else torch.float16,
                     device="cuda")
    probe.gemm16_paired(handle, to_dev(torch, Ab, kind), to_dev(torch, Bb, kind), out=out[:M, :N])
    assert "_mfma_128x256x32_w4x2_ring3" in handle.last_kernel, handle.last_kernel
    assert handle.last_plan == (128, 1)
    o = bits(torch, out)
    np.testing.assert_array_equal(o[:M, :N], narrow(oracle.gemm_f32(widen(Ab), widen(Bb))))
    three = narrow(np.float32(3.0))
    assert (o[M:] == three).all() and (o[:, N:] == three).all()


@pytest.mark.parametrize("kind", ["bf16", "f16"])
def test_paired_16bit_normal_inputs(handle, torch_gpu, oracle, rng, kind):
    torch = torch_gpu
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    widen = oracle.bf16_to_f32 if kind == "bf16" else oracle.f16_to_f32
    M, N, K = 1024, 1024, 4096
    Ab = narrow(rng.standard_normal((M, K)).astype(np.float32))
    Bb = narrow(rng.standard_normal((K, N)).astype(np.float32))
    c = probe.gemm16_paired(handle, to_dev(torch, Ab, kind), to_dev(torch, Bb, kind))
    ref, S = oracle.gemm_f64(widen(Ab), widen(Bb), with_abs=True)
    err = np.abs(widen(bits(torch, c)).astype(np.float64) - ref)
    assert (err <= error_bound_16(ref, S, K, kind)).all()


@pytest.mark.parametrize("M,N,K", [(128, 256, 64), (256, 512, 256), (100, 272, 1008), (513, 1040, 336),
                                   (64, 2048, 2048 + 16), (2048, 2048, 2048), (1, 16, 16)])
def test_paired_int8_kn(handle, torch_gpu, oracle, rng, M, N, K):
    torch = torch_gpu
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(A, B)
    a, b = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
    y = probe.gemm_i8_i32_paired(handle, a, b)
    assert "i8_mfma_128x256x64_w4x2_ring3_kn" == handle.last_kernel
    np.testing.assert_array_equal(y.cpu().numpy(), acc_ref)
    for out_type, ot in (("f32", ci.OUT_F32), ("bf16", ci.OUT_BF16)):
        out, acc = probe.gemm_i8_dequant_paired(handle, a, b, torch.from_numpy(sa).cuda(),
                                                torch.from_numpy(sb).cuda(), ot, dump_acc=True)
        np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
        expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=M > 1, sb_per_col=True)
        got = bits(torch, out) if out_type == "bf16" else out.cpu().numpy()
        np.testing.assert_array_equal(got, expect)


def test_paired_refuses_what_it_does_not_take(handle, torch_gpu):
    torch = torch_gpu
    a = torch.ones((64, 60), dtype=torch.bfloat16, device="cuda")      # K * 2 not a multiple of 16
    b = torch.ones((60, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ci.CigemmError, match="NOT_SUPPORTED"):
        probe.gemm16_paired(handle, a, b)
    a8 = torch.ones((64, 72), dtype=torch.int8, device="cuda")         # K not a multiple of 16
    b8 = torch.ones((72, 64), dtype=torch.int8, device="cuda")
    with pytest.raises(ci.CigemmError, match="NOT_SUPPORTED"):
        probe.gemm_i8_i32_paired(handle, a8, b8)

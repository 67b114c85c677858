"""Parity of the hand-written gfx950 kernels against the CPU oracle, through the
C ABI (ctypes -> liborion_kernels.so).  Triad: bit-exact.  GEMM: fp32 output
within 1e-3 of the exact result's RMS (the tolerance the job description names
for floating point); bf16 output equal to the nearest-even rounding of the fp32
output."""

import numpy as np
import pytest
import torch

from oracle import kernels_oracle as ko
from orion_amd import kernels

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GEMM_RTOL = 1e-3


def _uniform(n, seed):
    return (np.random.default_rng(seed).random(n, dtype=np.float32) * 2 - 1)


@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 255, 1023, 4096, 65537, (1 << 22) + 3])
def test_triad_bit_exact(n):
    b, c = _uniform(n, 1), _uniform(n, 2)
    s = 1.7
    a = torch.full((n,), 7.0, device=DEV)
    kernels.triad(a, torch.from_numpy(b).to(DEV), torch.from_numpy(c).to(DEV), s)
    torch.cuda.synchronize()
    assert np.array_equal(a.cpu().numpy().view(np.uint32), ko.triad(b, c, s).view(np.uint32))


@pytest.mark.parametrize("grid", [1, 7, 256, 4096])
def test_triad_any_grid_gives_the_same_bits(grid):
    n = 1_000_003
    b, c = _uniform(n, 3), _uniform(n, 4)
    a = torch.empty(n, device=DEV)
    kernels.triad(a, torch.from_numpy(b).to(DEV), torch.from_numpy(c).to(DEV), -0.3,
                  grid_blocks=grid)
    torch.cuda.synchronize()
    assert np.array_equal(a.cpu().numpy(), ko.triad(b, c, -0.3))


def test_triad_special_values_and_in_place():
    b = np.array([0.0, -0.0, np.inf, 1.0, np.nan, 1e38, -1e38, 1e-45], dtype=np.float32)
    c = np.array([0.0, 0.0, 1.0, np.inf, 1.0, 1e38, 1e38, 1e-45], dtype=np.float32)
    tb, tc = torch.from_numpy(b).to(DEV), torch.from_numpy(c).to(DEV)
    kernels.triad(tb, tb, tc, 2.0)              # a aliases b
    torch.cuda.synchronize()
    want = ko.triad(b, c, 2.0)
    assert np.array_equal(tb.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_triad_full_size_linearity():
    # 1 GiB arrays (the benchmark's size): triad(b, c, s) with c = 0 is the
    # identity on b, bit for bit, and with b = 0, s = 1 the identity on c.
    n = 1 << 28
    b = torch.rand(n, device=DEV) * 2 - 1
    z = torch.zeros(n, device=DEV)
    a = torch.empty(n, device=DEV)
    kernels.triad(a, b, z, 3.0)
    assert torch.equal(a, b)
    kernels.triad(a, z, b, 1.0)
    assert torch.equal(a, b)
    # and a sampled window against the oracle
    kernels.triad(a, b, b, 0.5)
    torch.cuda.synchronize()
    lo = n - 100_003
    hb = b[lo:].cpu().numpy()
    assert np.array_equal(a[lo:].cpu().numpy(), ko.triad(hb, hb, 0.5))


def test_triad_rejects_misaligned_and_mismatched():
    b = torch.zeros(64, device=DEV)
    with pytest.raises(kernels.KernelError) as e:
        kernels.triad(b[1:], b[1:], b[1:], 1.0)
    assert e.value.code == 3
    with pytest.raises(ValueError):
        kernels.triad(b, b[:8], b, 1.0)
    with pytest.raises(ValueError):
        kernels.triad(b.cpu(), b.cpu(), b.cpu(), 1.0)


def _gemm_case(m, n, k, seed):
    rng = np.random.default_rng(seed)
    a = ko.f32_to_bf16_bits(rng.random((m, k), dtype=np.float32) * 2 - 1)
    b = ko.f32_to_bf16_bits(rng.random((n, k), dtype=np.float32) * 2 - 1)
    ta = torch.from_numpy(a.view(np.int16)).view(torch.bfloat16).to(DEV)
    tb = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).to(DEV)
    return a, b, ta, tb


@pytest.mark.parametrize("shape", [(256, 256, 64), (256, 256, 128), (256, 256, 192), (256, 512, 256), (512, 256, 1024),
                                   (768, 1024, 512), (1024, 1024, 2048)])
def test_gemm_against_exact_product(shape):
    m, n, k = shape
    a, b, ta, tb = _gemm_case(m, n, k, sum(shape))
    ref = ko.gemm_bf16_nt(a, b)
    out = kernels.gemm_bf16_nt(ta, tb, out_dtype=torch.float32)
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    rms = np.sqrt(np.mean(ref ** 2))
    assert np.max(np.abs(got - ref)) <= GEMM_RTOL * rms
    out16 = kernels.gemm_bf16_nt(ta, tb)
    torch.cuda.synchronize()
    bits = out16.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(bits, ko.f32_to_bf16_bits(out.cpu().numpy()))


def test_gemm_exact_on_small_integers():
    # integer inputs: every partial sum is exact in fp32, so the result is exact
    rng = np.random.default_rng(5)
    a = rng.integers(-4, 5, (256, 256)).astype(np.float32)
    b = rng.integers(-4, 5, (512, 256)).astype(np.float32)
    ta = torch.from_numpy(a).to(torch.bfloat16).to(DEV)
    tb = torch.from_numpy(b).to(torch.bfloat16).to(DEV)
    out = kernels.gemm_bf16_nt(ta, tb, out_dtype=torch.float32)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), a @ b.T)


def test_gemm_full_size_sampled_rows_and_identity():
    m = n = k = 8192
    g = torch.Generator(device=DEV).manual_seed(11)
    ta = (torch.rand(m, k, device=DEV, generator=g) * 2 - 1).to(torch.bfloat16)
    tb = (torch.rand(n, k, device=DEV, generator=g) * 2 - 1).to(torch.bfloat16)
    out = kernels.gemm_bf16_nt(ta, tb, out_dtype=torch.float32)
    torch.cuda.synchronize()
    rows = [0, 1, 255, 256, 4097, 8191]
    a_bits = ta[rows].view(torch.int16).cpu().numpy().view(np.uint16)
    b_bits = tb.view(torch.int16).cpu().numpy().view(np.uint16)
    ref = ko.gemm_bf16_nt(a_bits, b_bits)
    got = out[rows].cpu().numpy().astype(np.float64)
    assert np.max(np.abs(got - ref)) <= GEMM_RTOL * np.sqrt(np.mean(ref ** 2))
    # size-independent property: B = identity returns A (in fp32) exactly
    eye = torch.eye(k, device=DEV, dtype=torch.bfloat16)
    out = kernels.gemm_bf16_nt(ta, eye, out_dtype=torch.float32)
    assert torch.equal(out, ta.float())


def test_gemm_rejects_bad_shapes_without_launching():
    for k in (80, 96):                                # K not a multiple of 64
        a = torch.zeros(256, k, device=DEV, dtype=torch.bfloat16)
        b = torch.zeros(256, k, device=DEV, dtype=torch.bfloat16)
        with pytest.raises(kernels.KernelError) as e:
            kernels.gemm_bf16_nt(a, b)
        assert e.value.code == 2
    a = torch.zeros(100, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(kernels.KernelError) as e:
        kernels.gemm_bf16_nt(a, torch.zeros(256, 64, device=DEV, dtype=torch.bfloat16))
    assert e.value.code == 2
    with pytest.raises(ValueError):
        kernels.gemm_bf16_nt(torch.zeros(256, 64, device=DEV), b)

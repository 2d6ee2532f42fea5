"""GPU parity of the 256x128-tile MXFP4 kernel with three stage buffers (a few hundred rows against many weight
rows) against the oracle and, bit for bit, against the 256x256-tile kernel, which adds up K in the same order."""
import numpy as np
import pytest
import torch

from avelang_amd import _lib, gemm_mxfp4_transposed_b
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
TILE, DECODE, NARROW = 2, 3, 4

# K = 512 .. 3072: 2, 4, 6, 8, 10 and 12 stages walk every path through the ring (prologue only, tail only, one and
# more trips of the main loop); ragged M and N, more than one row of tiles, a single column
CASES = [(256, 128, 512), (100, 300, 1024), (65, 8, 1536), (130, 1000, 2048), (256, 264, 2560), (300, 520, 3072),
         (1, 136, 512), (200, 4096, 1024)]


@pytest.mark.parametrize("m,n,k", CASES)
def test_narrow_matches_oracle_and_the_wide_tile_kernel(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=0, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=1, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=NARROW)
    H.assert_mx_close(c, a, a_s, b, b_s)
    assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s, variant=TILE))


def test_narrow_unit_scales_integer_exact(gpu):
    rng = np.random.default_rng(4)
    m, n, k = 192, 392, 2048
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127, dtype=np.uint8)
    b_s = np.full((n, k // 32), 127, dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=NARROW)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s)))


def test_narrow_random_scales_every_kblock(gpu):
    """Scale bytes differ per row and per 32-block: a wrong pair buffer, byte select or row permutation cannot pass."""
    rng = np.random.default_rng(5)
    m, n, k = 256, 256, 3584
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(117, 138, size=(m, k // 32), dtype=np.uint8)
    b_s = rng.integers(117, 138, size=(n, k // 32), dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=NARROW)
    H.assert_mx_close(c, a, a_s, b, b_s)


def test_dispatch_takes_the_narrow_kernel_for_a_few_hundred_rows(gpu):
    """65..256 rows against many weight rows go to the narrow kernel by themselves: same bits as forcing it."""
    m, n, k = 128, 2048, 1024
    a, a_s = H.mx_operand(m, k, seed=2)
    b, b_s = H.mx_operand(n, k, seed=3, std=0.02)
    auto = H.run_mx(gpu, a, a_s, b, b_s)
    assert np.array_equal(auto, H.run_mx(gpu, a, a_s, b, b_s, variant=NARROW))
    H.assert_mx_close(auto, a, a_s, b, b_s)
    lib = _lib.load()
    one = torch.zeros(64, dtype=torch.uint8, device=gpu)
    rc = lib.ave_fp4_gemm_mxfp4_ex(one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(),
                                   4, 4, 256, None, NARROW)
    assert rc == -1 and "narrow-tile kernel does not support" in _lib.last_error()


@pytest.mark.parametrize("m,n", [(40, 28672), (64, 32768), (33, 30000)])
def test_dispatch_takes_the_narrow_kernel_for_33_to_64_rows_against_a_full_round_of_tiles(gpu, m, n):
    """33..64 rows against 28 672 and more weight rows (a nearly full round of 128-row tiles on 256 compute units) run on
    the narrow-tile kernel by dispatch; fewer weight rows, and up to 32 rows, stay on the weight-streaming kernel."""
    k = 512
    a, a_s = H.mx_operand(m, k, seed=4)
    b, b_s = H.mx_operand(n, k, seed=5, std=0.02)
    auto = H.run_mx(gpu, a, a_s, b, b_s)
    H.assert_mx_close(auto, a, a_s, b, b_s)
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    tiles = -(-n // 128)
    if tiles <= cus and 8 * tiles >= 7 * cus:
        assert np.array_equal(auto, H.run_mx(gpu, a, a_s, b, b_s, variant=NARROW))
    few = 20480
    assert np.array_equal(H.run_mx(gpu, a, a_s, b[:few], b_s[:few]), H.run_mx(gpu, a, a_s, b[:few], b_s[:few], variant=DECODE))
    assert np.array_equal(H.run_mx(gpu, a[:32], a_s[:32], b, b_s), H.run_mx(gpu, a[:32], a_s[:32], b, b_s, variant=DECODE))


def test_dispatch_takes_the_narrow_kernel_for_the_fused_swiglu_at_33_to_64_rows(gpu):
    from avelang_amd import gemm_mxfp4_swiglu_transposed_b as swiglu

    m, n, k = 48, 14336, 512   # 224 tiles of 64 outputs: a nearly full round on 256 compute units
    a, a_s = H.mx_operand(m, k, seed=6)
    b, b_s = H.mx_operand(2 * n, k, seed=7, std=0.02)
    d = [H.to_dev(v, gpu) for v in (a, a_s, b, b_s)]
    auto = swiglu(*d)
    torch.cuda.synchronize()
    ok, rep = orc.check_swiglu_bf16(H.bits(auto), a, a_s, b, b_s)
    assert ok, rep
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    tiles = -(-n // 64)
    want = NARROW if tiles <= cus and 8 * tiles >= 7 * cus else DECODE
    assert torch.equal(auto, swiglu(*d, variant=want))
    assert torch.equal(swiglu(d[0][:32].clone(), d[1][:32].clone(), d[2], d[3]), swiglu(d[0][:32].clone(), d[1][:32].clone(), d[2], d[3], variant=DECODE))


# ---- the SwiGLU-fused form: 256 x 64-output tiles ----------------------------------------------------------------------
from avelang_amd import gemm_mxfp4_swiglu_transposed_b  # noqa: E402


def _swiglu(gpu, a, a_s, b, b_s, variant):
    c = gemm_mxfp4_swiglu_transposed_b(H.to_dev(a, gpu), H.to_dev(a_s, gpu), H.to_dev(b, gpu), H.to_dev(b_s, gpu),
                                       variant=variant)
    torch.cuda.synchronize()
    return H.bits(c)


@pytest.mark.parametrize("m,n,k", [(256, 64, 512), (100, 200, 1024), (65, 8, 1536), (130, 131, 2048), (256, 520, 2560),
                                   (300, 392, 3072), (128, 1792, 1024)])
def test_narrow_swiglu_matches_exact_arithmetic_and_the_wide_tile_kernel(gpu, m, n, k):
    """Ragged rows and columns, N % 8 != 0 (scalar stores), two rows of tiles; the fp32 sums and the activation
    are those of the 256 x 256 kernel's fused form, so the two must agree bit for bit."""
    a, a_s = H.mx_operand(m, k, seed=m + n)
    b, b_s = H.mx_operand(2 * n, k, seed=m + n + 1, std=0.05)
    c = _swiglu(gpu, a, a_s, b, b_s, NARROW)
    ok, rep = orc.check_swiglu_bf16(c, a, a_s, b, b_s)
    assert ok, rep
    assert np.array_equal(c, _swiglu(gpu, a, a_s, b, b_s, TILE))


def test_narrow_swiglu_is_what_dispatch_takes_for_a_few_hundred_rows(gpu):
    m, n, k = 128, 1024, 1024
    a, a_s = H.mx_operand(m, k, seed=8)
    b, b_s = H.mx_operand(2 * n, k, seed=9, std=0.05)
    auto = _swiglu(gpu, a, a_s, b, b_s, 0)
    assert np.array_equal(auto, _swiglu(gpu, a, a_s, b, b_s, NARROW))
    ok, rep = orc.check_swiglu_bf16(auto, a, a_s, b, b_s)
    assert ok, rep
    with pytest.raises(ValueError, match="narrow-tile kernel does not support"):
        gemm_mxfp4_swiglu_transposed_b(H.to_dev(a[:, :128], gpu), H.to_dev(a_s[:, :8], gpu), H.to_dev(b[:, :128], gpu),
                                       H.to_dev(b_s[:, :8], gpu), variant=NARROW)     # K = 256


# ---- the grouped form: expert layers at decode batch sizes ----------------------------------------------------------

@pytest.mark.parametrize("n,k,offsets", [(520, 1024, [0, 30, 30, 95, 130, 400]),        # an empty expert, one with 270 rows
                                         (128, 2560, [0, 1, 17, 17, 64, 100, 101, 140, 200]),
                                         (264, 512, [0, 256, 512, 600])])
def test_grouped_narrow_equals_per_expert_calls(gpu, n, k, offsets):
    """Every expert's rows equal the plain call on that expert bit for bit, through shape-based dispatch (at most 128
    rows per expert on average) and with the kernel forced; one expert is checked against the oracle."""
    e, total = len(offsets) - 1, offsets[-1]
    a, a_s = H.mx_operand(total, k, seed=80)
    bw = [H.mx_operand(n, k, seed=90 + i, std=0.02) for i in range(e)]
    b, b_s = np.stack([w[0] for w in bw]), np.stack([w[1] for w in bw])
    forced = H.run_grouped(gpu, a, a_s, b, b_s, offsets, variant=NARROW)
    if total <= 128 * e:
        assert np.array_equal(H.run_grouped(gpu, a, a_s, b, b_s, offsets), forced)
    assert np.array_equal(H.run_grouped(gpu, a, a_s, b, b_s, offsets, variant=TILE), forced)
    for i in range(e):
        r0, r1 = offsets[i], offsets[i + 1]
        if r1 > r0:
            plain = H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[i], b_s[i], variant=TILE)
            assert np.array_equal(plain, forced[r0:r1]), i
    r0, r1 = offsets[-2], offsets[-1]
    H.assert_mx_close(forced[r0:r1], a[r0:r1], a_s[r0:r1], b[e - 1], b_s[e - 1])


# ---- K with a tail behind the last multiple of 512: the tail comes straight from global memory --------------------------

@pytest.mark.parametrize("m,n,k", [(256, 128, 544), (100, 300, 1504), (65, 8, 992), (130, 1000, 2880), (300, 520, 3104),
                                   (1, 136, 736), (200, 4096, 1056), (128, 264, 4128)])
def test_narrow_k_tail_matches_oracle(gpu, m, n, k):
    """1, 15, 10 and other numbers of tail blocks on the 256-row and the 128-row form (the order of addition differs from
    the 256 x 256 kernel's staged tail, so that kernel is no bit-for-bit reference here)."""
    a, a_s = H.mx_operand(m, k, seed=0, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=1, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=NARROW)
    H.assert_mx_close(c, a, a_s, b, b_s)


def test_narrow_k_tail_unit_scales_integer_exact(gpu):
    rng = np.random.default_rng(14)
    m, n, k = 200, 300, 992
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127, dtype=np.uint8)
    b_s = np.full((n, k // 32), 127, dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=NARROW)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s)))


@pytest.mark.parametrize("m,n,k", [(256, 64, 544), (100, 200, 1504), (130, 131, 2880), (128, 1792, 1056)])
def test_narrow_swiglu_k_tail(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=m + n)
    b, b_s = H.mx_operand(2 * n, k, seed=m + n + 1, std=0.05)
    c = _swiglu(gpu, a, a_s, b, b_s, NARROW)
    ok, rep = orc.check_swiglu_bf16(c, a, a_s, b, b_s)
    assert ok, rep


@pytest.mark.parametrize("n,k,offsets", [(520, 1504, [0, 30, 30, 95, 130, 400]), (128, 2880, [0, 1, 17, 17, 64, 100, 101, 140, 200])])
def test_grouped_narrow_k_tail_equals_per_expert_calls(gpu, n, k, offsets):
    e, total = len(offsets) - 1, offsets[-1]
    a, a_s = H.mx_operand(total, k, seed=80)
    bw = [H.mx_operand(n, k, seed=90 + i, std=0.02) for i in range(e)]
    b, b_s = np.stack([w[0] for w in bw]), np.stack([w[1] for w in bw])
    forced = H.run_grouped(gpu, a, a_s, b, b_s, offsets, variant=NARROW)
    if total <= 128 * e:
        assert np.array_equal(H.run_grouped(gpu, a, a_s, b, b_s, offsets), forced)   # what dispatch takes
    for i in range(e):
        r0, r1 = offsets[i], offsets[i + 1]
        if r1 > r0:
            H.assert_mx_close(forced[r0:r1], a[r0:r1], a_s[r0:r1], b[i], b_s[i])
            if r1 - r0 <= 128:   # the plain call on at most 128 rows runs the same 128-row form
                assert np.array_equal(H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[i], b_s[i], variant=NARROW), forced[r0:r1]), i

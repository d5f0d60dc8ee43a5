"""GPU parity: the HIP path through the C ABI against the golden fixtures (outputs of the reference's own
portable code) and against the CPU oracle on seeded inputs. Integer outputs must be bit-exact."""
import zlib

import numpy as np
import pytest

import oracle
from computelibrary_amd import capi
from gpu_util import announce, run_gemm, to_dev

pytestmark = pytest.mark.gpu

PATHS = [capi.PATH_SIMPLE, capi.PATH_MFMA, capi.PATH_SKINNY]


def paths_for(M, batch=1):
    return [p for p in PATHS if p != capi.PATH_SKINNY or M <= 64]


def test_device_is_gfx950():
    name, cus = capi.device_info()
    assert name.startswith("gfx950"), name
    assert cus >= 200


@pytest.mark.parametrize("device", [False, True])
def test_s32_fixture(golden, device):
    g = golden("gemmlowp_s32.npz")
    for n in range(int(g["count"])):
        A, B = g["a%d" % n], g["b%d" % n]
        ao, bo = (int(x) for x in g["off%d" % n])
        for path in paths_for(A.shape[0]):
            announce("s32 fixture", n, A.shape, B.shape, A.dtype, B.dtype, ao, bo, "path", path, "device", device)
            got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=path, device=device)
            np.testing.assert_array_equal(got, g["dst%d" % n])


def test_s32_batched_fixture(golden):
    g = golden("gemmlowp_batched.npz")
    for n in range(int(g["count"])):
        A, B = g["a%d" % n], g["b%d" % n]
        ao, bo = (int(x) for x in g["off%d" % n])
        for path in paths_for(A.shape[1], A.shape[0]):
            announce("batched fixture", n, A.shape, B.shape, "path", path)
            got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=path, device=True)
            np.testing.assert_array_equal(got, g["dst%d" % n])


@pytest.mark.parametrize("device", [False, True])
def test_fused_fixedpoint_fixture(golden, device):
    g = golden("gemmlowp_fused_fixedpoint.npz")
    for n in range(int(g["count"])):
        ao, bo, roff, lo, hi, pc = (int(x) for x in g["p%d" % n])
        A, B, dst = g["a%d" % n], g["b%d" % n], g["dst%d" % n]
        for path in paths_for(A.shape[0]):
            announce("fused fixture", n, A.shape, B.shape, dst.dtype, "pc", pc, "path", path, "device", device)
            got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, dst.dtype, ao, bo, g["bias%d" % n], g["mult%d" % n],
                              g["shift%d" % n], roff, lo, hi, path=path, device=device)
            np.testing.assert_array_equal(got, dst)


def test_f32_fixture(golden):
    g = golden("gemmlowp_f32.npz")
    scale = float(g["scale"])
    for n in range(int(g["count"])):
        A, B = g["a%d" % n], g["b%d" % n]
        ao, bo = (int(x) for x in g["off%d" % n])
        want_ref = g["dst%d" % n]
        want_orc = oracle.gemmlowp_f32(A, B, None, ao, bo, scale)
        for path in paths_for(A.shape[0]):
            announce("f32 fixture", n, A.shape, B.shape, ao, bo, "path", path)
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=scale, path=path, device=True)
            # same float operations in the same order as the oracle: identical bits
            np.testing.assert_array_equal(got, want_orc)
            # and within the stated 1e-5 relative error of the reference's own test oracle
            tol = 1e-5 * np.maximum(np.abs(want_ref), np.abs(A.astype(np.float64) @ B.astype(np.float64)) * scale)
            assert (np.abs(got - want_ref) <= tol + 1e-30).all()


@pytest.mark.parametrize("a_dt,b_dt", [(np.uint8, np.uint8), (np.int8, np.int8), (np.uint8, np.int8),
                                        (np.int8, np.uint8)])
def test_seeded_against_oracle_all_sign_combinations(a_dt, b_dt):
    rng = np.random.default_rng(41)
    for (M, N, K) in [(300, 200, 520), (129, 257, 1000), (64, 64, 64), (5, 1000, 333)]:
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(np.iinfo(b_dt).min, np.iinfo(b_dt).max + 1, size=(K, N)).astype(b_dt)
        ao, bo = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
        want = oracle.gemmlowp_s32(A, B, ao, bo)
        bias = rng.integers(-5000, 5000, size=N, dtype=np.int32)
        mult, shift = oracle.calculate_quantized_multiplier(float(rng.uniform(0.0005, 0.01)))
        want_q = oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo, [mult], [shift], 3, 0, 255, np.uint8)
        for path in paths_for(M):
            announce("seeded", a_dt.__name__, b_dt.__name__, (M, N, K), ao, bo, "path", path)
            got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=path, device=True)
            np.testing.assert_array_equal(got, want)
            got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.uint8, ao, bo, bias, [mult], [shift], 3, 0, 255,
                              path=path, device=True)
            np.testing.assert_array_equal(got, want_q)


def test_random_shape_sweep_against_oracle():
    """60 seeded cases over ragged shapes, every epilogue, both operand signs, aligned and unaligned row strides, and
    K around the pipelined kernel's ring depth (1 to 6 steps of 128, with and without a tail)"""
    rng = np.random.default_rng(2024)
    for case in range(60):
        M = int(rng.choice([1, 3, 8, 16, 17, 63, 64, 65, 127, 129, 255, 257, 300]))
        N = int(rng.choice([1, 4, 15, 16, 33, 64, 100, 128, 129, 255, 256, 260]))
        K = int(rng.choice([16, 32, 100, 127, 128, 129, 240, 256, 272, 384, 400, 512, 640, 700, 768]))
        a_dt = np.int8 if rng.integers(2) else np.uint8
        b_dt = np.int8 if (a_dt == np.int8 or rng.integers(2)) else np.uint8
        lda = K + int(rng.choice([0, 0, 16, 4, 3]))
        ldd = N + int(rng.choice([0, 0, 16, 4, 1]))
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(-20, 20))
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(np.iinfo(b_dt).min, np.iinfo(b_dt).max + 1, size=(K, N)).astype(b_dt)
        epi = int(rng.integers(3))
        device = bool(rng.integers(2))
        path = capi.PATH_AUTO if rng.integers(4) else capi.PATH_MFMA
        announce("sweep", case, (M, N, K), a_dt.__name__, b_dt.__name__, "lda", lda, "ldd", ldd, "epi", epi, "dev", device,
                 "path", path)
        if epi == 0:
            got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=path, device=device, lda=lda, ldd=ldd)
            want = oracle.gemmlowp_s32(A, B, ao, bo)
        elif epi == 1:
            per_channel = bool(rng.integers(2)) and b_dt == np.int8
            bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
            reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N if per_channel else 1)) * 128.0 / np.sqrt(K)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            dt = a_dt
            lo, hi = (-128, 127) if dt == np.int8 else (0, 255)
            off = -7 if dt == np.int8 else 121
            bo_eff = 0 if per_channel else bo
            got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, dt, ao, bo_eff, bias, mult, shift, off, lo, hi, path=path,
                              device=device, lda=lda, ldd=ldd)
            want = oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo_eff, mult, shift, off, lo, hi, dt)
        else:
            if a_dt != np.int8 or b_dt != np.int8:
                A, B = A.view(np.int8), B.view(np.int8)
            bias = rng.normal(0.0, 1.0, size=N).astype(np.float32) if rng.integers(2) else None
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, bias_f32=bias, path=path, device=device,
                              lda=lda, ldd=ldd)
            want = oracle.gemmlowp_f32(A, B, bias, ao, bo, 3e-4)
            got, want = got.view(np.uint32), want.view(np.uint32)
        assert np.array_equal(got, want), "case %d" % case


@pytest.mark.parametrize("device", [True, False])
def test_f16_destination(device):
    """GEMMLowp dequantised into halfs (tests/validation/NEON/GEMMLowp.cpp:598-621: signed operands, with and without
    accumulation; the reference accepts 0.2 relative error there). Here: the bits of the oracle - the float result
    rounded to nearest even, added to the previous halfs the way the reference's test oracle adds halfs - on every
    kernel path, with padded destination rows, a float bias and an activation clamp after the accumulation."""
    rng = np.random.default_rng(1600)
    scale = (1.0 / 255) * (5.0 / 255)
    for (M, N, K) in [(21, 13, 33), (8, 300, 200), (150, 70, 520), (40, 4100, 128)]:
        A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
        B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(-20, 20))
        prev = rng.normal(0, 3, size=(M, N)).astype(np.float16)
        biasf = rng.normal(0.0, 1.0, size=N).astype(np.float32)
        for path in paths_for(M):
            announce("f16 destination", (M, N, K), ao, bo, "path", path, "device", device)
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float16, ao, bo, scale=scale, path=path, device=device, ldd=N + 3)
            np.testing.assert_array_equal(got.view(np.uint16), oracle.gemmlowp_f16(A, B, None, ao, bo, scale).view(np.uint16))
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float16, ao, bo, scale=scale, path=path, device=device, prev=prev,
                              flags=capi.GEMM_ACCUMULATE)
            np.testing.assert_array_equal(got.view(np.uint16),
                                          oracle.gemmlowp_f16(A, B, None, ao, bo, scale, prev=prev).view(np.uint16))
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float16, ao, bo, scale=scale, bias_f32=biasf, act=(0.0, 6.0), path=path,
                              device=device, prev=prev, flags=capi.GEMM_ACCUMULATE)
            want = oracle.gemmlowp_f16(A, B, biasf, ao, bo, scale, 0.0, 6.0, prev=prev)
            np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
            assert 0.05 < (want == 0).mean() < 0.95 or M * N < 400


def test_batched_small_products_take_the_streaming_kernel():
    """Batches of small products (tests/datasets/GEMMLowpFusedOffsetOutputDataset.h:142-162: up to 32 entries of a few
    rows) run the streaming kernel instead of a mostly empty tile per entry - one launch with the entries along the grid
    (and one more for the row sums of all entries), or, from 4 MiB of B per entry on, one launch per entry in the form
    that stages A once: per-entry and shared B, a B offset (row sums per entry), padded rows and batch strides, every
    epilogue."""
    rng = np.random.default_rng(4242)
    for (batch, M, N, K, b_batched) in [(3, 4, 5, 2, True), (3, 7, 29, 15, True), (32, 17, 5, 56, True), (32, 13, 19, 256, True),
                                        (5, 8, 300, 1024, False), (4, 32, 130, 200, True), (3, 8, 64, 2048, True),
                                        (2, 8, 1100, 4096, False)]:
        A = rng.integers(-128, 128, size=(batch, M, K), dtype=np.int8)
        B = rng.integers(-128, 128, size=(batch, K, N) if b_batched else (K, N), dtype=np.int8)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(1, 20))
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        mult, shift = oracle.calculate_quantized_multiplier(float(40.0 / (max(K, 4) ** 0.5 * 74.0 * 74.0)))
        announce("batched small", (batch, M, N, K), "b_batched", b_batched)
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, device=True, lda=K + 4 - K % 4, ldd=N + 1)
        assert name.startswith("skinny"), name
        for z in range(batch):
            np.testing.assert_array_equal(got[z], oracle.gemmlowp_s32(A[z], B[z] if b_batched else B, ao, bo))
        got, name = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, ao, bo, bias, [mult], [shift], -3, -128, 127, device=True)
        assert name == ("skinny_once" if N * K > (4 << 20) else "skinny_stream"), name
        for z in range(batch):
            np.testing.assert_array_equal(
                got[z], oracle.gemmlowp_fixedpoint(A[z], B[z] if b_batched else B, bias, ao, bo, [mult], [shift], -3, -128, 127, np.int8))
        for device in (False, True):
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, device=device)
            for z in range(batch):
                np.testing.assert_array_equal(got[z].view(np.uint32),
                                              oracle.gemmlowp_f32(A[z], B[z] if b_batched else B, None, ao, bo, 3e-4).view(np.uint32))


def test_f16_fixture(golden):
    """Halfs produced by the reference's own code (tests/golden/gemmlowp_f16.npz): with zero offsets the device result
    has the same bits, with and without accumulation into previous halfs."""
    g = golden("gemmlowp_f16.npz")
    scale = float(g["scale"])
    for n in range(int(g["count"])):
        A, B, prev = g["a%d" % n], g["b%d" % n], g["prev%d" % n]
        ao, bo = (int(x) for x in g["off%d" % n])
        if ao or bo:
            continue
        for path in paths_for(A.shape[0]):
            announce("f16 fixture", n, A.shape, B.shape, "path", path)
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float16, 0, 0, scale=scale, path=path, device=True)
            np.testing.assert_array_equal(got.view(np.uint16), g["dst%d" % n])
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float16, 0, 0, scale=scale, path=path, device=True, prev=prev,
                              flags=capi.GEMM_ACCUMULATE)
            np.testing.assert_array_equal(got.view(np.uint16), g["acc%d" % n])


PIPELINED_CONFIGS = ["pp_256x128x128_s3", "pp_128x128x128_s3", "pp_128x64x128_s3", "pp_64x64x128_s3", "pp_64x64x128_s6",
                     "pp_128x64x256_s3"]


@pytest.mark.parametrize("cfg", range(len(PIPELINED_CONFIGS)))
def test_every_pipelined_configuration(cfg):
    """Each tile / ring-depth configuration of the pipelined kernel, asked for by name (MI355_PATH_TILE + n), on K of
    one to nine steps with and without a tail (the 256-byte-step configuration needs a packed K that is a multiple of
    256 and is otherwise replaced by the automatic choice)."""
    tile = capi.PATH_TILE + cfg
    rng = np.random.default_rng(70 + cfg)
    for (M, N, K) in [(300, 200, 512), (70, 129, 100), (257, 64, 1100), (129, 300, 250), (64, 65, 2048)]:
        A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
        B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(-20, 20))
        announce("pipelined config", cfg, (M, N, K))
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=tile, device=True)
        kp = -(-K // 128) * 128
        if cfg != 5 or kp % 256 == 0:
            assert name.split("_splitk")[0] == PIPELINED_CONFIGS[cfg], name  # (K = 2048 under one tile runs as two K slices)
        np.testing.assert_array_equal(got, oracle.gemmlowp_s32(A, B, ao, bo))
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N)) * 128.0 / np.sqrt(K)
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, ao, 0, bias, mult, shift, -7, -128, 127, path=tile,
                          device=True)
        np.testing.assert_array_equal(got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, 0, mult, shift, -7, -128, 127, np.int8))
        got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, path=tile, device=True)
        np.testing.assert_array_equal(got.view(np.uint32), oracle.gemmlowp_f32(A, B, None, ao, bo, 3e-4).view(np.uint32))


@pytest.mark.parametrize("K,lda", [(1000, 1000), (1096, 1120), (130, 136), (1104, 1104)])
def test_k_tail_of_tiles_inside_the_matrix_on_the_256x128_tile(K, lda):
    """A K that ends inside the last K step, on the 4 + 4 wave form: row tiles inside the matrix fetch that step whole -
    the columns at and beyond K hold the next row's (or the next batch entry's) bytes and meet zero rows of B - except the
    last row tile of the last batch entry, whose reads may not pass the end of A; a ragged last row tile takes the
    general loader either way. One product and a batch of 3 (shared and per-entry B), rows that end where the next
    begins and rows with a gap, signed and unsigned A, a B offset (row sums from a pass of their own, or inside the
    kernel when K is a multiple of 16 - then the step is not fetched whole), all three epilogues."""
    rng = np.random.default_rng(zlib.crc32(repr((K, lda)).encode()))
    tile = capi.PATH_TILE + 0
    N = 200
    for (batch, M, a_dt, bo) in [(1, 768, np.int8, 0), (1, 700, np.uint8, -9), (3, 512, np.int8, 0), (3, 256, np.uint8, 4)]:
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(batch, M, K)).astype(a_dt)
        for b_batched in ((False, True) if batch > 1 else (False,)):
            B = rng.integers(-128, 128, size=((batch, K, N) if b_batched else (K, N)), dtype=np.int8)
            ao = int(rng.integers(-20, 20))
            Aa = A if batch > 1 else A[0]
            B3 = B if b_batched else np.broadcast_to(B, (batch, K, N))
            announce("k tail, 256x128 tile", (batch, M, N, K), "lda", lda, a_dt.__name__, "b_offset", bo, "b batched", b_batched)
            got, name = run_gemm(Aa, B, capi.EPI_S32, np.int32, ao, bo, path=tile, device=True, lda=lda)
            assert name == "pp_256x128x128_s3", name
            want = np.stack([oracle.gemmlowp_s32(A[z], B3[z], ao, bo) for z in range(batch)])
            np.testing.assert_array_equal(got if batch > 1 else got[None], want)
            bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
            reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N)) * 128.0 / np.sqrt(K)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            got, _ = run_gemm(Aa, B, capi.EPI_FIXEDPOINT, np.int8, ao, bo, bias, mult, shift, -7, -128, 127, path=tile, device=True, lda=lda)
            want = np.stack([oracle.gemmlowp_fixedpoint(A[z], B3[z], bias, ao, bo, mult, shift, -7, -128, 127, np.int8) for z in range(batch)])
            np.testing.assert_array_equal(got if batch > 1 else got[None], want)
            if a_dt == np.int8:
                got, _ = run_gemm(Aa, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, path=tile, device=True, lda=lda)
                want = np.stack([oracle.gemmlowp_f32(A[z], B3[z], None, ao, bo, 3e-4) for z in range(batch)])
                np.testing.assert_array_equal((got if batch > 1 else got[None]).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("cfg", range(len(PIPELINED_CONFIGS)))
def test_row_sums_taken_inside_the_pipelined_kernels(cfg):
    """A non-zero B offset (or an unsigned B) needs b_offset * rowsum(A): with dword-aligned rows and K a multiple of 16
    the pipelined kernels sum the rows of A themselves from the tiles that pass through them (one launch, no pass over A
    in front). Every tile configuration; K with whole steps and with a last step that is mostly padding (which an
    unsigned A turns into -128s that must not be counted); signed and unsigned A and B; a batch; a row stride with a
    gap; every epilogue."""
    tile = capi.PATH_TILE + cfg
    rng = np.random.default_rng(900 + cfg)
    for (M, N, K, a_dt, b_dt, batch) in [(300, 200, 512, np.int8, np.int8, 1), (257, 140, 400, np.uint8, np.uint8, 1),
                                         (70, 129, 144, np.uint8, np.int8, 3), (520, 260, 1040, np.int8, np.uint8, 2)]:
        shape_a = (batch, M, K) if batch > 1 else (M, K)
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=shape_a).astype(a_dt)
        B = rng.integers(np.iinfo(b_dt).min, np.iinfo(b_dt).max + 1, size=(K, N)).astype(b_dt)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(1, 20))
        lda = K + 16
        announce("row sums in kernel", cfg, (batch, M, N, K), a_dt.__name__, b_dt.__name__, ao, bo)
        As = A if batch > 1 else A[None]
        want = np.stack([oracle.gemmlowp_s32(As[z], B, ao, bo) for z in range(batch)])
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=tile, device=True, lda=lda)
        np.testing.assert_array_equal(got if batch > 1 else got[None], want)
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        mult, shift = oracle.calculate_quantized_multiplier(float(128.0 / np.sqrt(K) * 2e-4))
        lo, hi, off = (-128, 127, -7) if a_dt == np.int8 else (0, 255, 121)
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, bo, bias, [mult], [shift], off, lo, hi, path=tile, device=True,
                          lda=lda)
        wantq = np.stack([oracle.gemmlowp_fixedpoint(As[z], B, bias, ao, bo, [mult], [shift], off, lo, hi, a_dt)
                          for z in range(batch)])
        np.testing.assert_array_equal(got if batch > 1 else got[None], wantq)
        if a_dt == np.int8 and b_dt == np.int8:
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, path=tile, device=True, lda=lda)
            np.testing.assert_array_equal(got.view(np.uint32), oracle.gemmlowp_f32(A, B, None, ao, bo, 3e-4).view(np.uint32))


@pytest.mark.parametrize("M", [1, 5, 8, 9, 12, 16])
def test_skinny_kernel_with_staged_a(M):
    """Up to 8 rows the streaming kernel copies each wave's K slice of A into LDS once, 9 to 16 rows it stages the 512
    bytes per row of every step; both with 4 waves (many column groups) and 8 waves (few), signed and unsigned A,
    K with and without whole steps, row strides that are only dword aligned."""
    rng = np.random.default_rng(300 + M)
    for (N, K, lda) in [(300, 512, 512), (300, 4096, 4096), (8200, 1024, 1024), (8200, 1088, 1092), (520, 640, 656),
                        (100, 200, 200)]:
        a_dt = np.uint8 if (N + K) % 3 == 0 else np.int8
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(-20, 20))
        announce("skinny staged", (M, N, K), "lda", lda, a_dt.__name__)
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=capi.PATH_SKINNY, device=True, lda=lda)
        assert name.startswith("skinny"), name
        np.testing.assert_array_equal(got, oracle.gemmlowp_s32(A, B, ao, bo))
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N)) * 128.0 / np.sqrt(K)
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        lo, hi, off = (-128, 127, -7) if a_dt == np.int8 else (0, 255, 121)
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, 0, bias, mult, shift, off, lo, hi, path=capi.PATH_SKINNY,
                          device=True, lda=lda)
        np.testing.assert_array_equal(got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, 0, mult, shift, off, lo, hi, a_dt))


@pytest.mark.parametrize("M", [1, 3, 8, 9, 13, 16, 17, 25, 32, 33, 50, 64])
def test_skinny_stage_once_kernel(M):
    """Up to 32 rows (three builds: up to 8, where half of the matrix instruction's rows are padding, 9 to 16, and 17 to
    32 as two blocks of rows) and K <= 4096 (whole 64-byte blocks, 16-byte aligned rows): one workgroup of 16 waves per
    compute unit walks several column groups with A staged once: K picks 1, 2 or 4 k blocks per wave, with the last busy wave short
    (K = 2112, 3136) or waves without any k block (K = 64, 640); N covers a single ragged group, fewer groups than compute
    units, between one and two groups per compute unit (N = 4100, 5000: half as many workgroups as groups, one of them
    with three when the count is odd), 2 to 3 groups per workgroup, a sparse last round (N = 9300: fewer workgroups than
    compute units, three groups each), and more than four times the compute units (N = 16400, 70000: several workgroups
    per unit); every epilogue, signed and unsigned A, a non-zero B offset (row vector) and
    accumulation."""
    rng = np.random.default_rng(3300 + M)
    for once in (True,):
        for (N, K) in [(7, 64), (300, 640), (8200, 1024), (11008, 4096), (5000, 2112), (4100, 3136), (70000, 256),
                       (16400, 2048), (9300, 512)]:
            a_dt = np.uint8 if (N + K) % 3 == 0 else np.int8
            A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
            B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
            ao, bo = int(rng.integers(-20, 20)), int(rng.integers(1, 20))
            lda = K + (0 if K % 128 else 16)
            announce("skinny stage-once", once, (M, N, K), "lda", lda, a_dt.__name__)
            want = oracle.gemmlowp_s32(A, B, ao, bo)
            got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=capi.PATH_AUTO, device=True, lda=lda, ldd=N + 3)
            assert name.startswith("skinny"), name
            np.testing.assert_array_equal(got, want)
            prev = rng.integers(-10**6, 10**6, size=(M, N), dtype=np.int32)
            got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, device=True, lda=lda, prev=prev, flags=capi.GEMM_ACCUMULATE)
            np.testing.assert_array_equal(got, (want.astype(np.int64) + prev).astype(np.int32))
            bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
            reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N)) * 128.0 / np.sqrt(K)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            lo, hi, off = (-128, 127, -7) if a_dt == np.int8 else (0, 255, 121)
            got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, 0, bias, mult, shift, off, lo, hi, device=True, lda=lda)
            np.testing.assert_array_equal(got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, 0, mult, shift, off, lo, hi, a_dt))
            got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, bo, bias, [int(mult[0])], [int(shift[0])], off, lo, hi,
                              device=True, lda=lda)
            np.testing.assert_array_equal(
                got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo, [int(mult[0])], [int(shift[0])], off, lo, hi, a_dt))
            if a_dt == np.int8:
                biasf = rng.normal(0.0, 1.0, size=N).astype(np.float32)
                got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, bias_f32=biasf, device=True, lda=lda)
                np.testing.assert_array_equal(got.view(np.uint32),
                                              oracle.gemmlowp_f32(A, B, biasf, ao, bo, 3e-4).view(np.uint32))


def test_streaming_kernels_across_their_grid_rules():
    """The stage-once kernels pick their grid from the number of column groups per compute unit (one workgroup per group,
    half as many workgroups as groups, one per unit, equal shares on fewer units, whole rounds beyond four groups per
    unit) and their build from M and K (1, 2, 4 or 8 k blocks per wave; 8, 16, 32 or 64 rows; the deep-K form). A seeded
    sample of shapes on both sides of every boundary, raw S32 products against a float64 matrix product (exact: the sums
    stay far below 2^53), with one requantised case per shape class elsewhere in this file."""
    _, cus = capi.device_info()
    rng = np.random.default_rng(8800)
    group_counts = [cus - 1, cus, cus + 1, cus + cus // 2 + 1, 2 * cus - 1, 2 * cus, 2 * cus + 1, 2 * cus + cus // 8 - 1,
                    2 * cus + cus // 8, 2 * cus + cus // 2, 2 * cus + cus // 2 + 1, 3 * cus + cus // 4, 4 * cus, 4 * cus + 1, 5 * cus + 3]
    depths = [1024, 2112, 4096, 4160, 5120, 8192, 8256]
    rows = [3, 8, 12, 16, 20, 32, 40, 64]
    cases = [(rows[int(rng.integers(len(rows)))], group_counts[int(rng.integers(len(group_counts)))] * 16 - int(rng.integers(0, 16)),
              depths[int(rng.integers(len(depths)))]) for _ in range(40)]
    cases += [(8, (2 * cus + cus // 8) * 16, 8192), (16, (cus + 1) * 16, 8192), (8, 4 * cus * 16 + 1, 4096), (64, (cus + 3) * 16, 4096)]
    for (M, N, K) in cases:
        A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
        B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        announce("streaming grid rules", (M, N, K), "groups per unit %.2f" % ((N + 15) // 16 / cus))
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, 0, 0, path=capi.PATH_SKINNY, device=True)
        assert name.startswith("skinny"), name
        want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.int64)
        np.testing.assert_array_equal(got.astype(np.int64), want)


def test_pipelined_kernel_with_k_slices():
    """Few output tiles under a deep K: the K range runs as 2 to 8 slices (batch entries of one S32 launch) and a second
    kernel sums the planes and applies the epilogue. Shapes that take slices (how many, the cost model decides with the tile
    shape: 2, 4 or 8), ragged M and N (a plane pitch padded to
    4 columns), both signs of A, offsets on both sides (row and column terms applied once, by the second kernel), every
    epilogue, per-channel and per-tensor constants, accumulation into S32 and F32; a K that no slice count divides stays
    one launch."""
    rng = np.random.default_rng(6600)
    for (M, N, K, slices) in [(100, 512, 4096, 4), (200, 302, 8192, 8), (130, 200, 2560, 2), (70, 1000, 2049 + 63, 1)]:
        a_dt = np.uint8 if K % 3 == 0 else np.int8
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(1, 20))
        announce("k slices", (M, N, K), slices, a_dt.__name__)
        want = oracle.gemmlowp_s32(A, B, ao, bo)
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=capi.PATH_MFMA, device=True, ldd=N + 5)
        assert ("_splitk" in name) == (slices > 1), name
        np.testing.assert_array_equal(got, want)
        prev = rng.integers(-10**6, 10**6, size=(M, N), dtype=np.int32)
        got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=capi.PATH_MFMA, device=True, prev=prev, flags=capi.GEMM_ACCUMULATE)
        np.testing.assert_array_equal(got, (want.astype(np.int64) + prev).astype(np.int32))
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N)) * 128.0 / np.sqrt(K)
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        lo, hi, off = (-128, 127, -7) if a_dt == np.int8 else (0, 255, 121)
        got, name = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, bo, bias, mult, shift, off, lo, hi, path=capi.PATH_MFMA, device=True)
        assert ("_splitk" in name) == (slices > 1), name
        np.testing.assert_array_equal(got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, bo, mult, shift, off, lo, hi, a_dt))
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, 0, bias, [int(mult[0])], [int(shift[0])], off, lo, hi,
                          path=capi.PATH_MFMA, device=True, ldd=N + 16)
        np.testing.assert_array_equal(
            got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, 0, [int(mult[0])], [int(shift[0])], off, lo, hi, a_dt))
        if a_dt == np.int8:
            biasf = rng.normal(0.0, 1.0, size=N).astype(np.float32)
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, bias_f32=biasf, path=capi.PATH_MFMA, device=True)
            np.testing.assert_array_equal(got.view(np.uint32), oracle.gemmlowp_f32(A, B, biasf, ao, bo, 3e-4).view(np.uint32))
            prevf = rng.normal(0.0, 3.0, size=(M, N)).astype(np.float32)
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, bias_f32=biasf, act=(0.0, 6.0), path=capi.PATH_MFMA,
                              device=True, prev=prevf, flags=capi.GEMM_ACCUMULATE)
            np.testing.assert_array_equal(got.view(np.uint32),
                                          oracle.gemmlowp_f32(A, B, biasf, ao, bo, 3e-4, 0.0, 6.0, prev=prevf).view(np.uint32))


@pytest.mark.parametrize("M", [1, 8, 9, 16])
def test_skinny_stage_once_kernel_with_8_k_blocks_per_wave(M):
    """Up to 16 rows and 4096 < K <= 8192: the stage-once kernel with 8 k blocks per wave and one group's worth of B per
    wave, refilled half by half. K = 4160 leaves one wave with a single k block and seven without any, 5120 and 6656 a
    whole number of waves, 8192 all sixteen; N covers one workgroup per group, half as many workgroups as groups, one per
    compute unit with 2 to 3 groups, and equal shares on fewer units; every epilogue, both signs, accumulation."""
    rng = np.random.default_rng(5500 + M)
    for (N, K) in [(300, 4160), (5120, 5120), (8200, 8192), (9300, 6656), (4100, 8192)]:
        a_dt = np.uint8 if (N + K) % 3 == 0 else np.int8
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(1, 20))
        lda = K + (0 if K % 128 else 16)
        announce("skinny 8 k blocks per wave", (M, N, K), "lda", lda, a_dt.__name__)
        want = oracle.gemmlowp_s32(A, B, ao, bo)
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=capi.PATH_AUTO, device=True, lda=lda, ldd=N + 3)
        assert name.startswith("skinny"), name
        np.testing.assert_array_equal(got, want)
        prev = rng.integers(-10**6, 10**6, size=(M, N), dtype=np.int32)
        got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, device=True, lda=lda, prev=prev, flags=capi.GEMM_ACCUMULATE)
        np.testing.assert_array_equal(got, (want.astype(np.int64) + prev).astype(np.int32))
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N)) * 128.0 / np.sqrt(K)
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        lo, hi, off = (-128, 127, -7) if a_dt == np.int8 else (0, 255, 121)
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, 0, bias, mult, shift, off, lo, hi, device=True, lda=lda)
        np.testing.assert_array_equal(got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, 0, mult, shift, off, lo, hi, a_dt))
        if a_dt == np.int8:
            biasf = rng.normal(0.0, 1.0, size=N).astype(np.float32)
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, bias_f32=biasf, device=True, lda=lda)
            np.testing.assert_array_equal(got.view(np.uint32), oracle.gemmlowp_f32(A, B, biasf, ao, bo, 3e-4).view(np.uint32))


@pytest.mark.parametrize("M", [1, 5, 8])
def test_skinny_stage_once_kernel_deep_k(M):
    """Up to 8 rows, 8192 < K <= 16384 and no more column groups than compute units (the down projection of a feed-forward
    block): every wave stages 3 or 4 chunks of 4 k blocks of A and re-reads them per chunk; K picks both chunk counts,
    with a short last busy wave (K = 11008: 172 k blocks over waves of 12) and waves without k blocks (K = 8256: one k
    block more than the shallower form takes); N a ragged single group up to 256 groups; every epilogue, both signs.
    (K = 4160, 6400 and 8192 run the shallower form with one workgroup per group.)"""
    rng = np.random.default_rng(4400 + M)
    for (N, K) in [(4096, 11008), (40, 4160), (1000, 8192), (300, 12288), (2500, 16384), (777, 14336), (4096, 6400), (520, 8256)]:
        a_dt = np.uint8 if (N + K) % 3 == 0 else np.int8
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(1, 20))
        lda = K + (0 if K % 128 else 16)
        announce("skinny deep K", (M, N, K), "lda", lda, a_dt.__name__)
        want = oracle.gemmlowp_s32(A, B, ao, bo)
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=capi.PATH_AUTO, device=True, lda=lda, ldd=N + 3)
        assert name.startswith("skinny"), name
        np.testing.assert_array_equal(got, want)
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N)) * 128.0 / np.sqrt(K)
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        lo, hi, off = (-128, 127, -7) if a_dt == np.int8 else (0, 255, 121)
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, 0, bias, mult, shift, off, lo, hi, device=True, lda=lda)
        np.testing.assert_array_equal(got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, 0, mult, shift, off, lo, hi, a_dt))
        if a_dt == np.int8:
            biasf = rng.normal(0.0, 1.0, size=N).astype(np.float32)
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, bias_f32=biasf, device=True, lda=lda)
            np.testing.assert_array_equal(got.view(np.uint32), oracle.gemmlowp_f32(A, B, biasf, ao, bo, 3e-4).view(np.uint32))


@pytest.mark.parametrize("M", [17, 24, 25, 31, 32, 33, 48, 63, 64])
def test_skinny_kernel_with_several_row_blocks(M):
    """17 to 64 rows run as 2 or 4 blocks of 16 rows in the streaming kernel (from 25 rows on with A staged through LDS
    step by step); N picks 1, 2 or 4 column groups per workgroup and 4 or 8 waves; K covers whole steps only, a tail of
    whole 64-byte blocks, and a ragged tail."""
    rng = np.random.default_rng(900 + M)
    for (N, K) in [(100, 200), (4100, 1024), (8200, 333), (16400, 448), (21000, 192), (300, 4160), (11000, 2112)]:
        a_dt = np.int8 if (N // 100) % 2 else np.uint8
        A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
        B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
        ao, bo = int(rng.integers(-20, 20)), int(rng.integers(-20, 20))
        announce("skinny row blocks", (M, N, K), a_dt.__name__)
        got, name = run_gemm(A, B, capi.EPI_S32, np.int32, ao, bo, path=capi.PATH_SKINNY, device=True)
        assert name.startswith("skinny"), name
        np.testing.assert_array_equal(got, oracle.gemmlowp_s32(A, B, ao, bo))
        bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
        reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N)) * 128.0 / np.sqrt(K)
        mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
        lo, hi, off = (-128, 127, -7) if a_dt == np.int8 else (0, 255, 121)
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, a_dt, ao, 0, bias, mult, shift, off, lo, hi, path=capi.PATH_SKINNY,
                          device=True)
        np.testing.assert_array_equal(got, oracle.gemmlowp_fixedpoint(A, B, bias, ao, 0, mult, shift, off, lo, hi, a_dt))
        if a_dt == np.int8:
            biasf = rng.normal(0.0, 1.0, size=N).astype(np.float32)
            got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, bias_f32=biasf, path=capi.PATH_SKINNY,
                              device=True)
            np.testing.assert_array_equal(got.view(np.uint32), oracle.gemmlowp_f32(A, B, biasf, ao, bo, 3e-4).view(np.uint32))


@pytest.mark.parametrize("K,lda", [(1000, 1000), (1001, 1001), (998, 1000), (64, 80), (17, 17), (1, 1)])
def test_row_strides_and_k_tails(K, lda):
    """A rows that are not 16-byte aligned (dword-aligned: direct loads with a guarded tail; otherwise the padded
    copy), x-padding on A and on the destination (tests/validation/fixtures/GEMMLowpFixture.h:302)."""
    rng = np.random.default_rng(42)
    M, N = 70, 90
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    want = oracle.gemmlowp_s32(A, B, 7, -3)
    for path in (capi.PATH_MFMA, capi.PATH_SIMPLE):
        for device in (True, False):
            announce("strides", K, lda, "path", path, "device", device)
            got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, 7, -3, path=path, device=device, lda=lda, ldd=N + 5)
            np.testing.assert_array_equal(got, want)
    announce("strides skinny", K, lda)
    got, _ = run_gemm(A[:9], B, capi.EPI_S32, np.int32, 7, -3, path=capi.PATH_SKINNY, device=True, lda=lda)
    np.testing.assert_array_equal(got, want[:9])


def test_per_channel_left_and_right_shifts():
    rng = np.random.default_rng(43)
    M, N, K = 150, 130, 200
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    bias = rng.integers(-2000, 2000, size=N, dtype=np.int32)
    reals = np.exp(rng.uniform(np.log(1e-4), np.log(3.0), size=N))
    mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
    assert (shift < 0).any() and (shift > 0).any()
    want = oracle.gemmlowp_fixedpoint(A, B, bias, -3, 0, mult, shift, -5, -128, 127, np.int8)
    for path in (capi.PATH_MFMA, capi.PATH_SIMPLE):
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.int8, -3, 0, bias, mult, shift, -5, -128, 127, path=path,
                          device=True)
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", ["std", "mixed_shifts", "negative_mult", "big_offset", "uint8_out"])
@pytest.mark.parametrize("N,ldd", [(256, 256), (250, 256), (250, 252), (250, 251), (130, 144)])
def test_pipelined_kernel_epilogue_variants(case, N, ldd):
    """Every store path of the pipelined kernel's fused output stage (LDS-staged 16-byte rows with and without a ragged
    right edge, packed dwords, single bytes) crossed with every arithmetic path (common case, general branch-free
    case with left / zero / one-bit shifts, negative multipliers, offsets too large for the folded rounding)."""
    rng = np.random.default_rng(zlib.crc32(repr((case, N, ldd)).encode()))
    M, K = 300, 512
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    bias = rng.integers(-20000, 20000, size=N, dtype=np.int32)
    reals = np.exp(rng.uniform(np.log(2e-4), np.log(2e-3), size=N))
    off, dt, lo, hi = -5, np.int8, -128, 127
    if case == "mixed_shifts":
        reals = np.exp(rng.uniform(np.log(1e-4), np.log(3.0), size=N))
    mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
    if case == "mixed_shifts":
        shift[:4] = [0, 1, 2, 31]
        assert (shift < 0).any() and (shift > 1).any()
    elif case == "negative_mult":
        mult[::7] = -mult[::7]
    elif case == "big_offset":
        off, lo, hi = (1 << 29) + 77, -128, 127
    elif case == "uint8_out":
        off, dt, lo, hi = 128, np.uint8, 3, 250
    want = oracle.gemmlowp_fixedpoint(A, B, bias, -3, 0, mult, shift, off, lo, hi, dt)
    announce("pipelined epilogue", case, N, ldd)
    got, name = run_gemm(A, B, capi.EPI_FIXEDPOINT, dt, -3, 0, bias, mult, shift, off, lo, hi, path=capi.PATH_MFMA,
                         device=True, ldd=ldd)
    assert name.startswith("pp_"), name
    np.testing.assert_array_equal(got, want)

def test_run_can_be_captured_in_a_hip_graph():
    """run() with device buffers only enqueues kernels on the given stream, so it can be captured; every replay, with
    eager work and synchronisations in between, must reproduce the eager result."""
    import torch
    rng = np.random.default_rng(47)
    M, N, K = 300, 256, 512
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    bias = rng.integers(-5000, 5000, size=N).astype(np.int32)
    mult, shift = oracle.calculate_quantized_multipliers(1.0, rng.uniform(2e-4, 2e-3, size=N).astype(np.float32), 1.0)
    want = oracle.gemmlowp_fixedpoint(A, B, bias, -3, 0, mult, shift, -5, -128, 127, np.int8)
    g = capi.Gemm(M, N, K, capi.S8, capi.S8, capi.S8, capi.EPI_FIXEDPOINT, -3, 0,
                  capi.requant(0, 0, -5, -128, 127, per_channel=True))
    Ad, Bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    vecs = [torch.from_numpy(x).cuda() for x in (bias, mult, shift)]
    Dd = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    g.prepare(Bd, *vecs)
    g.run(Ad, Dd)  # first run outside the capture: allocates the handle's workspace
    torch.cuda.synchronize()
    np.testing.assert_array_equal(Dd.cpu().numpy(), want)
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    announce("graph capture")
    with torch.cuda.graph(graph, stream=side):
        g.run(Ad, Dd, None, torch.cuda.current_stream().cuda_stream)
    for rep in range(4):
        Dd.fill_(77)                                # eager work between replays
        A2 = torch.roll(Ad, rep, 0) if rep else Ad  # and new input contents in the same buffer
        Ad.copy_(A2)
        torch.cuda.synchronize()
        announce("graph replay", rep)
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(Dd.cpu().numpy(), np.roll(want, sum(range(rep + 1)), 0))
    g.close()

@pytest.mark.parametrize("M", [9, 70])
@pytest.mark.parametrize("k_interleave", [0, 16])
def test_b_handed_over_transposed_and_with_reordered_k(M, k_interleave):
    """Fully connected weights arrive as [num_outputs][num_inputs] and, after a convolution in the other data layout,
    with their K index permuted (CpuTransposeKernel + CpuConvertFullyConnectedWeightsKernel in the reference): both are
    folded into the packing of B."""
    import torch
    rng = np.random.default_rng(48 + M + k_interleave)
    N, K = 150, 240
    A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
    Wt = rng.integers(0, 256, size=(N, K), dtype=np.uint8)       # as handed over
    ldb = K + 8                                                  # with a row stride
    Wt_padded = np.zeros((N, ldb), dtype=np.uint8)
    Wt_padded[:, :K] = Wt
    if k_interleave:
        k = np.arange(K)
        src_k = (k % k_interleave) * (K // k_interleave) + k // k_interleave
        B = Wt[:, src_k].T
    else:
        B = Wt.T
    bias = rng.integers(-4000, 4000, size=N).astype(np.int32)
    mult, shift = oracle.calculate_quantized_multiplier(0.0009)
    want = oracle.gemmlowp_fixedpoint(A, np.ascontiguousarray(B), bias, -120, -131, [mult], [shift], 9, 0, 255, np.uint8)
    for path in paths_for(M):
        announce("transposed B", M, k_interleave, "path", path)
        g = capi.Gemm(M, N, K, capi.U8, capi.U8, capi.U8, capi.EPI_FIXEDPOINT, -120, -131,
                      capi.requant(mult, shift, 9, 0, 255), path=path, ldb=ldb, b_transposed=True,
                      b_k_interleave=k_interleave)
        Ad, Bd, Dd = torch.from_numpy(A).cuda(), torch.from_numpy(Wt_padded).cuda(), torch.zeros((M, N), dtype=torch.uint8, device="cuda")
        g.prepare(Bd, torch.from_numpy(bias).cuda())
        g.run(Ad, Dd)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(Dd.cpu().numpy(), want)
        g.close()

@pytest.mark.parametrize("device", [False, True])
@pytest.mark.parametrize("M,N,K,ldd,path", [(200, 136, 192, None, capi.PATH_MFMA), (70, 61, 100, 67, capi.PATH_MFMA),
                                            (8, 136, 192, None, capi.PATH_SKINNY), (9, 20, 33, None, capi.PATH_SIMPLE),
                                            (96, 130, 64, 131, capi.PATH_MFMA)])
def test_accumulate_into_s32_and_f32(M, N, K, ldd, path, device):
    """GEMMInfo::accumulate: dst += result. S32 adds wrap (the destination is the GEMM's own accumulator in the
    reference, tests/validation/fixtures/GEMMLowpFixture.h:469-483 only uses values that cannot overflow); F32 adds the
    previous value between the bias and the offset term (src/core/NEON/kernels/arm_gemm/quantized.cpp:1007-1014)."""
    rng = np.random.default_rng(zlib.crc32(("acc %d %d %d" % (M, N, K)).encode()))
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    prev_i = rng.integers(-(1 << 31), (1 << 31) - 1, size=(M, N), dtype=np.int64).astype(np.int32)
    announce("accumulate S32", M, N, K, ldd, path, device)
    got, _ = run_gemm(A, B, capi.EPI_S32, np.int32, 5, -3, path=path, device=device, ldd=ldd, prev=prev_i,
                      flags=capi.GEMM_ACCUMULATE)
    want = (oracle.gemmlowp_s32(A, B, 5, -3).astype(np.int64) + prev_i).astype(np.int32)  # wraps
    assert np.array_equal(got, want)
    prev_f = rng.normal(0.0, 3.0, size=(M, N)).astype(np.float32)
    bias = rng.normal(0.0, 1.0, size=N).astype(np.float32)
    for offs, act, twice in [((0, 0), (-np.inf, np.inf), False), ((5, -3), (0.0, 6.0), True), ((5, -3), (0.0, np.inf), False)]:
        announce("accumulate F32", M, N, K, ldd, path, device, offs, act, twice)
        flags = capi.GEMM_ACCUMULATE | (capi.GEMM_ACT_TWICE if twice else 0)
        got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, offs[0], offs[1], scale=1e-3, bias_f32=bias, act=act, path=path,
                          device=device, ldd=ldd, prev=prev_f, flags=flags)
        want = oracle.gemmlowp_f32(A, B, bias, offs[0], offs[1], 1e-3, act[0], act[1], prev=prev_f, act_twice=twice)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))  # same float operations in the same order


@pytest.mark.parametrize("M", [8, 150])
def test_f32_activation_clamps_before_and_after_the_offset_term(M):
    """With an activation its assembly GEMM fuses, the reference clamps float(acc)*scale+bias, adds the offset term and
    clamps again (quantized.cpp:1015, then CpuGemmLowpMatrixMultiplyCore.cpp:326-332): GEMM_ACT_TWICE. The two differ
    from a single clamp wherever the first clamp moved the value and the offset term moves it back inside."""
    rng = np.random.default_rng(77 + M)
    N, K = 96, 128
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    once = oracle.gemmlowp_f32(A, B, None, 40, 25, 1e-3, 0.0, 6.0)
    twice = oracle.gemmlowp_f32(A, B, None, 40, 25, 1e-3, 0.0, 6.0, act_twice=True)
    assert (once != twice).mean() > 0.05  # the case tells the two apart
    announce("act twice", M)
    got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, 40, 25, scale=1e-3, act=(0.0, 6.0), flags=capi.GEMM_ACT_TWICE)
    assert np.array_equal(got.view(np.uint32), twice.view(np.uint32))
    got, _ = run_gemm(A, B, capi.EPI_F32, np.float32, 40, 25, scale=1e-3, act=(0.0, 6.0))
    assert np.array_equal(got.view(np.uint32), once.view(np.uint32))


@pytest.mark.parametrize("device", [False, True])
@pytest.mark.parametrize("W,H,N,K,batch,epi", [(5, 4, 33, 40, 2, "s32"), (7, 9, 136, 64, 1, "s8"), (3, 2, 24, 19, 3, "f32acc"),
                                               (40, 8, 72, 100, 1, "s8")])
def test_rows_in_planes_with_gaps_between_them(W, H, N, K, batch, epi, device):
    """GEMMInfo::reinterpret_input_as_3d / depth_output_gemm3d on tensors padded along y: A is [batch][H][W rows + gap][K],
    D likewise (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:520-534 reads the tensors' strides): the same result
    as on dense matrices, the gaps of D untouched, strides given at create or afterwards through set_strides_3d."""
    import torch
    rng = np.random.default_rng(zlib.crc32(("planes %d %d %d %d" % (W, H, N, K)).encode()))
    M = W * H
    lda, ldd, gap_a, gap_d = K + 5, N + 3, 2, 3  # gaps in rows
    A = rng.integers(-128, 128, size=(batch, H, W, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    a_buf = np.full((batch, H, W + gap_a, lda), 99, dtype=np.int8)
    a_buf[:, :, :W, :K] = A
    dt = {"s32": np.int32, "s8": np.int8, "f32acc": np.float32}[epi]
    fill = {"s32": 0x5A5A5A5A, "s8": 0x5A, "f32acc": 7.5}[epi]
    d_buf = np.full((batch, H, W + gap_d, ldd), fill, dtype=dt)
    prev = rng.normal(0, 3, size=(batch, H, W, N)).astype(np.float32)
    if epi == "f32acc":
        d_buf[:, :, :W, :N] = prev
    A2 = A.reshape(batch * M, K)
    if epi == "s32":
        want = oracle.gemmlowp_s32(A2, B, 4, -2)
        kw = dict(epilogue=capi.EPI_S32, dst_dtype=capi.S32)
    elif epi == "s8":
        mult, shift = oracle.calculate_quantized_multipliers(0.02, [0.03], 0.9)
        want = oracle.gemmlowp_fixedpoint(A2, B, None, 4, -2, mult, shift, -3, -128, 127, np.int8)
        kw = dict(epilogue=capi.EPI_FIXEDPOINT, dst_dtype=capi.S8, rq=capi.requant(int(mult[0]), int(shift[0]), -3, -128, 127))
    else:
        want = oracle.gemmlowp_f32(A2, B, None, 4, -2, 1e-3, prev=prev.reshape(batch * M, N))
        kw = dict(epilogue=capi.EPI_F32, dst_dtype=capi.F32, scale=1e-3, flags=capi.GEMM_ACCUMULATE)
    a_ps, d_ps = (W + gap_a) * lda, (W + gap_d) * ldd
    late = (W + H) % 2 == 1
    announce("rows in planes", W, H, N, K, batch, epi, "device", device, "strides set late", late)
    if late:
        g = capi.Gemm(M, N, K, capi.S8, capi.S8, a_offset=4, b_offset=-2, batch=batch, a_planes=(W, W * K), d_planes=(W, W * N),
                      **kw)
        g.set_strides_3d(lda, N, ldd, H * a_ps, 0, H * d_ps, a_ps, d_ps)
    else:
        g = capi.Gemm(M, N, K, capi.S8, capi.S8, a_offset=4, b_offset=-2, batch=batch, lda=lda, ldd=ldd, a_planes=(W, a_ps),
                      d_planes=(W, d_ps), a_batch_stride=H * a_ps, d_batch_stride=H * d_ps, **kw)
    if device:
        bd, ad, dd = to_dev(B), to_dev(a_buf), to_dev(d_buf)
        g.prepare(bd)
        g.run(ad, dd)
        torch.cuda.synchronize()
        got = dd.cpu().numpy()
    else:
        g.prepare(B)
        got = d_buf.copy()
        g.run(a_buf, got)
    g.close()
    valid = got[:, :, :W, :N].reshape(batch * M, N)
    if epi == "f32acc":
        assert np.array_equal(valid.view(np.uint32), want.view(np.uint32))
    else:
        np.testing.assert_array_equal(valid, want)
    mask = np.ones(got.shape, dtype=bool)
    mask[:, :, :W, :N] = False
    assert (got[mask] == d_buf[mask]).all(), "gaps of the destination were overwritten"


def test_accumulate_is_rejected_with_an_output_stage():
    with pytest.raises(capi.Mi355Error, match="accumulation"):
        capi.Gemm(16, 16, 16, capi.S8, capi.S8, capi.S8, capi.EPI_FIXEDPOINT, rq=capi.requant(1 << 30, 1, 0, -128, 127),
                  flags=capi.GEMM_ACCUMULATE)
    with pytest.raises(capi.Mi355Error, match="flag"):
        capi.Gemm(16, 16, 16, capi.S8, capi.S8, capi.S32, capi.EPI_S32, flags=64)


def test_requant_extremes_on_device():
    """Accumulators and multipliers at the edges of int32 (saturating SQDMULH, shift 0 / 31, wrap-around adds)
    through the stand-alone output stage."""
    import torch
    I32_MIN, I32_MAX = -(1 << 31), (1 << 31) - 1
    vals = np.array([I32_MIN, I32_MIN + 1, -(1 << 30), -65537, -3, -2, -1, 0, 1, 2, 3, 65535, 1 << 30, I32_MAX - 1,
                     I32_MAX, 123456789], dtype=np.int32).reshape(1, -1)
    for m in (1 << 30, 1518500250, I32_MAX, I32_MIN, 1, -1):
        for s in (-3, -1, 0, 1, 8, 30, 31):
            for dt, lo, hi in ((np.int8, -128, 127), (np.uint8, 0, 255)):
                want = oracle.output_stage_fixedpoint(vals, None, [m], [s], 10, lo, hi, dt)
                dst = torch.zeros(vals.shape, dtype=torch.int8 if dt == np.int8 else torch.uint8, device="cuda")
                capi.output_stage(torch.from_numpy(vals).cuda(), None, dst, capi.requant(m, s, 10, lo, hi))
                np.testing.assert_array_equal(dst.cpu().numpy(), want)


def test_output_stage_fixture(golden):
    g = golden("output_stage.npz")
    for n in range(int(g["count"])):
        mult, shift, roff, lo, hi, with_bias = (int(x) for x in g["p%d" % n])
        src, dst = g["src%d" % n], g["dst%d" % n]
        out = np.zeros_like(dst)
        announce("output stage fixture", n, src.shape, dst.dtype)
        capi.output_stage(np.ascontiguousarray(src), np.ascontiguousarray(g["bias%d" % n]) if with_bias else None,
                          out, capi.requant(mult, shift, roff, lo, hi))
        np.testing.assert_array_equal(out, dst)


@pytest.mark.parametrize("device", [False, True])
@pytest.mark.parametrize("N,ld_dst", [(64, None), (37, None), (64, 68), (40, 41)])
def test_output_stage_to_qsymm16(N, ld_dst, device):
    """int32 -> QSYMM16 (CpuGemmLowpQuantizeDownInt32ToInt16ScaleByFixedPointKernel): rounding high multiply, no offset"""
    import torch
    rng = np.random.default_rng(160 + N)
    M = 50
    src = np.concatenate([rng.integers(-(1 << 31), 1 << 31, size=(M // 2, N)),
                          rng.integers(-(1 << 18), 1 << 18, size=(M - M // 2, N))]).astype(np.int32)
    bias = rng.integers(-5000, 5000, size=N).astype(np.int32)
    ld = ld_dst or N
    for mult, shift, lo, hi in [(1518500250, 3, -32768, 32767), ((1 << 31) - 1, 0, -(1 << 31), (1 << 31) - 1),
                                (1 << 30, -2, -100, 20000), (1073741825, 17, 0, 32767), (-(1 << 30), 5, -32768, 32767)]:
        for b in (bias, None):
            announce("output stage s16", N, ld_dst, device, mult, shift, lo, hi, b is not None)
            want = oracle.output_stage_fixedpoint_s16(src, b, mult, shift, lo, hi)
            dst = np.full((M, ld), 77, dtype=np.int16)
            rq = capi.requant(mult, shift, 0, lo, hi)
            if device:
                sd, dd = torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()
                bd = None if b is None else torch.from_numpy(b).cuda()
                capi.output_stage(sd, bd, dd, rq, ld_dst=ld)
                torch.cuda.synchronize()
                dst = dd.cpu().numpy()
            else:
                capi.output_stage(src, b, dst, rq, ld_dst=ld)
            assert np.array_equal(dst[:, :N], want)
            assert (dst[:, N:] == 77).all()
    with pytest.raises(capi.Mi355Error, match="result offset"):
        capi.output_stage(src, None, np.zeros((M, N), dtype=np.int16), capi.requant(1 << 30, 1, 5, -32768, 32767))
    with pytest.raises(capi.Mi355Error, match="int16 range"):
        capi.output_stage(src, None, np.zeros((M, N), dtype=np.int16), capi.requant(1 << 30, 1, 0, -40000, 100))


def test_output_stage_scale_fixture(golden):
    """QUANTIZE_DOWN (integer multiplier), stand-alone, against the reference oracle's outputs (per-tensor entries)."""
    g = golden("output_stage_scale.npz")
    ran = 0
    for n in range(int(g["count"])):
        roff, lo, hi, with_bias = (int(x) for x in g["p%d" % n])
        mult, shift = g["mult%d" % n], g["shift%d" % n]
        if len(mult) > 1:
            continue
        if lo == hi:
            lo, hi = -(1 << 31), (1 << 31) - 1
        src, dst = g["src%d" % n], g["dst%d" % n]
        out = np.zeros_like(dst)
        announce("scale output stage fixture", n, src.shape, dst.dtype)
        capi.output_stage(np.ascontiguousarray(src), np.ascontiguousarray(g["bias%d" % n]) if with_bias else None, out,
                          capi.requant(int(mult[0]), int(shift[0]), roff, lo, hi, stage=capi.STAGE_SCALE))
        np.testing.assert_array_equal(out, dst)
        ran += 1
    assert ran >= 10


@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("M", [7, 200])
def test_fused_scale_stage_on_every_path(M, per_channel):
    """GEMM + offset contribution + bias + QUANTIZE_DOWN (integer multiplier) fused, against the oracle whose stage is
    pinned by the reference's gemmlowp_quantize_down_scale (tests/test_oracle_gemm.py)."""
    rng = np.random.default_rng(49 + M + int(per_channel))
    N, K = 170, 256
    A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
    B = rng.integers(0, 256, size=(K, N), dtype=np.uint8)
    bias = rng.integers(-4000, 4000, size=N).astype(np.int32)
    cnt = N if per_channel else 1
    mult = rng.integers(1, 9, size=cnt).astype(np.int32)
    shift = rng.integers(13, 16, size=cnt).astype(np.int32)
    b_off = 0 if per_channel else -121
    want = oracle.gemmlowp_scale(A, B, bias, -130, b_off, mult, shift, 900, 3, 250, np.uint8)
    assert ((want > 3) & (want < 250)).mean() > 0.2
    for path in paths_for(M):
        announce("fused scale stage", M, per_channel, "path", path)
        got, _ = run_gemm(A, B, capi.EPI_FIXEDPOINT, np.uint8, -130, b_off, bias, mult, shift, 900, 3, 250, path=path,
                          device=True, stage=capi.STAGE_SCALE)
        np.testing.assert_array_equal(got, want)

def test_update_quant_and_rerun():
    """update_quantization_parameters: new offsets / multiplier without re-packing B; run twice gives identical bytes
    (tests/validation/NEON/GEMMLowp.cpp:211-297 MultipleExecutionWithConfigure)."""
    import torch
    rng = np.random.default_rng(44)
    M, N, K = 96, 80, 144
    A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
    B = rng.integers(0, 256, size=(K, N), dtype=np.uint8)
    bias = rng.integers(-500, 500, size=N, dtype=np.int32)
    g = capi.Gemm(M, N, K, capi.U8, capi.U8, capi.U8, capi.EPI_FIXEDPOINT, -10, -20,
                  capi.requant(1518500250, 9, 5, 0, 255))
    Ad, Bd, bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(bias).cuda()
    D1 = torch.zeros((M, N), dtype=torch.uint8, device="cuda")
    D2 = torch.zeros_like(D1)
    g.prepare(Bd, bd)
    g.run(Ad, D1)
    g.run(Ad, D2)
    torch.cuda.synchronize()
    want = oracle.gemmlowp_fixedpoint(A, B, bias, -10, -20, [1518500250], [9], 5, 0, 255, np.uint8)
    np.testing.assert_array_equal(D1.cpu().numpy(), want)
    np.testing.assert_array_equal(D2.cpu().numpy(), want)
    g.update_quant(-100, -128, capi.requant(1288490240, 10, 17, 3, 250))
    g.run(Ad, D1)
    torch.cuda.synchronize()
    want = oracle.gemmlowp_fixedpoint(A, B, bias, -100, -128, [1288490240], [10], 17, 3, 250, np.uint8)
    np.testing.assert_array_equal(D1.cpu().numpy(), want)
    g.close()


def test_run_before_prepare_is_an_error():
    g = capi.Gemm(32, 32, 32, capi.S8, capi.S8, capi.S32, capi.EPI_S32)
    with pytest.raises(capi.Mi355Error):
        g.run(np.zeros((32, 32), np.int8), np.zeros((32, 32), np.int32))
    g.close()

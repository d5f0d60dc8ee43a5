"""A seeded random sweep over the whole C ABI against the oracle: dense products of every shape class (skinny, mid-sized,
the 256 x 128 tile with and without K tails, deep K, tiny), every epilogue, batches with shared and per-entry B, row
strides on A and on the destination, signed and unsigned operands with offsets; NHWC convolutions of every class the cost
model tells apart (band forms with one and several panels, the narrow kernel, the tiled kernel, K slices), strides,
padding, dilation, weights with an offset. Bit-exact throughout (F32 only for signed operands, as in the other tests)."""
import numpy as np
import pytest

import oracle
from computelibrary_amd import capi
from gpu_util import announce, run_gemm
from test_gpu_conv import run_conv

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_random_sweep_against_the_oracle(seed):
    CASES = 70
    rng = np.random.default_rng(seed)
    n_g = n_c = 0
    bad = []

    def pick(*xs): return xs[int(rng.integers(len(xs)))]
    for _case in range(CASES):
        if rng.random() < 0.6:
            # ---- GEMM
            kind = pick("skinny", "skinny", "mid", "wide", "small", "deep")
            if kind == "skinny": M, N, K = int(rng.integers(1, 65)), int(rng.integers(1, 3000)), pick(64, 128, 1024, 2048, 4096, 4096 + 64, 777, 8192, 11008)
            elif kind == "mid": M, N, K = int(rng.integers(65, 600)), int(rng.integers(1, 700)), int(rng.integers(1, 1500))
            elif kind == "wide": M, N, K = pick(256, 512, 768, 700, 1024), pick(128, 256, 384, 200), pick(128, 1000, 1096, 512, 130, 2048)
            elif kind == "deep": M, N, K = int(rng.integers(1, 200)), int(rng.integers(1, 300)), pick(2048, 4096, 4608, 8192)
            else: M, N, K = int(rng.integers(1, 40)), int(rng.integers(1, 40)), int(rng.integers(1, 80))
            batch = pick(1, 1, 1, 2, 5) if M * N * K < 3e8 else 1
            a_dt, b_dt = pick(np.int8, np.uint8), pick(np.int8, np.int8, np.uint8)
            ao, bo = int(rng.integers(-30, 30)), pick(0, 0, int(rng.integers(-30, 30)))
            lda = K + pick(0, 0, 4, 16, 24)
            ldd = N + pick(0, 0, 3, 16)
            b_b = batch > 1 and rng.random() < 0.5
            path = pick(capi.PATH_AUTO, capi.PATH_AUTO, capi.PATH_MFMA, capi.PATH_TILE + 0) if kind != "skinny" else pick(capi.PATH_AUTO, capi.PATH_SKINNY)
            epi = pick("s32", "fix", "fix", "f32")
            A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(batch, M, K)).astype(a_dt)
            B = rng.integers(np.iinfo(b_dt).min + 1, np.iinfo(b_dt).max + 1, size=((batch, K, N) if b_b else (K, N))).astype(b_dt)
            Aa = A if batch > 1 else A[0]
            B3 = B if b_b else np.broadcast_to(B, (batch, K, N))
            announce("random sweep, gemm", kind, (batch, M, N, K), a_dt.__name__, b_dt.__name__, ao, bo, "lda", lda, "ldd", ldd, "bb", b_b, "path", path, epi)
            try:
                if epi == "s32":
                    got, name = run_gemm(Aa, B, capi.EPI_S32, np.int32, ao, bo, path=path, device=True, lda=lda, ldd=ldd)
                    want = np.stack([oracle.gemmlowp_s32(A[z], B3[z], ao, bo) for z in range(batch)])
                elif epi == "fix":
                    pc = rng.random() < 0.6
                    bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
                    reals = np.exp(rng.uniform(np.log(2e-5), np.log(2e-3), size=N if pc else 1)) * 128.0 / np.sqrt(K)
                    mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
                    o_dt = a_dt
                    lo, hi, off = (-128, 127, int(rng.integers(-20, 20))) if o_dt == np.int8 else (0, 255, int(rng.integers(100, 140)))
                    got, name = run_gemm(Aa, B, capi.EPI_FIXEDPOINT, o_dt, ao, bo, bias, mult, shift, off, lo, hi, path=path, device=True, lda=lda, ldd=ldd)
                    want = np.stack([oracle.gemmlowp_fixedpoint(A[z], B3[z], bias, ao, bo, mult, shift, off, lo, hi, o_dt) for z in range(batch)])
                else:
                    if a_dt != np.int8 or b_dt != np.int8:
                        continue
                    got, name = run_gemm(Aa, B, capi.EPI_F32, np.float32, ao, bo, scale=3e-4, path=path, device=True, lda=lda, ldd=ldd)
                    want = np.stack([oracle.gemmlowp_f32(A[z], B3[z], None, ao, bo, 3e-4) for z in range(batch)]).view(np.uint32)
                    got = got.view(np.uint32)
                g3 = got if batch > 1 else got[None]
                if not np.array_equal(g3, want):
                    bad.append(("gemm", kind, batch, M, N, K, a_dt.__name__, b_dt.__name__, ao, bo, lda, ldd, b_b, path, epi, name)); print("   MISMATCH", name, int((g3 != want).sum()))
                else:
                    print("   ok", name)
                n_g += 1
            except RuntimeError as e:
                print("   error:", e); bad.append(("gemm-error", str(e)))
        else:
            # ---- convolution
            kind = pick("band", "band", "multi", "narrow", "tile", "slices")
            if kind == "band": shape = (pick(1, 2, 4), int(rng.integers(60, 200)), int(rng.integers(60, 200)), pick(64, 64, 128, 256)); ofm = int(rng.integers(1, 65)); kh, kw = pick((3, 3), (1, 1), (3, 1), (2, 2), (5, 5) if shape[3] == 64 else (1, 1))
            elif kind == "multi": shape = (pick(2, 4, 8), int(rng.integers(120, 260)), int(rng.integers(120, 260)), pick(64, 64, 128)); ofm = int(rng.integers(65, 257)); kh, kw = pick((1, 1), (1, 1), (1, 3) if shape[3] == 64 else (1, 1))
            elif kind == "narrow": shape = (pick(1, 3), int(rng.integers(8, 60)), int(rng.integers(8, 60)), pick(16, 32, 48, 64, 96)); ofm = int(rng.integers(1, 257)); kh, kw = pick((3, 3), (1, 1), (2, 3))
            elif kind == "tile": shape = (pick(1, 2), int(rng.integers(8, 40)), int(rng.integers(8, 40)), pick(16, 64, 128, 200, 3, 24)); ofm = int(rng.integers(65, 400)); kh, kw = pick((3, 3), (1, 1), (3, 2))
            else: shape = (pick(1, 2), int(rng.integers(5, 16)), int(rng.integers(5, 16)), pick(256, 512)); ofm = int(rng.integers(64, 300)); kh, kw = pick((3, 3), (2, 2))
            if shape[3] * kh * kw > 1152 and kind in ("band",):
                kh, kw = 1, 1
            stride = pick((1, 1), (1, 1), (2, 2), (1, 2)); dil = pick((1, 1), (1, 1), (2, 2))
            pad = tuple(int(x) for x in rng.integers(0, 3, size=4))
            if shape[1] + pad[2] + pad[3] < (kh - 1) * dil[1] + 1 or shape[2] + pad[0] + pad[1] < (kw - 1) * dil[0] + 1:
                continue
            dt, w_dt = pick(np.int8, np.uint8), pick(np.int8, np.int8, np.uint8)
            w_zp = 0 if w_dt == np.int8 and rng.random() < 0.7 else int(rng.integers(-10, 10)) + (128 if w_dt == np.uint8 else 0)
            src = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max + 1, size=shape).astype(dt)
            w = rng.integers(np.iinfo(w_dt).min + 1, np.iinfo(w_dt).max + 1, size=(ofm, kh, kw, shape[3])).astype(w_dt)
            bias = rng.integers(-500, 500, size=ofm, dtype=np.int32)
            K = kh * kw * shape[3]
            zp = 5 if dt == np.int8 else 131
            lo, hi, ozp = (-128, 127, -5) if dt == np.int8 else (0, 255, 9)
            pc = rng.random() < 0.6
            reals = rng.uniform(0.5, 2.0, ofm if pc else 1) * 40.0 / (K ** 0.5 * 74.0 * 74.0)
            mult, shift = oracle.calculate_quantized_multipliers(1.0, reals, 1.0)
            announce("random sweep, conv", kind, shape, (ofm, kh, kw), stride, pad, dil, dt.__name__, w_dt.__name__, w_zp, "pc", pc)
            try:
                want = oracle.conv_nhwc_direct(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
                got, name = run_conv(src, w, bias, zp, w_zp, mult, shift, ozp, lo, hi, stride, pad, dil)
                if not np.array_equal(got, want):
                    bad.append(("conv", kind, shape, ofm, kh, kw, stride, pad, dil, dt.__name__, w_dt.__name__, w_zp, pc, name)); print("   MISMATCH", name, int((got != want).sum()))
                else:
                    print("   ok", name)
                n_c += 1
            except RuntimeError as e:
                print("   error:", e); bad.append(("conv-error", str(e)))
    assert not bad, bad
    assert n_g + n_c > CASES // 2

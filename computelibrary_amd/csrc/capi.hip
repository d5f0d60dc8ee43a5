// Implementation of the C ABI declared in include/mi355_gemmlowp.h: descriptor checks, kernel selection, device
// workspace ownership, host <-> device staging, and the launches. No arithmetic lives here.
#include "../../include/mi355_gemmlowp.h"
#include "internal.hpp"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>

using namespace mi355;

// Workspace of mi355_gemmlowp_run_noalloc: row sums of A, then (rows that are not dword aligned) the padded copy of A.
// One array per GPU for the life of the process; every call on a GPU shares it.
#define MI355_NOALLOC_SCRATCH_BYTES (8u << 20)
static __device__ __align__(256) unsigned char scratch[MI355_NOALLOC_SCRATCH_BYTES];

namespace
{
thread_local std::string g_err;

int fail(const char *fmt, ...)
{
    char    buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_err = buf;
    return 1;
}

#define HIP_TRY(expr)                                                                                  \
    do                                                                                                 \
    {                                                                                                  \
        const hipError_t e_ = (hipError_t)(expr);                                                      \
        if (e_ != hipSuccess)                                                                          \
            return fail("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__);    \
    } while (0)
#define TRY(expr)            \
    do                       \
    {                        \
        if ((expr) != 0)     \
            return 1;        \
    } while (0)

bool is_device_ptr(const void *p)
{
    if (p == nullptr)
        return false;
    hipPointerAttribute_t attr;
    const hipError_t      e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess)
    {
        (void)hipGetLastError(); // plain host memory: clear the sticky error
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

// What kind of memory an argument slot of a handle was last given: asked once per value and slot, so that a
// steady-state run() asks nothing. The answer lives and dies with the handle. It is stale only if the address is freed
// and handed out again by an allocation of the other kind between two runs of the same handle (the header says so).
struct PtrKind
{
    const void *p   = nullptr;
    bool        dev = false;
    bool        is_device(const void *q)
    {
        if (q == nullptr)
            return false;
        if (q != p)
            dev = is_device_ptr(q), p = q;
        return dev;
    }
};

struct DevBuf
{
    void  *p   = nullptr;
    size_t cap = 0;
    int    ensure(size_t bytes)
    {
        if (bytes <= cap && p != nullptr)
            return 0;
        if (p)
        {
            HIP_TRY(hipFree(p));
            p = nullptr, cap = 0;
        }
        if (bytes == 0)
            bytes = 16;
        HIP_TRY(hipMalloc(&p, bytes));
        cap = bytes;
        return 0;
    }
    void release()
    {
        if (p)
            (void)hipFree(p);
        p = nullptr, cap = 0;
    }
    template <typename T>
    T *as() const
    {
        return (T *)p;
    }
};

// brings `bytes` at `src` to the device if it is host memory; returns the device pointer to use
int to_device(const void *src, size_t bytes, DevBuf &stage, hipStream_t s, const void **out, PtrKind *kind = nullptr)
{
    if (src == nullptr)
    {
        *out = nullptr;
        return 0;
    }
    if (kind ? kind->is_device(src) : is_device_ptr(src))
    {
        *out = src;
        return 0;
    }
    TRY(stage.ensure(bytes));
    HIP_TRY(hipMemcpyAsync(stage.p, src, bytes, hipMemcpyHostToDevice, s));
    *out = stage.p;
    return 0;
}

int num_cus()
{
    static int cus = -1;
    if (cus < 0)
    {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess)
            return 256;
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess)
            return 256;
        cus = prop.multiProcessorCount;
    }
    return cus;
}

bool is_8bit(int dt)
{
    return dt == MI355_U8 || dt == MI355_S8;
}

// The part of a GEMM that both the dense handle and the convolution handle need
struct GemmCore
{
    int     M = 0, N = 0, K = 0, batch = 1;
    int     epi       = EPI_S32;
    int     dst_dtype = MI355_S32;
    bool    flip_a = false, flip_b = false;
    int32_t a_offset = 0, b_offset = 0; // as given (added convention)
    mi355_requant rq{};
    float   scale = 1.f, act_min = -INFINITY, act_max = INFINITY;
    bool    accumulate = false, act_twice = false;
    int     path = MI355_PATH_AUTO, cfg_idx = 0, dma_idx = -1;
    int     force_tile = -1; // >= 0: the pipelined kernel's tile configuration the caller asked for (MI355_PATH_TILE + n)
    int     Kp = 0, Np = 0;
    bool    b_shared = true; // one B for all batches
    bool    has_bias = false, has_pc = false, prepared = false;
    bool    has_narrow = false; // Bn holds the narrow kernel's image of B
    bool    pt_vectors = false; // streaming path, per-tensor requantisation: mult / shift hold the scalars, replicated
    std::string kname;
    DevBuf  Bp, Bs, Bn, colsum, colvec, rowvec, mult, shift, bias, Ap, fill, qp, zeros, parts, zerocol;
    int     splitk = 1;      // K slices of the pipelined kernel
    int     splitk_plan = 1; // what the cost model chose with the tile shape (create()); prepare() checks it and allocates
    bool    conv_core = false; // the GEMM inside a convolution handle
    int     k_const = 0;       // > 0: the K of the constant term a_offset * b_offset * K, where the kernels' K counts padded channels
    bool    qp_on = false; // the digested requantisation vectors (and the flag word behind them) exist
    std::string kname_mfma, kname_dma, kprefix;
    // The names a run can report, composed when the choice is made (create, prepare, update): a run only points at one
    // of them - it must not touch the host heap
    std::string        kname_narrow, kname_band, kname_dma_full, kname_splitk, kname_mfma_full;
    const char        *kname_static = nullptr; // the streaming kernel names its forms itself
    const std::string *kname_run = nullptr; // what the last run took (nullptr: no run yet, kname is what create announced)
    uint8_t fill_byte = 0; // value of the 16 filler bytes (0, or the im2col pad value)
    void   *ext_ws = nullptr; // set around a run that must not allocate: see run_dense
    size_t  ext_ws_bytes = 0;
    bool    ext_ws_busy = false; // the caller's workspace may still be read by kernels of another stream
    bool    ext_ws_used = false; // set by run_dense: this run put something into the caller's workspace

    void refresh_names()
    {
        kname_narrow    = kprefix + "narrow_32x64";
        kname_band      = kprefix + "band_32x64";
        kname_dma_full  = kprefix + kname_dma;
        kname_splitk    = kname_dma_full + "_splitk" + std::to_string(splitk);
        kname_mfma_full = kprefix + kname_mfma;
    }
    const char *name() const { return kname_static ? kname_static : (kname_run ? kname_run->c_str() : kname.c_str()); }

    int32_t a_off_eff() const { return (int32_t)((uint32_t)a_offset + (flip_a ? 128u : 0u)); }
    int32_t b_off_eff() const { return (int32_t)((uint32_t)b_offset + (flip_b ? 128u : 0u)); }
    int     nb() const { return b_shared ? 1 : batch; }

    void release()
    {
        Bp.release(), Bs.release(), Bn.release(), colsum.release(), colvec.release(), rowvec.release(), mult.release();
        shift.release(), bias.release(), Ap.release(), fill.release(), qp.release(), zeros.release(), parts.release(), zerocol.release();
    }

    int choose_kernel()
    {
        Kp = round_up(K, PACK_K_ALIGN);
        Np = round_up(N, PACK_N_ALIGN);
        if (path >= MI355_PATH_TILE)
        {
            if (path - MI355_PATH_TILE >= dma_num_configs())
                return fail("path %d names tile configuration %d; there are %d", path, path - MI355_PATH_TILE, dma_num_configs());
            force_tile = path - MI355_PATH_TILE, path = MI355_PATH_MFMA;
        }
        else if (path < 0 || path > MI355_PATH_SKINNY)
            return fail("unknown path %d", path);
        if (path == MI355_PATH_AUTO)
            // measured: up to 32 rows the streaming kernel always wins; up to 64 rows only while N is small enough
            // that the pipelined kernel would leave most compute units without a tile
            // (a batch of small products runs the streaming kernel once per entry: the tiled kernels would spend a 64-row
            // tile, mostly padding, on each)
            // (and up to 64 rows whenever K <= 4096 is a whole number of 64-byte blocks: the form of the streaming
            // kernel that keeps the operand blocks of A in registers for its whole run then applies)
            path = (M <= 32 || (batch == 1 && M <= SKINNY_MAX_M && (N < 8192 || (K <= 4096 && K % 64 == 0)))) ? MI355_PATH_SKINNY
                                                                                                         : MI355_PATH_MFMA;
        if (path == MI355_PATH_SKINNY && M > SKINNY_MAX_M)
            return fail("skinny path needs M <= %d", SKINNY_MAX_M);
        if (path == MI355_PATH_SIMPLE)
            kname = "simple";
        else if (path == MI355_PATH_SKINNY)
            kname = "skinny";
        else
        {
            const int cus = num_cus();
            auto      pick = [&](int count, MfmaConfig (*get)(int), const char *env) -> int
            {
                int  best = -1;
                long most = -1;
                for (int i = 0; i < count; ++i)
                {
                    const MfmaConfig c     = get(i);
                    const long       tiles = (long)((M + c.BM - 1) / c.BM) * ((N + c.BN - 1) / c.BN) * batch;
                    if (N <= 64 && c.BN > 64)
                        continue;
                    if (tiles >= cus)
                        return i;
                    if (tiles > most)
                        most = tiles, best = i;
                }
                (void)env;
                return best;
            };
            // The pipelined kernel's tile is chosen with a small cost model in clocks per compute unit, from what was
            // measured on the device: a K step costs the largest of its direct-to-LDS stream (about 44 bytes per
            // clock and compute unit), its matrix instructions (4096 multiply-accumulates per clock) and the two
            // barrier-separated slots of the consumer groups (about 1000 clocks per 128 bytes of K, whatever the tile);
            // every tile adds a fixed start-up plus an epilogue proportional to its outputs, which co-resident
            // workgroups overlap. Ties go to the deeper ring (more loads in flight when B comes from HBM).
            // A single dense GEMM may also run its K range as 2, 4 or 8 slices (see prepare()): the tiles of all slices
            // share the chip, every slice has 1/S of the K steps, and a second kernel reads the S planes of partial
            // sums back (measured: about 2.5 bytes per clock and compute unit of the whole chip, plus a launch).
            auto pick_dma = [&]() -> int
            {
                int    best = -1, best_lds = 0;
                double best_cost = 0;
                for (int i = 0; i < dma_num_configs(); ++i)
                {
                    const MfmaConfig c = dma_config(i);
                    if ((N <= 64 && c.BN > 64) || Kp % c.BK != 0)
                        continue;
                    const double tiles   = (double)((M + c.BM - 1) / c.BM) * ((N + c.BN - 1) / c.BN) * batch;
                    const int    occ_lds = (160 * 1024) / c.lds_bytes, occ_wav = 32 / c.waves;
                    const double occ     = std::max(1, std::min(occ_lds, occ_wav));
                    const double nk      = (double)((K + c.BK - 1) / c.BK);
                    const double step    = std::max({(double)(c.BM + c.BN) * c.BK / 44.0, (double)c.BM * c.BN * c.BK / 4096.0,
                                                     1000.0 * c.BK / 128.0});
                    const double fixed   = 6000.0 + (double)c.BM * c.BN / 4.4;
                    for (int sl = 1; sl <= 8; sl *= 2)
                    {
                        if (sl > 1 && (batch != 1 || K % (sl * c.BK) != 0 || K / sl < 1024))
                            break;
                        const double per_cu = std::ceil(tiles * sl / cus);
                        const double finish = sl > 1 ? 4000.0 + (double)sl * M * N * 4.0 / (2.5 * cus) : 0.0;
                        const double cost   = per_cu * (nk / sl) * step + std::ceil(per_cu / occ) * fixed + finish;
                        if (best < 0 || cost < best_cost || (cost == best_cost && sl == 1 && c.lds_bytes > best_lds))
                            best = i, best_cost = cost, best_lds = c.lds_bytes, splitk_plan = sl;
                    }
                }
                return best;
            };
            cfg_idx = pick(mfma_num_configs(), mfma_config, nullptr);
            dma_idx = pick_dma();
            if (force_tile >= 0 && Kp % dma_config(force_tile).BK == 0 && dma_idx != force_tile)
            {
                // a tile shape named by the caller: as many slices as fill the chip once, at least 1024 deep
                dma_idx = force_tile, splitk_plan = 1;
                const MfmaConfig c     = dma_config(dma_idx);
                const int64_t    tiles = (int64_t)((M + c.BM - 1) / c.BM) * ((N + c.BN - 1) / c.BN);
                if (batch == 1 && tiles * 2 <= cus && K >= 2048)
                {
                    int sl = (int)std::min<int64_t>(std::min<int64_t>(cus / tiles, K / 1024), 8);
                    while (sl > 1 && K % (sl * c.BK) != 0)
                        --sl;
                    splitk_plan = sl;
                }
            }
            if (K < 16)
                dma_idx = -1;
            kname_mfma = mfma_config(cfg_idx).name;
            kname_dma  = dma_idx >= 0 ? dma_config(dma_idx).name : "";
            kname      = dma_idx >= 0 ? kname_dma : kname_mfma;
        }
        refresh_names();
        return 0;
    }

    // after Bp / colsum have been written for every B: per-column vectors
    int finish_prepare(const int32_t *bias_in, const int32_t *mult_in, const int32_t *shift_in, hipStream_t s)
    {
        has_bias = bias_in != nullptr;
        if (has_bias)
        {
            TRY(bias.ensure(sizeof(int32_t) * (size_t)N));
            HIP_TRY(hipMemcpyAsync(bias.p, bias_in, sizeof(int32_t) * (size_t)N, hipMemcpyDefault, s));
        }
        has_pc = epi == EPI_FIXEDPOINT && rq.per_channel != 0;
        if (has_pc)
        {
            if (mult_in == nullptr || shift_in == nullptr)
                return fail("per-channel requantisation needs multiplier and shift arrays");
            // padded like the packed B panel: the epilogue reads these as 16-byte vectors
            TRY(mult.ensure(sizeof(int32_t) * (size_t)Np));
            TRY(shift.ensure(sizeof(int32_t) * (size_t)Np));
            HIP_TRY(fill_i32_launch(mult.as<int32_t>(), 0, Np, s));
            HIP_TRY(fill_i32_launch(shift.as<int32_t>(), 0, Np, s));
            HIP_TRY(hipMemcpyAsync(mult.p, mult_in, sizeof(int32_t) * (size_t)N, hipMemcpyDefault, s));
            HIP_TRY(hipMemcpyAsync(shift.p, shift_in, sizeof(int32_t) * (size_t)N, hipMemcpyDefault, s));
        }
        if (path == MI355_PATH_SKINNY)
        {
            TRY(Bs.ensure((size_t)nb() * Np * Kp));
            for (int b = 0; b < nb(); ++b)
                HIP_TRY(pack_b_skinny_launch(Bp.as<int8_t>() + (size_t)b * Np * Kp, Kp, Np, Bs.as<int8_t>() + (size_t)b * Np * Kp, s));
        }
        // few output columns and a short K: the image of the B panel the narrow kernel copies into LDS
        has_narrow = path == MI355_PATH_MFMA && nb() == 1 && (N <= 64 || (N <= 256 && K <= 192)) && narrow_panel_chunks(K) > 0;
        if (has_narrow)
        {
            const int chunks = narrow_panel_chunks(K);
            const int rows = round_up(N, 64); // panels of 64 columns (Np, a multiple of 256, covers them)
            TRY(Bn.ensure((size_t)rows * (chunks + NARROW_PAD_PIECES) * 16));
            HIP_TRY(pack_b_narrow_launch(Bp.as<int8_t>(), Kp, Np, chunks, rows, Bn.as<int8_t>(), s));
        }
        TRY(fill.ensure(16));
        HIP_TRY(fill_i32_launch(fill.as<int32_t>(), (int32_t)(0x01010101u * fill_byte), 4, s));
        if (path == MI355_PATH_SKINNY)
        {
            // the streaming kernel fetches its per-row vector without asking whether there is one
            TRY(zeros.ensure(sizeof(int32_t) * SKINNY_MAX_M));
            HIP_TRY(fill_i32_launch(zeros.as<int32_t>(), 0, SKINNY_MAX_M, s));
        }
        // A deep K under few output tiles: the pipelined kernel would leave most compute units idle, each of the others
        // walking the whole K. The K range is cut into slices that run as the batch entries of one S32 launch (the slice
        // offset is the batch stride of A and of the packed B alike), and a second kernel sums the planes and applies the
        // epilogue. Slices are whole k steps of the tile shape, so no slice but the matrix' own end has a tail.
        splitk = 1;
        if (path == MI355_PATH_MFMA && dma_idx >= 0 && batch == 1 && splitk_plan > 1 && K % (splitk_plan * dma_config(dma_idx).BK) == 0)
            splitk = splitk_plan;
        if (splitk > 1)
        {
            const size_t ldp = ((size_t)N + 3) & ~(size_t)3;
            TRY(parts.ensure(sizeof(int32_t) * (size_t)splitk * M * ldp));
            TRY(zerocol.ensure(sizeof(int32_t) * (size_t)Np));
            HIP_TRY(fill_i32_launch(zerocol.as<int32_t>(), 0, Np, s));
        }
        TRY(refresh_colvec(s));
        TRY(refresh_qparams(s));
        refresh_names();
        prepared = true;
        return 0;
    }

    int refresh_colvec(hipStream_t s)
    {
        TRY(colvec.ensure(sizeof(int32_t) * (size_t)Np * nb()));
        for (int b = 0; b < nb(); ++b)
            HIP_TRY(colvec_launch(colsum.as<int32_t>() + (size_t)b * Np,
                                  (has_bias && epi == EPI_FIXEDPOINT) ? bias.as<int32_t>() : nullptr, a_off_eff(),
                                  b_off_eff(), k_const > 0 ? k_const : K, N, colvec.as<int32_t>() + (size_t)b * Np, s));
        return 0;
    }

    // Digest multipliers / shifts for the pipelined kernel's epilogue. Whether the branch-free forms apply (no negative
    // multiplier; every column normalised) is left in a flag word behind the vectors, which the kernel reads itself:
    // nothing here waits for the device.
    int refresh_qparams(hipStream_t s)
    {
        qp_on = false;
        if (path == MI355_PATH_SKINNY && epi == EPI_FIXEDPOINT && !has_pc)
        {
            // the streaming kernel always reads per-column vectors (a fetch behind a condition would cost it the exact
            // count of its loads in flight): per-tensor constants are replicated
            TRY(mult.ensure(sizeof(int32_t) * (size_t)Np));
            TRY(shift.ensure(sizeof(int32_t) * (size_t)Np));
            HIP_TRY(fill_i32_launch(mult.as<int32_t>(), rq.multiplier, Np, s));
            HIP_TRY(fill_i32_launch(shift.as<int32_t>(), rq.shift, Np, s));
            pt_vectors = true;
        }
        if (epi != EPI_FIXEDPOINT || rq.stage != MI355_STAGE_FIXEDPOINT)
            return 0;
        TRY(qp.ensure(sizeof(int32_t) * ((size_t)QP_COUNT * Np + 4)));
        int32_t *flag = qp.as<int32_t>() + (size_t)QP_COUNT * Np;
        HIP_TRY(qparams_launch(has_pc ? mult.as<int32_t>() : nullptr, has_pc ? shift.as<int32_t>() : nullptr,
                               rq.multiplier, rq.shift, N, Np, qp.as<int32_t>(), flag, s));
        qp_on = true;
        return 0;
    }

    void fill_epi(EpiParams &p, const float *bias_f32) const
    {
        p.qp                  = qp_on ? qp.as<int32_t>() : nullptr;
        p.qp_flag             = qp_on ? qp.as<int32_t>() + (size_t)QP_COUNT * Np : nullptr;
        p.qp_std              = (qp_on && rq.result_offset > -(1 << 28) && rq.result_offset < (1 << 28)) ? 1 : 0;
        p.qp_stride           = Np;
        p.colvec              = colvec.as<int32_t>();
        p.rowvec              = nullptr;
        p.mult                = (has_pc || pt_vectors) ? mult.as<int32_t>() : nullptr;
        p.shift               = (has_pc || pt_vectors) ? shift.as<int32_t>() : nullptr;
        p.bias_f32            = bias_f32;
        p.colvec_batch_stride = b_shared ? 0 : Np;
        p.rowvec_batch_stride = M;
        p.mult_s              = rq.multiplier;
        p.shift_s             = rq.shift;
        p.result_offset       = rq.result_offset;
        p.stage               = rq.stage;
        const int32_t tlo = dst_dtype == MI355_S8 ? -128 : 0, thi = dst_dtype == MI355_S8 ? 127 : 255;
        p.lo                  = rq.min_bound > tlo ? rq.min_bound : tlo;
        p.hi                  = rq.max_bound < thi ? rq.max_bound : thi;
        p.qp_pk16             = (p.qp_std && rq.result_offset >= -1024 && rq.result_offset <= 1024 && p.lo >= -1024 && p.hi <= 1024) ? 1 : 0;
        p.scale               = scale;
        p.act_min             = act_min;
        p.act_max             = act_max;
        p.has_offsets         = (a_offset != 0 || b_offset != 0) ? 1 : 0;
        p.dst_signed          = dst_dtype == MI355_S8;
        p.accumulate          = accumulate ? 1 : 0;
        p.act_twice           = act_twice ? 1 : 0;
    }

    // A, D and bias_f32 are device pointers here
    int run_dense(const int8_t *A, int64_t lda, int64_t a_bs, void *D, int64_t ldd, int64_t d_bs,
                  const float *bias_f32, hipStream_t s)
    {
        if (!prepared)
            return fail("run before prepare");
        GemmArgs g{};
        fill_epi(g.epi, bias_f32);
        bool flip_in_loader = flip_a;
        int  k_valid        = K;
        const bool direct =
            path == MI355_PATH_SIMPLE || ((((uintptr_t)A | (uintptr_t)lda | (uintptr_t)a_bs) & 3) == 0);
        // the per-row term b_offset * rowsum(A): the pipelined kernels sum the rows of A themselves while its tiles pass
        // through them (dword-aligned rows, K a whole number of 16-byte columns, one launch); otherwise one pass over A
        // in front of the GEMM leaves the sums in a vector
        const bool rowsum_in_kernel = b_off_eff() != 0 && direct && path == MI355_PATH_MFMA && dma_idx >= 0 && K % 16 == 0 && K >= 16 &&
                                      splitk == 1 && (int64_t)lda * 256 + K < ((int64_t)1 << 32);
        const bool need_rowvec = b_off_eff() != 0 && !rowsum_in_kernel;
        // the two workspaces of a run: owned by the handle and grown on demand, or carved out of a buffer the caller of
        // this function brings (ext_ws != nullptr: nothing is allocated, sizes beyond ext_ws_bytes are an error)
        const size_t rv_bytes = need_rowvec ? ((sizeof(int32_t) * (size_t)M * batch + 255) & ~(size_t)255) : 0;
        const size_t ap_bytes = direct ? 0 : (size_t)batch * M * Kp;
        int32_t     *rv       = nullptr;
        int8_t      *ap       = nullptr;
        if (ext_ws != nullptr)
        {
            if (rv_bytes + ap_bytes > 0 && ext_ws_busy)
                return fail("mi355_gemmlowp_run_noalloc: this GPU's workspace is still in use by a call on another stream");
            ext_ws_used = rv_bytes + ap_bytes > 0;
            if (rv_bytes + ap_bytes > ext_ws_bytes)
                return fail("this run needs %zu bytes of workspace (row sums %zu + padded copy of A %zu); the fixed "
                            "workspace holds %zu",
                            rv_bytes + ap_bytes, rv_bytes, ap_bytes, ext_ws_bytes);
            rv = (int32_t *)ext_ws, ap = (int8_t *)ext_ws + rv_bytes;
        }
        else
        {
            if (need_rowvec)
                TRY(rowvec.ensure(rv_bytes));
            if (!direct)
                TRY(Ap.ensure(ap_bytes));
            rv = rowvec.as<int32_t>(), ap = Ap.as<int8_t>();
        }
        if (!direct)
        {
            // rows not dword aligned: padded, sign-normalised copy (and the row sums in the same pass)
            HIP_TRY(a_prepass_launch(A, lda, a_bs, batch, M, K, flip_a, ap, Kp, need_rowvec ? rv : nullptr, b_off_eff(), s));
            A = ap, lda = Kp, a_bs = (int64_t)M * Kp, k_valid = Kp, flip_in_loader = false;
        }
        else if (need_rowvec)
        {
            HIP_TRY(a_prepass_launch(A, lda, a_bs, batch, M, K, flip_a, nullptr, Kp, rv, b_off_eff(), s));
        }
        if (rowsum_in_kernel)
            g.epi.rowsum_mul = b_off_eff();
        if (need_rowvec)
            g.epi.rowvec = rv;
        else if (path == MI355_PATH_SKINNY)
            g.epi.rowvec = zeros.as<int32_t>();
        g.A = A, g.lda = lda, g.a_batch_stride = a_bs;
        g.Bp = Bp.as<int8_t>(), g.Kp = Kp, g.bp_batch_stride = b_shared ? 0 : (int64_t)Np * Kp;
        g.D = D, g.ldd = ldd, g.d_batch_stride = d_bs;
        g.M = M, g.N = N, g.K = k_valid;
        set_vec_store(g);
        return launch(g, flip_in_loader, false, s);
    }

    // 4 consecutive outputs of a row may leave as one store when every row start is aligned to 4 elements
    void set_vec_store(GemmArgs &g) const
    {
        const size_t esz = (epi == EPI_FIXEDPOINT) ? 1 : 4;
        g.epi.vec_store  = (((uintptr_t)g.D % (4 * esz)) == 0 && g.ldd % 4 == 0 && g.d_batch_stride % 4 == 0) ? 1 : 0;
        g.epi.vec_store16 = (esz == 1 && ((uintptr_t)g.D % 16) == 0 && g.ldd % 16 == 0 && g.d_batch_stride % 16 == 0) ? 1 : 0;
    }

    int launch(GemmArgs &g, bool flip_in_loader, bool conv, hipStream_t s)
    {
        if (path == MI355_PATH_SIMPLE)
            HIP_TRY(simple_gemm_launch(epi, flip_in_loader, g, batch, s));
        else if (path == MI355_PATH_SKINNY)
        {
            GemmArgs gb        = g;
            gb.Bp              = Bs.as<int8_t>();
            gb.bp_batch_stride = b_shared ? 0 : (int64_t)Np * Kp;
            if (g.epi.rowvec == zeros.as<int32_t>() || g.epi.rowvec == nullptr)
                gb.epi.rowvec_batch_stride = 0;
            // A batch of small products (under 4 MiB of B each, where the launches themselves are what costs) goes out
            // as one launch with the entries along the grid; larger ones one launch per entry, each free to take the
            // form that stages its A once
            if (batch > 1 && (int64_t)Np * Kp <= ((int64_t)4 << 20) && batch <= 65535)
                HIP_TRY(skinny_launch(epi, flip_in_loader, gb, batch, s, &kname_static));
            else
                for (int b = 0; b < batch; ++b)
                {
                    GemmArgs ge = gb;
                    ge.A        = gb.A + (int64_t)b * gb.a_batch_stride;
                    ge.Bp       = gb.Bp + (int64_t)b * gb.bp_batch_stride;
                    ge.D        = (char *)gb.D + (int64_t)b * gb.d_batch_stride * (epi == EPI_FIXEDPOINT ? 1 : 4);
                    ge.epi.colvec += (int64_t)b * gb.epi.colvec_batch_stride;
                    if (ge.epi.rowvec != nullptr)
                        ge.epi.rowvec += (int64_t)b * gb.epi.rowvec_batch_stride;
                    HIP_TRY(skinny_launch(epi, flip_in_loader, ge, 1, s, &kname_static));
                }
        }
        else
        {
            g.fill16 = fill.as<int8_t>();
            // the pipelined kernel moves 16-byte columns of dword-aligned rows straight into LDS
            const bool aligned =
                conv ? (g.conv.C % 16 == 0 && ((uintptr_t)g.A & 15) == 0 && g.K % 16 == 0)
                     : ((((uintptr_t)g.A | (uintptr_t)g.lda | (uintptr_t)g.a_batch_stride) & 3) == 0);
            g.a_end = conv ? nullptr : g.A + (int64_t)(batch - 1) * g.a_batch_stride + (int64_t)(g.M - 1) * g.lda + g.K;
            // its producers address a block's A rows (dense) or the whole image batch (convolution) with 32-bit offsets
            const int64_t span = conv ? (int64_t)((g.M + g.conv.OH * g.conv.OW - 1) / (g.conv.OH * g.conv.OW)) *
                                            g.conv.H * g.conv.W * g.conv.C
                                      : (int64_t)g.lda * 256 + g.K;
            // few output columns and a short K: every wave for itself, weights resident in LDS (gemm_narrow.hip)
            if (has_narrow && batch == 1 && conv && !g.epi.accumulate && span < ((int64_t)1 << 31) &&
                narrow_applies(g, conv))
            {
                g.Bp            = Bn.as<int8_t>();
                g.conv.pad_word = 0x01010101u * fill_byte; // as in the image: the kernel flips what it loads
                bool band       = false;
                HIP_TRY(narrow_launch(epi, flip_in_loader, conv, g, s, &band));
                kname_run = band ? &kname_band : &kname_narrow;
            }
            else if (dma_idx >= 0 && aligned && g.K >= 16 && span < ((int64_t)1 << 32))
            {
                const MfmaConfig c = dma_config(dma_idx);
                g.tiles_m          = (g.M + c.BM - 1) / c.BM;
                g.tiles_n          = (g.N + c.BN - 1) / c.BN;
                kname_run          = &kname_dma_full;
                if (splitk > 1 && batch == 1 && g.K == K && K % (splitk * c.BK) == 0)
                {
                    const int     ldp = (N + 3) & ~3;
                    const int64_t kc  = K / splitk;
                    GemmArgs      gp  = g;
                    gp.epi                     = EpiParams{};
                    gp.epi.colvec              = zerocol.as<int32_t>();
                    gp.epi.colvec_batch_stride = 0;
                    gp.epi.vec_store           = 1;
                    gp.D = parts.as<int32_t>(), gp.ldd = ldp, gp.d_batch_stride = (int64_t)M * ldp;
                    // (dense: a slice starts kc bytes into every row of A; convolution: kc values into every patch,
                    // which the loader adds to the k it decodes)
                    gp.K = (int)kc, gp.a_batch_stride = conv ? 0 : kc, gp.bp_batch_stride = kc, gp.k_slice = conv ? (int32_t)kc : 0;
                    kname_run = &kname_splitk;
                    HIP_TRY(dma_launch(dma_idx, EPI_S32, flip_in_loader, conv, gp, splitk, s));
                    HIP_TRY(splitk_finish_launch(epi, g, parts.as<int32_t>(), (int64_t)M * ldp, ldp, splitk, s));
                    return 0;
                }
                HIP_TRY(dma_launch(dma_idx, epi, flip_in_loader, conv, g, batch, s));
            }
            else
            {
                const MfmaConfig c = mfma_config(cfg_idx);
                g.tiles_m          = (g.M + c.BM - 1) / c.BM;
                g.tiles_n          = (g.N + c.BN - 1) / c.BN;
                kname_run          = &kname_mfma_full;
                if (conv)
                    g.conv.pad_word = (0x01010101u * fill_byte) ^ (flip_in_loader ? 0x80808080u : 0u);
                HIP_TRY(mfma_launch(cfg_idx, epi, flip_in_loader, conv, g, batch, s));
            }
        }
        return 0;
    }
};

int check_requant(const mi355_requant &rq, int dst_dtype)
{
    if (rq.min_bound > rq.max_bound)
        return fail("min_bound > max_bound");
    if (rq.stage != MI355_STAGE_FIXEDPOINT && rq.stage != MI355_STAGE_SCALE)
        return fail("unknown output stage %d", rq.stage);
    if (rq.stage == MI355_STAGE_SCALE && !rq.per_channel && (rq.shift < 0 || rq.shift > 31))
        return fail("QUANTIZE_DOWN needs a shift in [0, 31] (got %d)", rq.shift);
    // Bounds inside the destination type's range clamp; bounds that cover it only saturate. Bounds with one end inside
    // and one outside are refused: the reference's three implementations disagree there (the stand-alone kernel narrows
    // the bound to 8 bits, src/cpu/kernels/CpuGemmLowpOffsetContributionOutputStageKernel.cpp:502-503; the assembly path
    // clamps in int32 and keeps the low byte, src/core/NEON/kernels/arm_gemm/quantized.cpp:36-46,254-261)
    const int32_t tlo = dst_dtype == MI355_S8 ? -128 : 0, thi = dst_dtype == MI355_S8 ? 127 : 255;
    const bool    covers = rq.min_bound <= tlo && rq.max_bound >= thi;
    const bool    inside = rq.min_bound >= tlo && rq.max_bound <= thi;
    if (!covers && !inside)
        return fail("clamp bounds [%d,%d] are partly outside the destination type's range [%d,%d]", rq.min_bound,
                    rq.max_bound, tlo, thi);
    return 0;
}
} // namespace

struct mi355_gemm_handle
{
    mi355_gemm_desc d;
    GemmCore        core;
    DevBuf          stageA, stageB, stageD, stageBiasF, stageBias, stageMult, stageShift;
    DevBuf          wsF32; // MI355_F16 destination: the dense F32 matrix the kernels write
    DevBuf          denseA, denseD; // matrices handed over as planes with gaps between them, without the gaps
    PtrKind         kindA, kindD, kindBiasF; // host or device memory, per argument of run()
    bool a_planes() const { return d.a_plane_rows > 0 && d.a_plane_stride != (int64_t)d.a_plane_rows * d.lda; }
    bool d_planes() const { return d.d_plane_rows > 0 && d.d_plane_stride != (int64_t)d.d_plane_rows * d.ldd; }
};

static int check_planes(const mi355_gemm_desc &d)
{
    if (d.a_plane_rows < 0 || d.d_plane_rows < 0 || (d.a_plane_rows > 0 && d.M % d.a_plane_rows != 0) ||
        (d.d_plane_rows > 0 && d.M % d.d_plane_rows != 0))
        return fail("plane_rows must divide M");
    if (d.a_plane_rows > 0 && d.a_plane_stride < (int64_t)(d.a_plane_rows - 1) * d.lda + d.K)
        return fail("A plane stride smaller than one plane");
    if (d.d_plane_rows > 0 && d.d_plane_stride < (int64_t)(d.d_plane_rows - 1) * d.ldd + d.N)
        return fail("D plane stride smaller than one plane");
    return 0;
}

// bytes (A) / elements (D) from the first element of a batch entry's matrix to one past its last
static int64_t a_span(const mi355_gemm_desc &d)
{
    return d.a_plane_rows > 0 ? (int64_t)(d.M / d.a_plane_rows - 1) * d.a_plane_stride + (int64_t)(d.a_plane_rows - 1) * d.lda + d.K
                              : (int64_t)(d.M - 1) * d.lda + d.K;
}
static int64_t d_span(const mi355_gemm_desc &d)
{
    return d.d_plane_rows > 0 ? (int64_t)(d.M / d.d_plane_rows - 1) * d.d_plane_stride + (int64_t)(d.d_plane_rows - 1) * d.ldd + d.N
                              : (int64_t)(d.M - 1) * d.ldd + d.N;
}

struct mi355_conv_handle
{
    mi355_conv_desc d;
    GemmCore        core;
    ConvGeom        geom;
    bool            implicit = false;
    DevBuf          stageSrc, stageW, stageDst, stageBias, stageMult, stageShift, cols;
    DevBuf          nhwcSrc, nhwcW, nhwcDst; // MI355_NCHW: the tensors in the kernels' layout
    DevBuf          denseSrc, denseW, denseDst; // tensors that came with gaps, without them
    DevBuf          biasF;                   // F32 destination: the float bias
    bool            has_bias_f32 = false;
    int             c_pad = 0;               // > 0: the kernels see this many channels (source and weights padded, see create)
    ConvGeom        geom_true;               // ... and the geometry with the caller's channel count, for the patches' row sums
    DevBuf          padSrc, padW;
    PtrKind         kindSrc, kindDst; // host or device memory, per argument of run()
};

extern "C"
{
const char *mi355_last_error(void)
{
    return g_err.c_str();
}

int mi355_device_info(char *name, size_t name_len)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess)
    {
        (void)hipGetLastError();
        fail("no HIP device");
        return -1;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess)
    {
        fail("hipGetDeviceProperties failed");
        return -1;
    }
    if (name && name_len)
    {
        strncpy(name, prop.gcnArchName, name_len - 1);
        name[name_len - 1] = 0;
    }
    return prop.multiProcessorCount;
}

int mi355_gemmlowp_create(const mi355_gemm_desc *desc, mi355_gemm_handle **out)
{
    if (!desc || !out)
        return fail("null argument");
    const mi355_gemm_desc &d = *desc;
    if (d.M < 1 || d.N < 1 || d.K < 1 || d.batch < 1)
        return fail("M, N, K, batch must be positive (got %d %d %d %d)", d.M, d.N, d.K, d.batch);
    if (!is_8bit(d.a_dtype) || !is_8bit(d.b_dtype))
        return fail("A and B must be 8-bit");
    if (d.lda < d.K || d.ldb < (d.b_transposed ? d.K : d.N) || d.ldd < d.N)
        return fail("row stride smaller than the row");
    if (d.b_k_interleave < 0 || (d.b_k_interleave > 1 && d.K % d.b_k_interleave != 0))
        return fail("b_k_interleave must divide K");
    switch (d.epilogue)
    {
        case MI355_EPI_S32:
            if (d.dst_dtype != MI355_S32)
                return fail("S32 epilogue needs an S32 destination");
            break;
        case MI355_EPI_FIXEDPOINT:
            if (!is_8bit(d.dst_dtype))
                return fail("FIXEDPOINT epilogue needs an 8-bit destination");
            if (check_requant(d.requant, d.dst_dtype))
                return 1;
            break;
        case MI355_EPI_F32:
            if (d.dst_dtype != MI355_F32 && d.dst_dtype != MI355_F16)
                return fail("F32 epilogue needs an F32 or F16 destination");
            break;
        default:
            return fail("unknown epilogue %d", d.epilogue);
    }
    if ((d.flags & ~(MI355_GEMM_ACCUMULATE | MI355_GEMM_ACT_TWICE)) != 0)
        return fail("unknown flag bits 0x%x", d.flags);
    if ((d.flags & MI355_GEMM_ACCUMULATE) && d.epilogue == MI355_EPI_FIXEDPOINT)
        return fail("accumulation is only possible into an S32 or F32 destination");
    TRY(check_planes(d));
    if (d.batch > 1 && (d.a_batch_stride < a_span(d) || d.d_batch_stride < d_span(d)))
        return fail("batch stride smaller than one matrix");
    if (d.batch > 1 && d.b_batch_stride != 0 &&
        d.b_batch_stride < (d.b_transposed ? (int64_t)(d.N - 1) * d.ldb + d.K : (int64_t)(d.K - 1) * d.ldb + d.N))
        return fail("B batch stride smaller than one matrix");
    mi355_gemm_handle *h = new (std::nothrow) mi355_gemm_handle();
    if (!h)
        return fail("out of host memory");
    h->d        = d;
    GemmCore &c = h->core;
    c.M = d.M, c.N = d.N, c.K = d.K, c.batch = d.batch;
    c.epi = d.epilogue, c.dst_dtype = d.dst_dtype;
    c.flip_a = d.a_dtype == MI355_U8, c.flip_b = d.b_dtype == MI355_U8;
    c.a_offset = d.a_offset, c.b_offset = d.b_offset;
    c.rq = d.requant, c.scale = d.scale, c.act_min = d.act_min, c.act_max = d.act_max;
    c.path     = d.path;
    c.accumulate = (d.flags & MI355_GEMM_ACCUMULATE) != 0, c.act_twice = (d.flags & MI355_GEMM_ACT_TWICE) != 0;
    c.b_shared = d.batch == 1 || d.b_batch_stride == 0;
    if (c.choose_kernel())
    {
        delete h;
        return 1;
    }
    *out = h;
    return 0;
}

int mi355_gemmlowp_prepare(mi355_gemm_handle *h, const void *B, const int32_t *bias, const int32_t *mult,
                           const int32_t *shift, void *stream)
{
    if (!h || !B)
        return fail("null argument");
    hipStream_t            s = (hipStream_t)stream;
    GemmCore              &c = h->core;
    const mi355_gemm_desc &d = h->d;
    const int              nb = c.nb();
    const size_t           b_bytes = (size_t)(nb - 1) * d.b_batch_stride +
                           (d.b_transposed ? (size_t)(d.N - 1) * d.ldb + d.K : (size_t)(d.K - 1) * d.ldb + d.N);
    const void            *Bd, *biasd, *multd, *shiftd;
    TRY(to_device(B, b_bytes, h->stageB, s, &Bd));
    TRY(to_device(bias, sizeof(int32_t) * d.N, h->stageBias, s, &biasd));
    TRY(to_device(c.rq.per_channel ? mult : nullptr, sizeof(int32_t) * d.N, h->stageMult, s, &multd));
    TRY(to_device(c.rq.per_channel ? shift : nullptr, sizeof(int32_t) * d.N, h->stageShift, s, &shiftd));
    TRY(c.Bp.ensure((size_t)nb * c.Np * c.Kp));
    TRY(c.colsum.ensure(sizeof(int32_t) * (size_t)nb * c.Np));
    for (int b = 0; b < nb; ++b)
    {
        const uint8_t *src = (const uint8_t *)Bd + (size_t)b * d.b_batch_stride;
        int8_t        *dst = c.Bp.as<int8_t>() + (size_t)b * c.Np * c.Kp;
        int32_t       *cs  = c.colsum.as<int32_t>() + (size_t)b * c.Np;
        if (d.b_transposed)
            HIP_TRY(pack_bt_launch(src, d.ldb, d.K, d.N, c.Kp, c.Np, c.flip_b, d.b_k_interleave, dst, cs, s));
        else
            HIP_TRY(pack_b_launch(src, d.ldb, d.K, d.N, c.Kp, c.Np, c.flip_b, d.b_k_interleave, dst, cs, s));
    }
    TRY(c.finish_prepare((const int32_t *)biasd, (const int32_t *)multd, (const int32_t *)shiftd, s));
    // staging buffers are reused by later calls: make sure the copies out of them have finished
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int mi355_gemmlowp_update_quant(mi355_gemm_handle *h, int32_t a_offset, int32_t b_offset, const mi355_requant *requant,
                                float scale, void *stream)
{
    if (!h)
        return fail("null argument");
    GemmCore &c = h->core;
    if (requant)
    {
        if (c.epi == EPI_FIXEDPOINT && check_requant(*requant, c.dst_dtype))
            return 1;
        if (requant->per_channel != c.rq.per_channel)
            return fail("update cannot switch between per-tensor and per-channel requantisation");
        c.rq = *requant;
    }
    c.a_offset = a_offset, c.b_offset = b_offset, c.scale = scale;
    h->d.a_offset = a_offset, h->d.b_offset = b_offset, h->d.scale = scale;
    if (c.prepared)
    {
        TRY(c.refresh_colvec((hipStream_t)stream));
        TRY(c.refresh_qparams((hipStream_t)stream));
    }
    return 0;
}

static int set_gemm_strides(mi355_gemm_handle *h, int64_t lda, int64_t ldb, int64_t ldd, int64_t a_batch_stride,
                            int64_t b_batch_stride, int64_t d_batch_stride, int64_t a_plane_stride, int64_t d_plane_stride)
{
    const mi355_gemm_desc &d = h->d;
    if (lda < d.K || ldb < (d.b_transposed ? d.K : d.N) || ldd < d.N)
        return fail("row stride smaller than the row");
    mi355_gemm_desc n = d;
    n.lda = lda, n.ldb = ldb, n.ldd = ldd;
    n.a_plane_stride = a_plane_stride, n.d_plane_stride = d_plane_stride;
    n.a_batch_stride = a_batch_stride, n.b_batch_stride = b_batch_stride, n.d_batch_stride = d_batch_stride;
    TRY(check_planes(n));
    if (d.batch > 1 && (a_batch_stride < a_span(n) || d_batch_stride < d_span(n)))
        return fail("batch stride smaller than one matrix");
    if (d.batch > 1 && (b_batch_stride == 0) != h->core.b_shared)
        return fail("set_strides cannot switch between one shared B and one B per batch entry");
    if (d.batch > 1 && b_batch_stride != 0 &&
        b_batch_stride < (d.b_transposed ? (int64_t)(d.N - 1) * ldb + d.K : (int64_t)(d.K - 1) * ldb + d.N))
        return fail("B batch stride smaller than one matrix");
    h->d = n;
    return 0;
}

int mi355_gemmlowp_set_strides(mi355_gemm_handle *h, int64_t lda, int64_t ldb, int64_t ldd, int64_t a_batch_stride,
                               int64_t b_batch_stride, int64_t d_batch_stride)
{
    if (!h)
        return fail("null argument");
    // planes keep following one another without a gap under the new row strides
    return set_gemm_strides(h, lda, ldb, ldd, a_batch_stride, b_batch_stride, d_batch_stride,
                            (int64_t)h->d.a_plane_rows * lda, (int64_t)h->d.d_plane_rows * ldd);
}

int mi355_gemmlowp_set_strides_3d(mi355_gemm_handle *h, int64_t lda, int64_t ldb, int64_t ldd, int64_t a_batch_stride,
                                  int64_t b_batch_stride, int64_t d_batch_stride, int64_t a_plane_stride,
                                  int64_t d_plane_stride)
{
    if (!h)
        return fail("null argument");
    return set_gemm_strides(h, lda, ldb, ldd, a_batch_stride, b_batch_stride, d_batch_stride, a_plane_stride, d_plane_stride);
}

int mi355_gemmlowp_run(mi355_gemm_handle *h, const void *A, const float *bias_f32, void *D, void *stream)
{
    if (!h || !A || !D)
        return fail("null argument");
    hipStream_t            s = (hipStream_t)stream;
    GemmCore              &c = h->core;
    const mi355_gemm_desc &d = h->d;
    if (bias_f32 && c.epi != EPI_F32)
        return fail("float bias is only valid with the F32 epilogue");
    const bool   f16     = d.dst_dtype == MI355_F16;
    const size_t esz     = d.dst_dtype == MI355_S32 || d.dst_dtype == MI355_F32 ? 4 : (f16 ? 2 : 1);
    const size_t a_bytes = (size_t)(d.batch - 1) * d.a_batch_stride + (size_t)a_span(d);
    const size_t d_elems = (size_t)(d.batch - 1) * d.d_batch_stride + (size_t)d_span(d);
    const void  *Ad, *bfd;
    TRY(to_device(A, a_bytes, h->stageA, s, &Ad, &h->kindA));
    TRY(to_device(bias_f32, sizeof(float) * d.N, h->stageBiasF, s, &bfd, &h->kindBiasF));
    const bool d_host = !h->kindD.is_device(D);
    void      *Dd     = D;
    if (d_host)
    {
        TRY(h->stageD.ensure(d_elems * esz));
        Dd = h->stageD.p;
        if (c.accumulate || d.ldd != d.N || h->d_planes() || (d.batch > 1 && d.d_batch_stride != (int64_t)d.M * d.ldd))
            HIP_TRY(hipMemcpyAsync(Dd, D, d_elems * esz, hipMemcpyHostToDevice, s)); // previous values / padding
    }
    const bool staged_in = Ad != A || bfd != bias_f32;
    // planes with gaps between them: the kernels see dense copies
    int64_t lda = d.lda, a_bs = d.a_batch_stride, ldd = d.ldd, d_bs = d.d_batch_stride;
    void   *Dplanes = nullptr;
    if (h->a_planes())
    {
        const int64_t row = round_up(d.K, 16);
        TRY(h->denseA.ensure((size_t)d.batch * d.M * row));
        HIP_TRY(restride_nd_launch(Ad, h->denseA.p, d.K, d.a_plane_rows, d.M / d.a_plane_rows, d.batch,
                                   RestrideSteps{{d.lda, d.a_plane_stride, d.a_batch_stride}},
                                   RestrideSteps{{row, row * d.a_plane_rows, row * d.M}}, s));
        Ad = h->denseA.p, lda = row, a_bs = row * d.M;
    }
    const RestrideSteps d_given{{d.ldd * (int64_t)esz, d.d_plane_stride * (int64_t)esz, d.d_batch_stride * (int64_t)esz}};
    const RestrideSteps d_dense{{d.N * (int64_t)esz, d.N * (int64_t)esz * d.d_plane_rows, d.N * (int64_t)esz * d.M}};
    if (h->d_planes())
    {
        TRY(h->denseD.ensure((size_t)d.batch * d.M * d.N * esz));
        Dplanes = Dd, Dd = h->denseD.p, ldd = d.N, d_bs = (int64_t)d.M * d.N;
        if (c.accumulate) // the previous values
            HIP_TRY(restride_nd_launch(Dplanes, Dd, (int)(d.N * esz), d.d_plane_rows, d.M / d.d_plane_rows, d.batch, d_given, d_dense, s));
    }
    if (f16)
    {
        // the kernels write a dense F32 matrix, which is rounded into the half destination afterwards. Accumulating:
        // the addition (and the activation, which has to follow it) happens in that second step, on halfs.
        TRY(h->wsF32.ensure(sizeof(float) * (size_t)d.batch * d.M * d.N));
        float      *ws  = h->wsF32.as<float>();
        const bool  acc = c.accumulate, twice = c.act_twice;
        const float lo = c.act_min, hi = c.act_max;
        if (acc)
            c.accumulate = false, c.act_twice = false, c.act_min = -INFINITY, c.act_max = INFINITY;
        const int rc = c.run_dense((const int8_t *)Ad, lda, a_bs, ws, d.N, (int64_t)d.M * d.N, (const float *)bfd, s);
        c.accumulate = acc, c.act_twice = twice, c.act_min = lo, c.act_max = hi;
        if (rc)
            return rc;
        HIP_TRY(f32_to_f16_launch(ws, Dd, d.batch, d.M, d.N, ldd, d_bs, acc, lo, hi, s));
    }
    else
        TRY(c.run_dense((const int8_t *)Ad, lda, a_bs, Dd, ldd, d_bs, (const float *)bfd, s));
    if (Dplanes)
    {
        HIP_TRY(restride_nd_launch(Dd, Dplanes, (int)(d.N * esz), d.d_plane_rows, d.M / d.d_plane_rows, d.batch, d_dense, d_given, s));
        Dd = Dplanes;
    }
    if (d_host)
    {
        HIP_TRY(hipMemcpyAsync(D, Dd, d_elems * esz, hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
    }
    else if (staged_in)
        HIP_TRY(hipStreamSynchronize(s)); // staged inputs must be consumed before the caller may reuse them
    return 0;
}

// Per GPU: the address of its copy of the workspace array, asked once (with that device current), and an event behind
// the last call's kernels, created in the same set-up step. Calls on one stream are ordered by the stream; a call that
// arrives on another stream while the event is still pending would overwrite the workspace under running kernels and
// is refused.
struct NoallocState
{
    void       *ptr      = nullptr;
    hipEvent_t  done     = nullptr;
    hipStream_t last     = nullptr;
    bool        recorded = false;
};
static std::mutex g_noalloc_mutex;
static int noalloc_state(NoallocState **out)
{
    static NoallocState states[64];
    int                 dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64)
        return fail("device index %d out of range", dev);
    NoallocState &st = states[dev];
    if (st.ptr == nullptr)
    {
        void *p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr)
            return fail("hipGetSymbolAddress returned no address for the workspace");
        HIP_TRY(hipEventCreateWithFlags(&st.done, hipEventDisableTiming));
        st.ptr = p;
    }
    *out = &st;
    return 0;
}

size_t mi355_gemmlowp_noalloc_workspace_bytes(void)
{
    return MI355_NOALLOC_SCRATCH_BYTES;
}

int mi355_gemmlowp_run_noalloc(mi355_gemm_handle *h, const void *A, const float *bias_f32, void *D, void *stream)
{
    if (!h || !A || !D)
        return fail("null argument");
    hipStream_t            s = (hipStream_t)stream;
    GemmCore              &c = h->core;
    const mi355_gemm_desc &d = h->d;
    if (!c.prepared)
        return fail("run before prepare");
    if (bias_f32 && c.epi != EPI_F32)
        return fail("float bias is only valid with the F32 epilogue");
    if (d.dst_dtype == MI355_F16)
        return fail("mi355_gemmlowp_run_noalloc does not write F16 destinations (they need a float matrix as workspace)");
    if (h->a_planes() || h->d_planes())
        return fail("mi355_gemmlowp_run_noalloc does not take planes with gaps between them (they need dense copies)");
    if (!h->kindA.is_device(A) || !h->kindD.is_device(D) || (bias_f32 && !h->kindBiasF.is_device(bias_f32)))
        return fail("mi355_gemmlowp_run_noalloc takes device memory only");
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    NoallocState               *st = nullptr;
    TRY(noalloc_state(&st));
    // (a stream under graph capture records no event and is not checked: the graph's own order is the caller's)
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) != hipSuccess)
    {
        (void)hipGetLastError();
        cap = hipStreamCaptureStatusActive;
    }
    const bool tracked = cap == hipStreamCaptureStatusNone;
    if (tracked && st->recorded && st->last != s)
    {
        const hipError_t q = hipEventQuery(st->done);
        if (q == hipErrorNotReady)
        {
            (void)hipGetLastError();
            c.ext_ws_busy = true; // an error if this run needs the workspace at all
        }
        else
            HIP_TRY(q);
    }
    c.ext_ws = st->ptr, c.ext_ws_bytes = MI355_NOALLOC_SCRATCH_BYTES, c.ext_ws_used = false;
    const int  rc   = c.run_dense((const int8_t *)A, d.lda, d.a_batch_stride, D, d.ldd, d.d_batch_stride, bias_f32, s);
    const bool used = c.ext_ws_used;
    c.ext_ws = nullptr, c.ext_ws_bytes = 0, c.ext_ws_busy = false;
    if (tracked && used && rc == 0)
    {
        HIP_TRY(hipEventRecord(st->done, s));
        st->last = s, st->recorded = true;
    }
    return rc;
}

void mi355_gemmlowp_destroy(mi355_gemm_handle *h)
{
    if (!h)
        return;
    h->core.release();
    h->stageA.release(), h->stageB.release(), h->stageD.release(), h->stageBiasF.release(), h->stageBias.release();
    h->stageMult.release(), h->stageShift.release(), h->wsF32.release(), h->denseA.release(), h->denseD.release();
    delete h;
}

const char *mi355_gemmlowp_kernel_name(const mi355_gemm_handle *h)
{
    return h ? h->core.name() : "";
}

int mi355_output_stage_run(const mi355_output_stage_desc *desc, const int32_t *src, const int32_t *bias, void *dst,
                           void *stream)
{
    if (!desc || !src || !dst)
        return fail("null argument");
    const mi355_output_stage_desc &d = *desc;
    if (d.M < 1 || d.N < 1 || d.ld_src < d.N || d.ld_dst < d.N)
        return fail("bad output-stage shape");
    const bool s16 = d.dst_dtype == MI355_S16;
    if (!is_8bit(d.dst_dtype) && !s16)
        return fail("output stage writes QASYMM8, QASYMM8_SIGNED or QSYMM16");
    if (d.requant.per_channel)
        return fail("the stand-alone output stage is per-tensor");
    if (s16)
    {
        if (d.requant.stage != MI355_STAGE_FIXEDPOINT || d.requant.result_offset != 0)
            return fail("the QSYMM16 output stage is QUANTIZE_DOWN_FIXEDPOINT without a result offset");
        if (d.requant.min_bound > d.requant.max_bound)
            return fail("min_bound > max_bound");
        // the reference narrows the bounds to int16 with a plain cast: only bounds that survive it are meaningful
        const bool whole = d.requant.min_bound <= -32768 && d.requant.max_bound >= 32767;
        if (!whole && (d.requant.min_bound < -32768 || d.requant.max_bound > 32767))
            return fail("QSYMM16 clamp bounds [%d,%d] are partly outside the int16 range", d.requant.min_bound,
                        d.requant.max_bound);
    }
    else if (check_requant(d.requant, d.dst_dtype))
        return 1;
    const size_t desz = s16 ? 2 : 1;
    hipStream_t s = (hipStream_t)stream;
    DevBuf      sSrc, sBias, sDst;
    const void *srcd, *biasd;
    const size_t s_elems = (size_t)(d.M - 1) * d.ld_src + d.N, d_elems = (size_t)(d.M - 1) * d.ld_dst + d.N;
    int          rc      = 0;
    void        *Dd      = dst;
    const bool   d_host  = !is_device_ptr(dst);
    EpiParams    p{};
    p.mult_s = d.requant.multiplier, p.shift_s = d.requant.shift, p.result_offset = d.requant.result_offset;
    p.stage  = d.requant.stage;
    const int32_t tlo = s16 ? -32768 : d.dst_dtype == MI355_S8 ? -128 : 0, thi = s16 ? 32767 : d.dst_dtype == MI355_S8 ? 127 : 255;
    p.lo = d.requant.min_bound > tlo ? d.requant.min_bound : tlo;
    p.hi = d.requant.max_bound < thi ? d.requant.max_bound : thi;
    auto body = [&]() -> int
    {
        TRY(to_device(src, s_elems * 4, sSrc, s, &srcd));
        TRY(to_device(bias, sizeof(int32_t) * d.N, sBias, s, &biasd));
        if (d_host)
        {
            TRY(sDst.ensure(d_elems * desz));
            Dd = sDst.p;
            if (d.ld_dst != d.N)
                HIP_TRY(hipMemcpyAsync(Dd, dst, d_elems * desz, hipMemcpyHostToDevice, s));
        }
        if (s16)
            HIP_TRY(output_stage_s16_launch((const int32_t *)srcd, d.ld_src, (const int32_t *)biasd, Dd, d.ld_dst, d.M, d.N, p, s));
        else
            HIP_TRY(output_stage_launch((const int32_t *)srcd, d.ld_src, (const int32_t *)biasd, Dd, d.ld_dst, d.M, d.N, p, s));
        if (d_host)
            HIP_TRY(hipMemcpyAsync(dst, Dd, d_elems * desz, hipMemcpyDeviceToHost, s));
        if (d_host || srcd != src || biasd != bias)
            HIP_TRY(hipStreamSynchronize(s));
        return 0;
    };
    rc = body();
    sSrc.release(), sBias.release(), sDst.release();
    return rc;
}

static void conv_geom(const mi355_conv_desc &d, ConvGeom &g)
{
    g.H = d.H, g.W = d.W, g.C = d.C, g.KH = d.KH, g.KW = d.KW;
    g.stride_x = d.stride_x, g.stride_y = d.stride_y, g.pad_left = d.pad_left, g.pad_top = d.pad_top;
    g.dil_x = d.dilation_x, g.dil_y = d.dilation_y;
    // FLOOR rounding of PadStrideInfo (src/core/Utils.cpp:288-332)
    int w = (int)std::floor((float)(d.W + d.pad_left + d.pad_right - (d.dilation_x * (d.KW - 1) + 1)) / (float)d.stride_x + 1.f);
    int h = (int)std::floor((float)(d.H + d.pad_top + d.pad_bottom - (d.dilation_y * (d.KH - 1) + 1)) / (float)d.stride_y + 1.f);
    g.OW = w < 1 ? 1 : w;
    g.OH = h < 1 ? 1 : h;
    auto magic = [](int32_t dv) -> uint32_t { return dv == 1 ? 0u : (uint32_t)(((uint64_t)1 << 32) / (uint64_t)dv) + 1u; };
    g.magic_C = magic(g.C), g.magic_KW = magic(g.KW), g.magic_OW = magic(g.OW), g.magic_OH = magic(g.OH);
}

// the implicit-GEMM loader divides by C, KW, OW and OH with 32-bit reciprocal multiplies: exact while x * d < 2^32
static bool conv_fast_div_ok(const mi355_conv_desc &d, const ConvGeom &g)
{
    const int64_t M = (int64_t)d.batch * g.OH * g.OW, K = (int64_t)d.KH * d.KW * d.C, lim = (int64_t)1 << 32;
    return M * g.OW < lim && (M / g.OW + 1) * g.OH < lim && (K + 256) * d.C < lim && ((int64_t)d.KH * d.KW + 256) * d.KW < lim;
}

void mi355_conv_out_dims(const mi355_conv_desc *desc, int32_t *OH, int32_t *OW)
{
    ConvGeom g{};
    conv_geom(*desc, g);
    if (OH)
        *OH = g.OH;
    if (OW)
        *OW = g.OW;
}

// One tensor of a convolution as runs of contiguous bytes: seg bytes per run, n1 x n2 x n3 runs along dimensions 1..3 of
// the tensor, 'given' the caller's byte strides of those dimensions (0 resolved to "no gap"), 'dense' the gap-free ones
struct ConvTensorSteps
{
    int           seg = 0;
    int64_t       n1 = 0, n2 = 0, n3 = 0;
    RestrideSteps given{}, dense{};
    bool          padded = false;
    size_t        extent = 0, bytes = 0; // bytes spanned from the first element with and without the gaps
};

static int conv_tensor_steps(const char *name, int64_t seg, int64_t n1, int64_t n2, int64_t n3, int64_t s1, int64_t s2,
                             int64_t s3, ConvTensorSteps &t)
{
    const int64_t g1 = s1 ? s1 : seg, g2 = s2 ? s2 : g1 * n1, g3 = s3 ? s3 : g2 * n2;
    if (g1 < seg || g2 < g1 * n1 || g3 < g2 * n2)
        return fail("%s: a stride is smaller than what it steps over", name);
    t.seg = (int)seg, t.n1 = n1, t.n2 = n2, t.n3 = n3;
    t.given  = RestrideSteps{{g1, g2, g3}};
    t.dense  = RestrideSteps{{seg, seg * n1, seg * n1 * n2}};
    t.padded = g1 != t.dense.st[0] || g2 != t.dense.st[1] || g3 != t.dense.st[2];
    t.extent = (size_t)((n1 - 1) * g1 + (n2 - 1) * g2 + (n3 - 1) * g3 + seg);
    t.bytes  = (size_t)(seg * n1 * n2 * n3);
    return 0;
}

static int conv_src_steps(const mi355_conv_desc &d, ConvTensorSteps &t)
{
    return d.layout == MI355_NHWC
               ? conv_tensor_steps("src", d.C, d.W, d.H, d.batch, d.src_pixel_stride, d.src_stride2, d.src_stride3, t)
               : conv_tensor_steps("src", d.W, d.H, d.C, d.batch, d.src_pixel_stride, d.src_stride2, d.src_stride3, t);
}

static int conv_weights_steps(const mi355_conv_desc &d, ConvTensorSteps &t)
{
    return d.layout == MI355_NHWC ? conv_tensor_steps("weights", d.C, d.KW, d.KH, d.OFM, d.weights_pixel_stride,
                                                      d.weights_stride2, d.weights_stride3, t)
                                  : conv_tensor_steps("weights", d.KW, d.KH, d.C, d.OFM, d.weights_pixel_stride,
                                                      d.weights_stride2, d.weights_stride3, t);
}

static int conv_dst_steps(const mi355_conv_desc &d, ConvTensorSteps &t)
{
    ConvGeom g;
    conv_geom(d, g);
    const int64_t esz = d.dst_dtype == MI355_F32 ? 4 : 1;
    return d.layout == MI355_NHWC
               ? conv_tensor_steps("dst", d.OFM * esz, g.OW, g.OH, d.batch, d.dst_pixel_stride, d.dst_stride2, d.dst_stride3, t)
               : conv_tensor_steps("dst", g.OW * esz, g.OH, d.OFM, d.batch, d.dst_pixel_stride, d.dst_stride2, d.dst_stride3, t);
}

static int conv_check(const mi355_conv_desc &d)
{
    if (d.batch < 1 || d.H < 1 || d.W < 1 || d.C < 1 || d.OFM < 1 || d.KH < 1 || d.KW < 1)
        return fail("convolution dimensions must be positive");
    if (d.stride_x < 1 || d.stride_y < 1 || d.dilation_x < 1 || d.dilation_y < 1)
        return fail("stride and dilation must be >= 1");
    if (d.pad_left < 0 || d.pad_top < 0 || d.pad_right < 0 || d.pad_bottom < 0)
        return fail("negative padding");
    if (!is_8bit(d.src_dtype) || !is_8bit(d.weights_dtype) || (!is_8bit(d.dst_dtype) && d.dst_dtype != MI355_F32))
        return fail("convolution source and weights must be 8-bit, the destination 8-bit or F32");
    if (d.dst_dtype == MI355_F32)
    {
        if ((d.flags & ~MI355_GEMM_ACT_TWICE) != 0)
            return fail("unknown flag bits 0x%x", d.flags);
    }
    if (d.path < MI355_CONV_AUTO || d.path > MI355_CONV_IN_PLACE)
        return fail("unknown convolution path %d", d.path);
    if (d.layout != MI355_NHWC && d.layout != MI355_NCHW)
        return fail("unknown layout %d", d.layout);
    ConvGeom g;
    conv_geom(d, g);
    if (g.OH < 1 || g.OW < 1)
        return fail("the kernel does not fit into the padded image");
    ConvTensorSteps t;
    TRY(conv_src_steps(d, t));
    TRY(conv_weights_steps(d, t));
    TRY(conv_dst_steps(d, t));
    return 0;
}

int mi355_conv_create(const mi355_conv_desc *desc, mi355_conv_handle **out)
{
    if (!desc || !out)
        return fail("null argument");
    const mi355_conv_desc &d = *desc;
    TRY(conv_check(d));
    const bool f32 = d.dst_dtype == MI355_F32;
    if (!f32)
        TRY(check_requant(d.requant, d.dst_dtype));
    mi355_conv_handle *h = new (std::nothrow) mi355_conv_handle();
    if (!h)
        return fail("out of host memory");
    h->d = d;
    conv_geom(d, h->geom);
    GemmCore     &c  = h->core;
    // A channel count that is not a multiple of 16 (the RGB of a first layer, 24, 40 ...): the implicit loaders move
    // 16-byte pieces of one tap, and the fallback that looks up every byte runs at a few percent of what the bytes
    // allow. Channels can be added for nothing: source pixels and weight taps are copied into buffers with the channels
    // padded to the next multiple of 16, the added weights are zero in the kernels' signed form, so no dot product
    // changes and neither do the column sums of the weights. The two other offset terms are kept on the caller's
    // channel count: the row sums of the patches (needed under a weights offset) are taken from the unpadded source,
    // and the constant a_offset * b_offset * K uses the unpadded K.
    h->geom_true = h->geom;
    {
        if (d.path == MI355_CONV_AUTO && d.C % 16 != 0)
        {
            mi355_conv_desc dp = d;
            dp.C               = round_up(d.C, 16);
            ConvGeom gp;
            conv_geom(dp, gp);
            if (conv_fast_div_ok(dp, gp) && conv_fast_div_ok(d, h->geom) && (int64_t)d.batch * d.H * d.W * dp.C < ((int64_t)1 << 31))
                h->c_pad = dp.C, h->geom = gp;
        }
    }
    const int     c_eff = h->c_pad ? h->c_pad : d.C;
    const int64_t M64 = (int64_t)d.batch * h->geom.OH * h->geom.OW;
    const int64_t K64 = (int64_t)d.KH * d.KW * c_eff;
    if (M64 > INT32_MAX || K64 > INT32_MAX)
    {
        delete h;
        return fail("convolution too large");
    }
    c.M = (int)M64, c.N = d.OFM, c.K = (int)K64, c.batch = 1, c.conv_core = true;
    c.k_const = h->c_pad ? d.KH * d.KW * d.C : 0;
    c.epi = f32 ? EPI_F32 : EPI_FIXEDPOINT, c.dst_dtype = d.dst_dtype;
    c.flip_a = d.src_dtype == MI355_U8, c.flip_b = d.weights_dtype == MI355_U8;
    c.a_offset = d.src_offset, c.b_offset = d.weights_offset;
    c.rq = d.requant, c.path = MI355_PATH_MFMA, c.b_shared = true;
    if (f32)
    {
        c.rq    = mi355_requant{};
        c.scale = d.scale, c.act_min = d.act_min, c.act_max = d.act_max;
        c.act_twice = (d.flags & MI355_GEMM_ACT_TWICE) != 0;
    }
    if (c.choose_kernel())
    {
        delete h;
        return 1;
    }
    // The patch matrix is only materialised on request (path 1) or where the loaders' reciprocal divisions would not be
    // exact. Channel counts that are not a multiple of 16 take the register-staged kernel, whose loader then looks up
    // every byte; a weights offset adds a pass over the source for the patches' row sums.
    h->implicit      = d.path != MI355_CONV_EXPLICIT && (h->c_pad > 0 || conv_fast_div_ok(d, h->geom));
    h->geom.pad_word = ((uint32_t)d.pad_value & 0xFFu) * 0x01010101u;
    if (h->implicit)
        c.fill_byte = (uint8_t)(d.pad_value & 0xFF);
    c.kprefix = h->implicit ? "implicit_" : "im2col+";
    c.kname   = c.kprefix + c.kname;
    c.refresh_names();
    *out                = h;
    return 0;
}

int mi355_conv_prepare(mi355_conv_handle *h, const void *weights, const void *bias, const int32_t *mult,
                       const int32_t *shift, void *stream)
{
    if (!h || !weights)
        return fail("null argument");
    hipStream_t s = (hipStream_t)stream;
    GemmCore   &c = h->core;
    const void *wd, *biasd, *multd, *shiftd;
    const bool  f32 = c.epi == EPI_F32;
    if (f32)
    {
        // the float bias is an argument of every launch: keep a device copy of the caller's values
        h->has_bias_f32 = bias != nullptr;
        if (bias)
        {
            TRY(h->biasF.ensure(sizeof(float) * (size_t)c.N));
            HIP_TRY(hipMemcpyAsync(h->biasF.p, bias, sizeof(float) * (size_t)c.N, hipMemcpyDefault, s));
        }
        bias = nullptr;
    }
    ConvTensorSteps wt;
    TRY(conv_weights_steps(h->d, wt));
    TRY(to_device(weights, wt.extent, h->stageW, s, &wd));
    if (wt.padded)
    {
        TRY(h->denseW.ensure(wt.bytes));
        HIP_TRY(restride_nd_launch(wd, h->denseW.p, wt.seg, wt.n1, wt.n2, wt.n3, wt.given, wt.dense, s));
        wd = h->denseW.p;
    }
    if (h->d.layout == MI355_NCHW)
    {
        // [OFM][C][KH*KW] -> [OFM][KH*KW][C]
        TRY(h->nhwcW.ensure((size_t)c.N * c.K));
        HIP_TRY(transpose_bytes_launch(wd, h->nhwcW.p, c.N, h->d.C, h->d.KH * h->d.KW, s));
        wd = h->nhwcW.p;
    }
    if (h->c_pad)
    {
        // taps of C weights -> taps of c_pad weights; the added ones are zero once the packing has put them in signed form
        TRY(h->padW.ensure((size_t)c.N * c.K));
        HIP_TRY(channel_pad_launch(wd, h->padW.p, (int64_t)c.N * h->d.KH * h->d.KW, h->d.C, h->c_pad, c.flip_b ? 0x80 : 0x00, s));
        wd = h->padW.p;
    }
    TRY(to_device(bias, sizeof(int32_t) * c.N, h->stageBias, s, &biasd));
    TRY(to_device(c.rq.per_channel ? mult : nullptr, sizeof(int32_t) * c.N, h->stageMult, s, &multd));
    TRY(to_device(c.rq.per_channel ? shift : nullptr, sizeof(int32_t) * c.N, h->stageShift, s, &shiftd));
    TRY(c.Bp.ensure((size_t)c.Np * c.Kp));
    TRY(c.colsum.ensure(sizeof(int32_t) * (size_t)c.Np));
    // weights [OFM][KH][KW][C] are already the K-contiguous layout with k = c + kx*C + ky*C*KW
    // (src/cpu/kernels/CpuWeightsReshapeKernel.cpp:150-166)
    HIP_TRY(pack_bt_launch(wd, c.K, c.K, c.N, c.Kp, c.Np, c.flip_b, 0, c.Bp.as<int8_t>(), c.colsum.as<int32_t>(), s));
    TRY(c.finish_prepare((const int32_t *)biasd, (const int32_t *)multd, (const int32_t *)shiftd, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int mi355_conv_update_quant(mi355_conv_handle *h, int32_t src_offset, int32_t weights_offset, int32_t pad_value,
                            const mi355_requant *requant, const int32_t *mult, const int32_t *shift, void *stream)
{
    if (!h || !requant)
        return fail("null argument");
    hipStream_t s = (hipStream_t)stream;
    GemmCore   &c = h->core;
    if (c.epi == EPI_F32)
        return fail("the F32 destination has no requantisation to update: create a new handle for new scales");
    TRY(check_requant(*requant, c.dst_dtype));
    if ((requant->per_channel != 0) != (c.rq.per_channel != 0))
        return fail("update cannot switch between per-tensor and per-channel requantisation");
    h->d.src_offset = src_offset, h->d.weights_offset = weights_offset, h->d.pad_value = pad_value, h->d.requant = *requant;
    c.a_offset = src_offset, c.b_offset = weights_offset, c.rq = *requant;
    h->implicit      = h->d.path != MI355_CONV_EXPLICIT && (h->c_pad > 0 || conv_fast_div_ok(h->d, h->geom));
    h->geom.pad_word = ((uint32_t)pad_value & 0xFFu) * 0x01010101u;
    c.fill_byte      = (uint8_t)(pad_value & 0xFF);
    c.kprefix        = h->implicit ? "implicit_" : "im2col+";
    c.refresh_names();
    if (!c.prepared)
        return 0;
    if (c.rq.per_channel)
    {
        if (!mult || !shift)
            return fail("per-channel requantisation needs multiplier and shift arrays");
        const void *multd, *shiftd;
        TRY(to_device(mult, sizeof(int32_t) * c.N, h->stageMult, s, &multd));
        TRY(to_device(shift, sizeof(int32_t) * c.N, h->stageShift, s, &shiftd));
        HIP_TRY(hipMemcpyAsync(c.mult.p, multd, sizeof(int32_t) * (size_t)c.N, hipMemcpyDeviceToDevice, s));
        HIP_TRY(hipMemcpyAsync(c.shift.p, shiftd, sizeof(int32_t) * (size_t)c.N, hipMemcpyDeviceToDevice, s));
    }
    HIP_TRY(fill_i32_launch(c.fill.as<int32_t>(), (int32_t)(0x01010101u * c.fill_byte), 4, s));
    TRY(c.refresh_colvec(s));
    TRY(c.refresh_qparams(s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int mi355_conv_set_strides(mi355_conv_handle *h, int64_t src_pixel_stride, int64_t weights_pixel_stride,
                           int64_t dst_pixel_stride)
{
    if (!h)
        return fail("null argument");
    const int64_t a[3] = {src_pixel_stride, 0, 0}, b[3] = {weights_pixel_stride, 0, 0}, c[3] = {dst_pixel_stride, 0, 0};
    return mi355_conv_set_strides_nd(h, a, b, c);
}

int mi355_conv_set_strides_nd(mi355_conv_handle *h, const int64_t src[3], const int64_t weights[3], const int64_t dst[3])
{
    if (!h || !src || !weights || !dst)
        return fail("null argument");
    mi355_conv_desc d = h->d;
    d.src_pixel_stride = src[0], d.src_stride2 = src[1], d.src_stride3 = src[2];
    d.weights_pixel_stride = weights[0], d.weights_stride2 = weights[1], d.weights_stride3 = weights[2];
    d.dst_pixel_stride = dst[0], d.dst_stride2 = dst[1], d.dst_stride3 = dst[2];
    TRY(conv_check(d));
    h->d = d;
    return 0;
}

int mi355_conv_run(mi355_conv_handle *h, const void *src, void *dst, void *stream)
{
    if (!h || !src || !dst)
        return fail("null argument");
    hipStream_t            s = (hipStream_t)stream;
    GemmCore              &c = h->core;
    const mi355_conv_desc &d = h->d;
    if (!c.prepared)
        return fail("run before prepare");
    ConvTensorSteps st, dt;
    TRY(conv_src_steps(d, st));
    TRY(conv_dst_steps(d, dt));
    const size_t src_bytes = st.bytes, dst_bytes = dt.bytes, dst_ext = dt.extent;
    const bool   s_pad = st.padded, d_pad = dt.padded;
    const void  *srcd;
    TRY(to_device(src, st.extent, h->stageSrc, s, &srcd, &h->kindSrc));
    if (s_pad)
    {
        TRY(h->denseSrc.ensure(src_bytes));
        HIP_TRY(restride_nd_launch(srcd, h->denseSrc.p, st.seg, st.n1, st.n2, st.n3, st.given, st.dense, s));
        srcd = h->denseSrc.p;
    }
    const bool d_host = !h->kindDst.is_device(dst);
    void      *Dd     = dst;
    if (d_host)
    {
        TRY(h->stageDst.ensure(dst_ext));
        Dd = h->stageDst.p;
        if (d_pad)
            HIP_TRY(hipMemcpyAsync(Dd, dst, dst_ext, hipMemcpyHostToDevice, s)); // keep the caller's padding bytes
    }
    void *Dpadded = Dd;
    if (d_pad)
    {
        TRY(h->denseDst.ensure(dst_bytes));
        Dd = h->denseDst.p;
    }
    const bool nchw   = d.layout == MI355_NCHW;
    void      *Dfinal = Dd;
    if (nchw)
    {
        // every image [C][H*W] -> [H*W][C]; the kernels write [OH*OW][OFM] per image into a buffer of their own
        TRY(h->nhwcSrc.ensure(src_bytes));
        TRY(h->nhwcDst.ensure(dst_bytes));
        HIP_TRY(transpose_bytes_launch(srcd, h->nhwcSrc.p, d.batch, d.C, d.H * d.W, s));
        srcd = h->nhwcSrc.p;
        Dd   = h->nhwcDst.p;
    }
    const void *src_true = srcd; // the caller's channel count
    if (h->c_pad)
    {
        // pixels of C channels -> pixels of c_pad channels (what the added ones hold meets zero weights; the padding value
        // keeps them in range of the source type)
        TRY(h->padSrc.ensure((size_t)d.batch * d.H * d.W * h->c_pad));
        HIP_TRY(channel_pad_launch(srcd, h->padSrc.p, (int64_t)d.batch * d.H * d.W, d.C, h->c_pad, (uint8_t)(d.pad_value & 0xFF), s));
        srcd = h->padSrc.p;
    }
    if (h->implicit)
    {
        GemmArgs g{};
        c.fill_epi(g.epi, h->has_bias_f32 ? h->biasF.as<float>() : nullptr);
        if (c.b_off_eff() != 0)
        {
            ConvGeom gr = h->c_pad ? h->geom_true : h->geom;
            gr.pad_word = ((uint32_t)d.pad_value & 0xFFu) * 0x01010101u;
            TRY(c.rowvec.ensure(sizeof(int32_t) * (size_t)c.M));
            HIP_TRY(conv_rowsum_launch(h->c_pad ? src_true : srcd, gr, c.M, c.flip_a, c.b_off_eff(), c.rowvec.as<int32_t>(), s));
            g.epi.rowvec = c.rowvec.as<int32_t>();
        }
        g.A = (const int8_t *)srcd, g.lda = 0, g.a_batch_stride = 0;
        g.Bp = c.Bp.as<int8_t>(), g.Kp = c.Kp, g.bp_batch_stride = 0;
        g.D = Dd, g.ldd = c.N, g.d_batch_stride = 0;
        g.M = c.M, g.N = c.N, g.K = c.K;
        g.conv = h->geom;
        c.set_vec_store(g);
        TRY(c.launch(g, c.flip_a, true, s));
    }
    else
    {
        // explicit lowering: patch matrix [M][Kp] in workspace, then the dense path
        ConvGeom g2   = h->geom;
        g2.pad_word   = ((uint32_t)d.pad_value & 0xFFu) * 0x01010101u;
        const int ldc = round_up(c.K, 16);
        TRY(h->cols.ensure((size_t)c.M * ldc));
        HIP_TRY(im2col_nhwc_launch(srcd, h->cols.p, d.batch, g2, ldc, s));
        TRY(c.run_dense(h->cols.as<int8_t>(), ldc, 0, Dd, c.N, 0, h->has_bias_f32 ? h->biasF.as<float>() : nullptr, s));
    }
    if (nchw)
    {
        HIP_TRY((c.epi == EPI_F32 ? transpose_words_launch : transpose_bytes_launch)(Dd, Dfinal, d.batch, h->geom.OH * h->geom.OW, c.N, s));
        Dd = Dfinal;
    }
    if (d_pad)
    {
        HIP_TRY(restride_nd_launch(Dd, Dpadded, dt.seg, dt.n1, dt.n2, dt.n3, dt.dense, dt.given, s));
        Dd = Dpadded;
    }
    if (d_host)
    {
        HIP_TRY(hipMemcpyAsync(dst, Dd, dst_ext, hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
    }
    else if (!h->kindSrc.is_device(src))
        HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

void mi355_conv_destroy(mi355_conv_handle *h)
{
    if (!h)
        return;
    h->core.release();
    h->stageSrc.release(), h->stageW.release(), h->stageDst.release(), h->stageBias.release();
    h->stageMult.release(), h->stageShift.release(), h->cols.release();
    h->nhwcSrc.release(), h->nhwcW.release(), h->nhwcDst.release(), h->biasF.release();
    h->denseSrc.release(), h->denseW.release(), h->denseDst.release(), h->padSrc.release(), h->padW.release();
    delete h;
}

const char *mi355_conv_kernel_name(const mi355_conv_handle *h)
{
    return h ? h->core.name() : "";
}

int mi355_im2col_nhwc_run(const mi355_conv_desc *desc, const void *src, void *dst, void *stream)
{
    if (!desc || !src || !dst)
        return fail("null argument");
    const mi355_conv_desc &d = *desc;
    TRY(conv_check(d));
    if (d.layout != MI355_NHWC)
        return fail("mi355_im2col_nhwc_run lowers NHWC tensors only");
    ConvGeom g{};
    conv_geom(d, g);
    g.pad_word      = ((uint32_t)d.pad_value & 0xFFu) * 0x01010101u;
    hipStream_t s   = (hipStream_t)stream;
    const size_t K  = (size_t)d.KH * d.KW * d.C, rows = (size_t)d.batch * g.OH * g.OW;
    DevBuf       sSrc, sDst;
    const void  *srcd;
    void        *Dd     = dst;
    const bool   d_host = !is_device_ptr(dst);
    auto         body   = [&]() -> int
    {
        TRY(to_device(src, (size_t)d.batch * d.H * d.W * d.C, sSrc, s, &srcd));
        if (d_host)
        {
            TRY(sDst.ensure(rows * K));
            Dd = sDst.p;
        }
        HIP_TRY(im2col_nhwc_launch(srcd, Dd, d.batch, g, (int64_t)K, s));
        if (d_host)
            HIP_TRY(hipMemcpyAsync(dst, Dd, rows * K, hipMemcpyDeviceToHost, s));
        if (d_host || srcd != src)
            HIP_TRY(hipStreamSynchronize(s));
        return 0;
    };
    const int rc = body();
    sSrc.release(), sDst.release();
    return rc;
}
} // extern "C"

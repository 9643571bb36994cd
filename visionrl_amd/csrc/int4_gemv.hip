// int4 weight-only decode linears for MI355X (gfx950 / CDNA4).
//
// Replaces the bf16 nn.Linear calls of the rollout decode step that the
// reference reaches at vrl/models/families/janus_pro/policy.py:673-678 (Llama
// trunk projections) and policy.py:138-160 (gen_head).  Operand formats and the
// arithmetic contract are stated in include/vrl_int4.h.
//
// Kernels
//   dequant_kernel        packed int4 -> bf16 [N,K], bit-exact, write-bound.
//   gemv_tile_kernel      the hot path.  A workgroup owns TILE_ROWS weight rows;
//                         its waves split K in 128-wide chunks.  Each lane
//                         streams 16-byte pieces of "its" row (lane%16) with
//                         global_load_dwordx4, rebuilds the exactly rounded bf16
//                         weights in registers and feeds them to
//                         v_mfma_f32_16x16x32_bf16 as the B operand; the
//                         activations are staged once per workgroup in LDS (in
//                         the k-order the unpack produces) and read as the A
//                         operand.  Partial sums of the K split meet in LDS.
//   gemv_generic_kernel   any legal shape (K%8, G%8): one wave per row, VALU
//                         dot product, DPP/shuffle reduction.  Correctness
//                         fallback for shapes the tile kernel does not take.
//
// In-register dequant, exact by construction: nibble pairs (i, i+4) of a packed
// word are turned into two bf16 numbers 128+q with one shift and one and-or
// ((v >> 4i) & 0x000F000F | 0x43004300), then
//   v_dot2_f32_bf16(pair, (s,0) or (0,s), c)   with  c = -(128+z)*s  (fp32, exact)
// gives (q-z)*s exactly (16-bit products, 12-bit result), and
// v_cvt_pk_bf16_f32 applies the one round-to-nearest-even the contract asks for.
//
// Source layout: common.hpp (types, bf16 helpers, the problem record), canonical.hpp (kernels over the
// canonical triple), prepacked.hpp (repack, stream and latency kernels over the MFMA-shaped blob),
// stream_kernel.hpp (the grouped stream kernel that dispatches to both halves), this file (plan building,
// launchers, the C ABI).

#include <atomic>

#include "stream_kernel.hpp"
#include "rows32.hpp"

namespace {

// -------------------------------------------------------------------------
// host side
// -------------------------------------------------------------------------
constexpr int TILE_WPB = 8;
constexpr int MAX_TILE_M = 16;                  // activation rows one single-launch slab / canonical record takes
constexpr int MAX_PP_M = 32;                    // activation rows a prepacked record of a grouped plan takes
constexpr size_t LDS_X_BUDGET = 40 * 1024;      // split kernel: staged activations per workgroup
constexpr int STAGE_STEP = KCHUNK * TILE_WPB;   // split kernel: shorter staged extents are multiples of this
// stream kernel: workgroup shapes by the LDS the staged activations need
struct StreamShape { int wpb; int per_cu; size_t lds; };
// {waves per workgroup, workgroups per CU to launch when the runtime cannot say how many are
// resident, LDS the shape may use}
constexpr StreamShape STREAM_SHAPES[3] = {{4, 15, 32 * 1024}, {8, 2, 72 * 1024}, {16, 1, 144 * 1024}};
constexpr size_t LDS_PER_CU = 160 * 1024;
constexpr size_t STREAM_LDS_CAP = LDS_PER_CU - 1024;   // dynamic LDS a grouped launch may ask for (the kernels hold a few static words)
constexpr size_t DIRECT_LDS_CAP = 150 * 1024;   // plan-free launches: staged activations + partial tiles

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_problem(const void *x, const void *qw, const void *sc, const void *qz, const void *y,
                  long M, long N, long K, long G) {
    if (!x || !qw || !sc || !qz || !y) return VRL_INT4_ENULL;
    if (M < 1 || N < 1 || K < 8 || G < 8) return VRL_INT4_ESHAPE;
    if (K % 8 != 0 || G % 8 != 0 || K % G != 0) return VRL_INT4_ESHAPE;
    if (N * K >= (1L << 40) || M * K >= (1L << 31) || M * N >= (1L << 31)) return VRL_INT4_ESHAPE;
    if (!aligned16(x) || !aligned16(qw) || !aligned16(sc) || !aligned16(qz) || !aligned16(y))
        return VRL_INT4_EALIGN;
    return VRL_INT4_OK;
}

bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

// shapes the MFMA kernels take; everything else goes to the generic kernel
bool tile_path_ok(const DevProblem &p) {
    return p.K % KCHUNK == 0 && p.G % 32 == 0 && pow2(p.G) && p.M <= (p.prepacked ? MAX_PP_M : MAX_TILE_M);
}

// split kernel: k extent of x staged per pass, all of K when M rows of it fit the budget,
// else the largest multiple of STAGE_STEP that does (M <= 16 always fits one step)
int staged_k(int M, int K) {
    if ((size_t)M * (K + XPAD) * 2 <= LDS_X_BUDGET) return K;
    long kc = (long)(LDS_X_BUDGET / ((size_t)M * 2)) - XPAD;
    kc -= kc % STAGE_STEP;
    if (kc < STAGE_STEP) kc = STAGE_STEP;
    return (int)(kc < K ? kc : K);
}

// stream kernel, canonical records: all of K if it fits `lds`, else passes that are multiples of KCHUNK
int stream_staged_k(int M, int K, size_t lds) {
    if ((size_t)M * (K + XPAD) * 2 <= lds) return K;
    long kc = (long)(lds / ((size_t)M * 2)) - XPAD;
    kc -= kc % KCHUNK;
    if (kc < KCHUNK) kc = KCHUNK;
    return (int)(kc < K ? kc : K);
}

// prepacked blobs exist for group sizes 32, 64 and 128
// the stream kernel addresses a blob with 32-bit byte offsets, so a blob stays below 2 GiB
bool prepack_ok(long N, long K, long G) {
    if ((G != 128 && G != 64 && G != 32) || K % 128 != 0 || N < 1 || K < 128 || N * K >= (1L << 40)) return false;
    return ((N + 15) / 16) * pp_tile_u4((int)K, (int)G) * 16 < (long)PP_OUT_OF_RANGE;
}

// stream kernel, prepacked records: all of the padded K if it fits, else whole super-chunks per pass
int pp_staged_k(int M, int K, size_t lds) {
    const int kpad = pp_nsc(K) * PP_SC;
    if ((size_t)M * (kpad + XPAD) * 2 <= lds) return kpad;
    long kc = (long)(lds / ((size_t)M * 2)) - XPAD;
    kc -= kc % PP_SC;
    if (kc < PP_SC) kc = PP_SC;
    return (int)kc;
}

template <int R, int MB>
size_t tile_smem_bytes(int M, int kc) {
    const size_t xbytes = (size_t)M * (kc + XPAD) * 2;
    const size_t rbytes = (size_t)TileCfg<R, MB, TILE_WPB>::RED_FLOATS * 4;
    return xbytes > rbytes ? xbytes : rbytes;
}

int device_cu_count() {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            cus = v;
    }
    return cus;
}

template <int R, int MB>
int launch_tile(const DevProblem &p, hipStream_t stream) {
    const int out_cols = p.fused ? p.N / 2 : p.N;
    const int cols_per_tile = p.fused ? 16 * (R / 2) : 16 * R;
    const int tiles = (out_cols + cols_per_tile - 1) / cols_per_tile;
    const size_t smem = tile_smem_bytes<R, MB>(p.M, p.kc);
    return vrl_launch(&gemv_tile_kernel<R, MB, TILE_WPB>, dim3(tiles), dim3(TILE_WPB * WAVE), smem,
                       stream, p);
}

int launch_problem(DevProblem p, hipStream_t stream) {
    const int out_cols = p.fused ? p.N / 2 : p.N;
    if (!tile_path_ok(p)) {
        // the generic kernel walks activation rows itself, any M
        const int waves = 4;
        return vrl_launch(&gemv_generic_kernel, dim3((out_cols + waves - 1) / waves),
                           dim3(waves * WAVE), 0, stream, p);
    }
    p.kc = staged_k(p.M, p.K);
    // widest tile that still gives every CU two workgroups; narrow tiles otherwise
    const int cus = device_cu_count();
    const int cols_r4 = p.fused ? 32 : 64;
    if ((out_cols + cols_r4 - 1) / cols_r4 >= 2 * cus) return launch_tile<4, 1>(p, stream);
    if (p.fused || (out_cols + 31) / 32 >= 2 * cus) return launch_tile<2, 1>(p, stream);
    return launch_tile<1, 1>(p, stream);
}

int run_rows(const void *x, const void *qw, const void *sc, const void *qz, void *y, int M, int N,
             int K, int G, int fused, void *hip_stream) {
    int rc = check_problem(x, qw, sc, qz, y, M, N, K, G);
    if (rc != VRL_INT4_OK) return rc;
    if (fused && (N % 2 != 0)) return VRL_INT4_ESHAPE;
    const int out_cols = fused ? N / 2 : N;
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    // activation rows go in slabs of MAX_TILE_M (weights are re-read per slab)
    for (int m0 = 0; m0 < M; m0 += MAX_TILE_M) {
        DevProblem p;
        memset(&p, 0, sizeof p);
        p.x = static_cast<const uint16_t *>(x) + (long)m0 * K;
        p.qweight = static_cast<const uint32_t *>(qw);
        p.scales = static_cast<const uint16_t *>(sc);
        p.qzeros = static_cast<const uint32_t *>(qz);
        p.y = static_cast<uint16_t *>(y) + (long)m0 * out_cols;
        p.M = (M - m0 < MAX_TILE_M) ? (M - m0) : MAX_TILE_M;
        p.N = N;
        p.K = K;
        p.G = G;
        p.fused = fused;
        rc = launch_problem(p, stream);
        if (rc != 0) return rc;
    }
    return VRL_INT4_OK;
}

// Plan blob: [PlanHeader][DevProblem x n_records][int2 {first tile, its record} x (MAX_PLAN_GRID + 1)]
struct PlanHeader {
    uint32_t magic;
    int32_t n_records;
    int32_t total_tiles;
    int32_t grid;
};
static_assert(sizeof(PlanHeader) == 16, "plan header is 16 bytes");
constexpr uint32_t PLAN_MAGIC = 0x34544956u;  // "VIT4"
constexpr int MAX_PLAN_GRID = 4096;

// With recs == nullptr nothing is launched: info->grid receives the number of workgroups of
// this build that one CU holds at info->lds_bytes (the plan builder sizes the grid with it).
template <int WPB, int MB, bool CANON, bool PP, bool FUSED, bool PASSES, int GQ = 1>
int launch_stream(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *block_begin,
                  hipStream_t stream) {
    auto kernel = &gemv_stream_kernel<WPB, MB, CANON, PP, FUSED, PASSES, GQ>;
    if (info->lds_bytes > 64 * 1024) {
        // once per instantiation and device (the attribute belongs to the function on that device), at the
        // largest size a plan may ask for: no runtime call in a timed or captured launch after the first
        static std::atomic<uint64_t> raised{0};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) dev = 0;
        const uint64_t bit = 1ull << (dev & 63);
        if (!(raised.load(std::memory_order_relaxed) & bit)) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)STREAM_LDS_CAP);
            if (e != hipSuccess) return (int)e;
            raised.fetch_or(bit, std::memory_order_relaxed);
        }
    }
    if (!recs) {
        int per_cu = 0;
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &per_cu, reinterpret_cast<const void *>(kernel), WPB * WAVE, (size_t)info->lds_bytes);
        if (e != hipSuccess) return (int)e;
        info->grid = per_cu;
        return VRL_INT4_OK;
    }
    return vrl_launch(kernel, dim3(info->grid), dim3(WPB * WAVE), (size_t)info->lds_bytes,
                       stream, recs, block_begin, info->n_problems);
}

// prepacked-only plans: fused or not, staged passes or not (only the widest workgroups ever
// need passes: narrower shapes are chosen because x fits), group size
template <int WPB, int MB, bool FUSED, int GQ>
int launch_stream_pp_g(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *bb, hipStream_t stream,
                       bool passes) {
    if constexpr (WPB == 16) {
        if (passes) return launch_stream<WPB, MB, false, true, FUSED, true, GQ>(info, recs, bb, stream);
    }
    return launch_stream<WPB, MB, false, true, FUSED, false, GQ>(info, recs, bb, stream);
}

template <int WPB, int MB>
int launch_stream_pp(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *bb, hipStream_t stream,
                     bool fused, bool passes, int gq) {
    if (fused) {
        if (gq == 1) return launch_stream_pp_g<WPB, MB, true, 1>(info, recs, bb, stream, passes);
        if (gq == 2) return launch_stream_pp_g<WPB, MB, true, 2>(info, recs, bb, stream, passes);
        return launch_stream_pp_g<WPB, MB, true, 4>(info, recs, bb, stream, passes);
    }
    if (gq == 1) return launch_stream_pp_g<WPB, MB, false, 1>(info, recs, bb, stream, passes);
    if (gq == 2) return launch_stream_pp_g<WPB, MB, false, 2>(info, recs, bb, stream, passes);
    return launch_stream_pp_g<WPB, MB, false, 4>(info, recs, bb, stream, passes);
}

// which record kinds a kernel build must handle, for a given workgroup shape
template <int WPB, int MB>
int launch_stream_variant(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *bb,
                          hipStream_t stream) {
    const int v = info->variant & (VARIANT_CANON | VARIANT_PP | VARIANT_FUSED);
    const bool passes = (info->variant & VARIANT_PASSES) != 0;
    // prepacked-only plans hold one group size (the kernel build is specialised for it)
    const int gq = (info->variant & VARIANT_G32) ? 4 : ((info->variant & VARIANT_G64) ? 2 : 1);
    if (v == VARIANT_PP || v == (VARIANT_PP | VARIANT_FUSED)) {
        return launch_stream_pp<WPB, MB>(info, recs, bb, stream, (v & VARIANT_FUSED) != 0, passes, gq);
    }
    if (gq != 1) return VRL_INT4_EPLAN;
    if constexpr (MB == 1 && WPB != 8) {  // canonical records: narrow and widest workgroups only
        if (v & VARIANT_FUSED) return launch_stream<WPB, 1, true, true, true, WPB == 16>(info, recs, bb, stream);
        return launch_stream<WPB, 1, true, true, false, WPB == 16>(info, recs, bb, stream);
    }
    return VRL_INT4_EPLAN;
}


template <bool FUSED, int WPB>
int launch_split(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *block_tab, hipStream_t stream) {
    auto kernel = &gemv_split_kernel<FUSED, WPB>;
    if (!recs) {
        int per_cu = 0;
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &per_cu, reinterpret_cast<const void *>(kernel), WPB * WAVE, (size_t)info->lds_bytes);
        if (e != hipSuccess) return (int)e;
        info->grid = per_cu;
        return VRL_INT4_OK;
    }
    return vrl_launch(kernel, dim3(info->grid), dim3(WPB * WAVE), (size_t)info->lds_bytes, stream, recs,
                       block_tab, info->n_problems);
}

template <int WPB>
int launch_split_variant(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *block_tab,
                         hipStream_t stream) {
    return (info->variant & VARIANT_FUSED) ? launch_split<true, WPB>(info, recs, block_tab, stream)
                                           : launch_split<false, WPB>(info, recs, block_tab, stream);
}

template <bool FUSED, int KS, int TW, bool NORM, bool XG = false, bool LD = false, bool UP = false, bool EPI = false>
int launch_direct(const DirectArgs &args, int workgroups, size_t lds, hipStream_t stream) {
    auto kernel = &gemv_split_direct_kernel<FUSED, KS, TW, NORM, XG, LD, UP, EPI>;
    if (lds > 64 * 1024) {
        // once per instantiation and device: the attribute belongs to the function on that device
        static std::atomic<uint64_t> raised{0};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) dev = 0;
        const uint64_t bit = 1ull << (dev & 63);
        if (!(raised.load(std::memory_order_relaxed) & bit)) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)DIRECT_LDS_CAP);
            if (e != hipSuccess) return (int)e;
            raised.fetch_or(bit, std::memory_order_relaxed);
        }
    }
    return vrl_launch(kernel, dim3(workgroups), dim3(KS * TW * WAVE), lds, stream, args);
}

template <bool FUSED, bool NORM>
int launch_direct_shape(const DirectArgs &args, int ks, int tw, bool xg, int workgroups, size_t lds,
                        hipStream_t stream) {
    if constexpr (!NORM) {
        if constexpr (!FUSED) {
            if (xg && ks == 16) return launch_direct<false, 16, 1, false, true>(args, workgroups, lds, stream);
        }
        if (xg && ks == 16) return VRL_INT4_EPLAN;
        if (xg && ks == 8) return launch_direct<FUSED, 8, 1, false, true>(args, workgroups, lds, stream);
        if (xg) return launch_direct<FUSED, 4, 1, false, true>(args, workgroups, lds, stream);
    }
    if (ks == 4 && tw == 1) return launch_direct<FUSED, 4, 1, NORM>(args, workgroups, lds, stream);
    if (ks == 4 && tw == 2) return launch_direct<FUSED, 4, 2, NORM>(args, workgroups, lds, stream);
    if (ks == 4 && tw == 4) return launch_direct<FUSED, 4, 4, NORM>(args, workgroups, lds, stream);
    if (ks == 8 && tw == 1) return launch_direct<FUSED, 8, 1, NORM>(args, workgroups, lds, stream);
    if (ks == 8 && tw == 2) return launch_direct<FUSED, 8, 2, NORM>(args, workgroups, lds, stream);
    if (ks == 16 && tw == 1) return launch_direct<FUSED, 16, 1, NORM>(args, workgroups, lds, stream);
    return VRL_INT4_EPLAN;
}

// records of 17 to 32 rows: four waves per tile, four tiles per workgroup
constexpr size_t ROWS32_LDS_CAP = 160 * 1024;
template <bool FUSED, int KS, int TW, int MB>
int launch_rows32(const DirectArgs &args, int workgroups, size_t lds, hipStream_t stream) {
    auto kernel = &gemv_rows32_direct_kernel<FUSED, KS, TW, MB>;
    static std::atomic<uint64_t> raised{0};   // once per instantiation and device
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    const uint64_t bit = 1ull << (dev & 63);
    if (!(raised.load(std::memory_order_relaxed) & bit)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)ROWS32_LDS_CAP);
        if (e != hipSuccess) return (int)e;
        raised.fetch_or(bit, std::memory_order_relaxed);
    }
    return vrl_launch(kernel, dim3(workgroups), dim3(KS * TW * WAVE), lds, stream, args);
}

// with bias, activation or residual applied before the store: one plain problem
template <bool NORM>
int launch_direct_epilogue(const DirectArgs &args, int ks, int tw, bool xg, int workgroups, size_t lds,
                           hipStream_t stream) {
    if constexpr (!NORM) {
        if (xg && ks == 16) return launch_direct<false, 16, 1, false, true, false, false, true>(args, workgroups, lds, stream);
        if (xg && ks == 8) return launch_direct<false, 8, 1, false, true, false, false, true>(args, workgroups, lds, stream);
        if (xg) return launch_direct<false, 4, 1, false, true, false, false, true>(args, workgroups, lds, stream);
    }
    if (ks == 4 && tw == 1) return launch_direct<false, 4, 1, NORM, false, false, false, true>(args, workgroups, lds, stream);
    if (ks == 4 && tw == 2) return launch_direct<false, 4, 2, NORM, false, false, false, true>(args, workgroups, lds, stream);
    if (ks == 4 && tw == 4) return launch_direct<false, 4, 4, NORM, false, false, false, true>(args, workgroups, lds, stream);
    if (ks == 8 && tw == 1) return launch_direct<false, 8, 1, NORM, false, false, false, true>(args, workgroups, lds, stream);
    if (ks == 8 && tw == 2) return launch_direct<false, 8, 2, NORM, false, false, false, true>(args, workgroups, lds, stream);
    if (ks == 16 && tw == 1) return launch_direct<false, 16, 1, NORM, false, false, false, true>(args, workgroups, lds, stream);
    return VRL_INT4_EPLAN;
}

// with an adapter's up-projection added before the store: one plain problem, one tile per workgroup
int launch_direct_up(const DirectArgs &args, int ks, bool xg, int workgroups, size_t lds, hipStream_t stream) {
    if (ks == 4) return xg ? launch_direct<false, 4, 1, false, true, false, true>(args, workgroups, lds, stream)
                           : launch_direct<false, 4, 1, false, false, false, true>(args, workgroups, lds, stream);
    if (ks == 8) return xg ? launch_direct<false, 8, 1, false, true, false, true>(args, workgroups, lds, stream)
                           : launch_direct<false, 8, 1, false, false, false, true>(args, workgroups, lds, stream);
    if (xg) return VRL_INT4_EPLAN;   // never chosen: see the choice of xg in direct_launch
    return launch_direct<false, 16, 1, false, false, false, true>(args, workgroups, lds, stream);
}

// with the adapters' down-projection as extra workgroups: plain (staged, unfused) problems only
int launch_direct_lora(const DirectArgs &args, int ks, int tw, int workgroups, size_t lds, hipStream_t stream) {
    if (ks == 4 && tw == 1) return launch_direct<false, 4, 1, false, false, true>(args, workgroups, lds, stream);
    if (ks == 4 && tw == 2) return launch_direct<false, 4, 2, false, false, true>(args, workgroups, lds, stream);
    if (ks == 4 && tw == 4) return launch_direct<false, 4, 4, false, false, true>(args, workgroups, lds, stream);
    if (ks == 8 && tw == 1) return launch_direct<false, 8, 1, false, false, true>(args, workgroups, lds, stream);
    if (ks == 8 && tw == 2) return launch_direct<false, 8, 2, false, false, true>(args, workgroups, lds, stream);
    if (ks == 16 && tw == 1) return launch_direct<false, 16, 1, false, false, true>(args, workgroups, lds, stream);
    return VRL_INT4_EPLAN;
}

// the same with residual add and RMSNorm applied to the shared input (rows of up to 2048 values: four waves per tile)
int launch_direct_lora_norm(const DirectArgs &args, int ks, int tw, int workgroups, size_t lds, hipStream_t stream) {
    if (ks == 4 && tw == 1) return launch_direct<false, 4, 1, true, false, true>(args, workgroups, lds, stream);
    if (ks == 4 && tw == 2) return launch_direct<false, 4, 2, true, false, true>(args, workgroups, lds, stream);
    return VRL_INT4_EPLAN;   // (sixteen-wave workgroups leave the adapters' rows too few registers: not built)
}

int dispatch_stream(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *block_tab,
                    hipStream_t stream) {
    const bool mb2 = (info->variant & VARIANT_MB2) != 0;
    if (info->variant & VARIANT_SPLIT) {
        if (mb2 || (size_t)info->lds_bytes > 64 * 1024 || (info->variant & (VARIANT_CANON | VARIANT_PASSES)))
            return VRL_INT4_EPLAN;
        switch (info->block_threads) {
            case 4 * WAVE: return launch_split_variant<4>(info, recs, block_tab, stream);
            case 8 * WAVE: return launch_split_variant<8>(info, recs, block_tab, stream);
            case 16 * WAVE: return launch_split_variant<16>(info, recs, block_tab, stream);
            default: return VRL_INT4_EPLAN;
        }
    }
    switch (info->block_threads) {
        case 4 * WAVE: return mb2 ? VRL_INT4_EPLAN : launch_stream_variant<4, 1>(info, recs, block_tab, stream);
        case 8 * WAVE: return mb2 ? VRL_INT4_EPLAN : launch_stream_variant<8, 1>(info, recs, block_tab, stream);
        case 16 * WAVE:
            return mb2 ? launch_stream_variant<16, 2>(info, recs, block_tab, stream)
                       : launch_stream_variant<16, 1>(info, recs, block_tab, stream);
        default: return VRL_INT4_EPLAN;
    }
}

size_t plan_bytes_for(int n_records) {
    return sizeof(PlanHeader) + (size_t)n_records * sizeof(DevProblem) +
           (size_t)(MAX_PLAN_GRID + 1) * sizeof(int2);
}

}  // namespace

extern "C" {

int vrl_int4_abi_version(void) { return VRL_INT4_ABI_VERSION; }

const char *vrl_int4_error_string(int code) {
    switch (code) {
        case VRL_INT4_OK: return "ok";
        case VRL_INT4_ESHAPE: return "shape violates a precondition (M,N>=1; K%8==0; G%8==0; K%G==0)";
        case VRL_INT4_EALIGN: return "pointer is not 16-byte aligned";
        case VRL_INT4_ENULL: return "required pointer is NULL";
        case VRL_INT4_EPLAN: return "malformed or undersized grouped plan";
        case VRL_INT4_ELIMIT: return "beyond the fixed size of the library's own scratch memory";
        default: break;
    }
    if (code > 0 && code < 1000) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error code";
}

int vrl_int4_gemv_bf16(const void *x, const void *qweight, const void *scales, const void *qzeros,
                       void *y, int M, int N, int K, int G, void *hip_stream) {
    return run_rows(x, qweight, scales, qzeros, y, M, N, K, G, 0, hip_stream);
}

int vrl_int4_gate_up_silu_bf16(const void *x, const void *qweight_gu, const void *scales_gu,
                               const void *qzeros_gu, void *y, int M, int I, int K, int G,
                               void *hip_stream) {
    if (I < 1 || I > (1 << 29)) return VRL_INT4_ESHAPE;
    return run_rows(x, qweight_gu, scales_gu, qzeros_gu, y, M, 2 * I, K, G, 1, hip_stream);
}

int vrl_int4_dequant_bf16(const void *qweight, const void *scales, const void *qzeros, void *w,
                          int N, int K, int G, void *hip_stream) {
    int rc = check_problem(qweight, qweight, scales, qzeros, w, 1, N, K, G);
    if (rc != VRL_INT4_OK) return rc;
    const long total = (long)N * (K >> 3);
    long blocks = (total + 255) / 256;
    const long cap = (long)device_cu_count() * 32;
    if (blocks > cap) blocks = cap;
    return vrl_launch(&dequant_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(hip_stream),
                       static_cast<const uint32_t *>(qweight), static_cast<const uint16_t *>(scales),
                       static_cast<const uint32_t *>(qzeros), static_cast<uint16_t *>(w), N, K, G);
}

size_t vrl_int4_prepacked_bytes(int N, int K, int G) {
    if (!prepack_ok(N, K, G)) return 0;
    return (size_t)((N + 15) / 16) * (size_t)pp_tile_u4(K, G) * 16;
}

int vrl_int4_prepack(const void *qweight, const void *scales, const void *qzeros, void *packed,
                     int N, int K, int G, void *hip_stream) {
    int rc = check_problem(qweight, qweight, scales, qzeros, packed, 1, N, K, G);
    if (rc != VRL_INT4_OK) return rc;
    if (!prepack_ok(N, K, G)) return VRL_INT4_ESHAPE;
    const long total = (long)((N + 15) / 16) * pp_tile_u4(K, G);
    long blocks = (total + 255) / 256;
    const long cap = (long)device_cu_count() * 32;
    if (blocks > cap) blocks = cap;
    return vrl_launch(&prepack_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(hip_stream),
                       static_cast<const uint32_t *>(qweight), static_cast<const uint16_t *>(scales),
                       static_cast<const uint32_t *>(qzeros), static_cast<u32x4_t *>(packed), N, K, G);
}

struct DirectLora {   // adapters joined to a plan-free launch: down-projections (up false) or one up-projection
    const vrl_lora_adapter *adapters;
    int n_adapters;
    float *t;
    bool up;
    int t_parts;
};

static int direct_launch(const vrl_int4_problem *problems, int n_problems, const vrl_int4_norm *norm,
                         const DirectLora *lora, void *hip_stream, const vrl_int4_epilogue *epilogue = nullptr) {
    if (!problems) return VRL_INT4_ENULL;
    if (n_problems < 1 || n_problems > DIRECT_MAX) return VRL_INT4_ESHAPE;
    if (epilogue) {   // one plain problem: the bias belongs to its columns
        if (n_problems != 1 || problems[0].fused_gate_up || lora) return VRL_INT4_ESHAPE;
        if (epilogue->activation != VRL_INT4_ACT_NONE && epilogue->activation != VRL_INT4_ACT_GELU) return VRL_INT4_ESHAPE;
        if ((reinterpret_cast<uintptr_t>(epilogue->bias) | reinterpret_cast<uintptr_t>(epilogue->residual)) & 1u)
            return VRL_INT4_EALIGN;
    }
    bool fused_any = false;
    int max_nsc = 1, max_m = 1;
    long slab_tiles = 0;  // 16-column tiles x 16-row slabs of the launch
    for (int i = 0; i < n_problems; ++i) {
        const vrl_int4_problem &q = problems[i];
        if (!q.prepacked) return VRL_INT4_ESHAPE;
        int rc = check_problem(q.x, q.qweight, q.qweight, q.qweight, q.y, q.M, q.N, q.K, q.G);
        if (rc != VRL_INT4_OK) return rc;
        if (!prepack_ok(q.N, q.K, q.G)) return VRL_INT4_ESHAPE;
        if (q.fused_gate_up && (q.N % 2 != 0 || (q.N / 2) % 16 != 0)) return VRL_INT4_ESHAPE;
        fused_any |= q.fused_gate_up != 0;
        max_nsc = std::max(max_nsc, pp_nsc(q.K));
        max_m = std::max(max_m, q.M);
        slab_tiles += (long)(((q.fused_gate_up ? q.N / 2 : q.N) + 15) / 16) * ((q.M + MAX_TILE_M - 1) / MAX_TILE_M);
    }
    // KS waves split K of a tile (one super-chunk each where K allows); with 8 or more
    // activation rows a workgroup carries several tiles so that one staging of x serves them
    int ks = max_nsc > 8 ? 16 : (max_nsc > 4 ? 8 : 4);
    // The waves can fetch their own activations, with nothing staged and one tile per workgroup.  Long K
    // does with one super-chunk per wave, and with two when staging would need more than one slab of
    // rows (the second fetch waits for the first super-chunk's arithmetic); shorter K with 8+ rows and one
    // super-chunk per wave does while the launch is small (every tile then fetches its rows from L2
    // itself: for a wide matrix one staging per TW tiles wins).
    const bool lora_up = lora && lora->up, lora_down = lora && !lora->up;
    // rows of the longest K that LDS holds beside a 16-wave workgroup's partial tiles
    const long staged_rows = (long)((DIRECT_LDS_CAP - (size_t)15 * (fused_any ? 2 : 1) * WAVE * sizeof(f32x4_t)) /
                                    ((size_t)(max_nsc * PP_SC + XPAD) * 2));
    // (the 16-wave register-fed form is not built for fused gate|up records or with an adapter's up-projection:
    // its accumulators and operands did not fit the registers, and the staged form serves those launches)
    bool xg = !norm && !lora_down &&
              (ks == 16 ? !fused_any && !lora_up && (max_nsc <= ks || (max_nsc <= 2 * ks && max_m > staged_rows))
                        : max_nsc <= ks && max_m >= 8 && slab_tiles <= 2L * device_cu_count());
    // Tiles per workgroup.  One staging of x serves them, but fewer workgroups share the launch: up to 16 rows
    // of a launch with many tiles (q|k|v, gate|up) two tiles per workgroup measured best at every row count
    // (K = 2048, 384 tiles, fused norm: 5.9 / 6.5 / 7.8 us at 2 / 8 / 16 rows against 6.1 / 7.9 / 10.9 us with one
    // and 7.1 / 8.0 / 8.7 us with four; K = 4096, 768 tiles: 10.3 / 12.4 / 13.9 against 11.3 / 14.1 / 25.0 us with
    // one), except that fused records of 12 or more rows of K > 2048 fill LDS with one workgroup per CU
    // either way and then three sets of one tile beat two sets of two (688 tiles: 18.9 against 26.0 us).  With
    // few tiles (o_proj: 128 or 256) one tile per workgroup below 8 rows (4.2 against 4.9 us at 2 rows).
    int tw = (max_m >= 8 && !xg && !lora_up) ? 16 / ks : 1;
    const bool many_tiles = slab_tiles >= 5L * device_cu_count() / 4;
    if (norm && lora_down && tw > 2) tw = 2;   // the build of that launch with four tiles per workgroup spills
    if (!xg && !lora_up && max_m <= MAX_TILE_M && ks <= 8 && many_tiles)
        tw = (ks == 8 && fused_any && max_m >= 12) ? 1 : 2;
    // Three more measured preferences, all about how the rows get into LDS.  A register-fed wave asks for its
    // rows' fragments sixteen bytes at a time, one cache line per lane and instruction: with 8 or more rows that
    // is slower than staging with coalesced loads, where LDS holds the rows in one or two slabs (K = 5632,
    // N = 2048: 6.9 / 7.7 us staged against 7.8 / 9.9 us register-fed at 8 / 16 rows; a tie at 2 to 4 rows).
    if (xg && ks == 16 && !lora_up && max_m >= 6 && max_m <= MAX_TILE_M && max_nsc <= 16 && max_m <= 2 * staged_rows)
        xg = false;
    // Staging is shared by all waves of a workgroup, so few tiles of short K are served faster by sixteen waves
    // of which only the first few stream (K = 2048, N = 2048 at 4 / 8 / 16 rows: 4.6 / 4.8 / 5.2 against 5.0 /
    // 5.0 / 5.3 us; K = 4096, N = 4096 at 8 / 16 rows: 6.3 / 7.3 against 6.8 / 8.2 us register-fed).
    if (!norm && !lora && !fused_any && !many_tiles && ks <= 8 && max_m >= 4 && max_m <= MAX_TILE_M &&
        max_m <= staged_rows) {
        ks = 16;
        tw = 1;
        xg = false;
    }
    // A normalising launch over rows of 2049 to 4096 values: four waves per tile (two super-chunks each) and four
    // tiles per workgroup up to 8 rows (768 tiles: 10.2 / 10.8 / 11.9 us at 2 / 4 / 8 rows against 10.9 / 11.3 /
    // 12.5 us; 688 fused tiles: 15.3 / 16.4 / 17.5 against 16.5 / 17.7 / 18.9 us), and for plain records up to 16
    // (13.5 against 14.1 us); rows of up to 2048 values at 13 to 16 rows: eight waves per tile, half of them
    // streaming (384 tiles: 7.6 against 8.0 us; 352 fused tiles: 9.7 against 10.2 us).
    // At 17 to 32 rows (two slabs): 17.9 against 29.8 us for 768 tiles, and four waves per tile with two tiles per
    // workgroup for fused records (688 tiles: 27.5 against 38.3 us).
    if (norm && !lora && many_tiles) {
        if (ks == 8 && (max_m <= 8 || !fused_any)) ks = 4, tw = 4;
        else if (ks == 8 && max_m > MAX_TILE_M) ks = 4, tw = 2;
        else if (ks == 4 && max_m > 12) ks = 8, tw = 2;   // also two slabs: 9.2 against 9.4 us, fused 12.2 against 12.7
    }
    // Long K at 17 to 32 rows, register-fed: four waves per tile that walk three super-chunks each leave the CU's
    // L1 fewer fragment requests at a time than sixteen waves with one (K = 5632, N = 2048: 9.2 against 9.9 us).
    if (xg && ks == 16 && max_m > MAX_TILE_M && max_nsc <= 12 && !lora) ks = 4;
    // Few tiles of 17 to 32 rows of K up to 4096 with an epilogue (the passes over K above serve plain launches):
    // staged, two tiles per workgroup, against register-fed slabs 8.5 against 13.1 us (K = 4096, N = 4096).
    if (xg && ks == 8 && max_m > MAX_TILE_M && !lora && MAX_TILE_M <= staged_rows) xg = false, tw = 2;
    const size_t red = (size_t)tw * (ks - 1) * (fused_any ? 2 : 1) * WAVE * sizeof(f32x4_t);
    // activations go in slabs of at most 16 rows that fit LDS beside the partial tiles; one record per slab
    DirectArgs args;
    memset(&args, 0, sizeof args);
    if (norm) {
        // one normalised input for every problem of the launch: same rows, same K, x is the un-normed tensor
        const vrl_int4_problem &q0 = problems[0];
        if (!norm->x || !norm->weight) return VRL_INT4_ENULL;
        if (q0.K > NORM_MAX_K || !(norm->eps >= 0.0f)) return VRL_INT4_ESHAPE;
        for (int i = 0; i < n_problems; ++i)
            if (problems[i].x != norm->x || problems[i].M != q0.M || problems[i].K != q0.K) return VRL_INT4_ESHAPE;
        if (norm->h_out && (norm->h_out == norm->x || norm->h_out == norm->residual)) return VRL_INT4_ESHAPE;
        if ((reinterpret_cast<uintptr_t>(norm->residual) | reinterpret_cast<uintptr_t>(norm->weight) |
             reinterpret_cast<uintptr_t>(norm->h_out)) & 15u)
            return VRL_INT4_EALIGN;
        args.norm.x0 = static_cast<const uint16_t *>(norm->x);
        args.norm.residual = static_cast<const uint16_t *>(norm->residual);
        args.norm.weight = static_cast<const uint16_t *>(norm->weight);
        args.norm.h_out = static_cast<uint16_t *>(norm->h_out);
        args.norm.eps = norm->eps;
        args.norm.enabled = 1;
    }
    if (epilogue && (epilogue->bias || epilogue->residual || epilogue->activation != VRL_INT4_ACT_NONE)) {
        args.epi.bias = static_cast<const uint16_t *>(epilogue->bias);
        args.epi.residual = static_cast<const uint16_t *>(epilogue->residual);
        args.epi.y0 = static_cast<const uint16_t *>(problems[0].y);
        args.epi.act = epilogue->activation;
        args.epi.enabled = 1;
    }
    if (max_m > MAX_TILE_M && max_m <= 2 * MAX_TILE_M && max_nsc > 4 && !norm && !lora && !args.epi.enabled) {
        // 17 to 32 rows of K > 2048: two forms of gemv_rows32_direct_kernel, K in passes of what LDS holds of the rows.
        // (a) One record per problem holds all its rows (a weight word is read and rebuilt once for both blocks of
        // 16 rows): four waves per tile, four tiles per workgroup.  (b) Records of 16 rows, eight waves per tile, two
        // tiles per workgroup, fused records excepted.  Measured at 32 rows against two register-fed or staged
        // slabs (7B-class layer): q|k|v (a) 14.6, (b) 23.2, slabs 23.7 us; gate|up (a) 21.1, slabs 32.2 us; o_proj
        // (a) 13.2, (b) 8.2, slabs 12.8 us; down_proj, K = 11008: (a) 30.8 (six passes), (b) 17.1 (three), slabs
        // 29.9 us (every tile's workgroup fetches all of x there: 180 MB from L2); and a form of (a) that fetches
        // its operands into registers 11.7 / 27.0 us for o_proj / down_proj.  With few tiles the slabs win
        // (K = 5632, N = 2048: (b) 10.1, slabs 9.8 us), and at K = 2048 they run side by side (7.5 against 8.9 us).
        const long cus = device_cu_count();
        const bool whole = max_nsc <= 8 && slab_tiles >= 4 * cus;
        const bool slabs16 = !whole && !fused_any && slab_tiles >= 2 * cus;
        if (whole || slabs16) {
            const int ks = whole ? 4 : 8, tw = whole ? 4 : 2, rows = whole ? 2 * MAX_TILE_M : MAX_TILE_M;
            const size_t red = (size_t)tw * (ks - 1) * (fused_any ? 2 : 1) * WAVE * sizeof(f32x4_t);
            long sc_pass = ((long)((ROWS32_LDS_CAP - red) / ((size_t)std::min(rows, max_m) * 2)) - XPAD) / PP_SC;
            sc_pass -= sc_pass % ks;
            if (sc_pass > max_nsc) sc_pass = max_nsc;
            if (sc_pass >= 1) {
                long wgs = 0;
                for (int i = 0; i < n_problems; ++i) {
                    const vrl_int4_problem &q = problems[i];
                    const int out_cols = q.fused_gate_up ? q.N / 2 : q.N;
                    for (int m0 = 0; m0 < q.M; m0 += rows) {
                        if (args.n == DIRECT_MAX) return VRL_INT4_ESHAPE;
                        DevProblem &p = args.recs[args.n++];
                        p.x = static_cast<const uint16_t *>(q.x) + (long)m0 * q.K;
                        p.qweight = static_cast<const uint32_t *>(q.qweight);
                        p.y = static_cast<uint16_t *>(q.y) + (long)m0 * out_cols;
                        p.M = std::min<int>(rows, q.M - m0);
                        p.N = q.N; p.K = q.K; p.G = q.G;
                        p.fused = q.fused_gate_up ? 1 : 0;
                        p.prepacked = 1;
                        p.kc = (int)std::min<long>(sc_pass, pp_nsc(q.K)) * PP_SC;
                        p.tile_begin = (int)wgs;
                        wgs += ((out_cols + 15) / 16 + tw - 1) / tw;
                    }
                }
                if (wgs > (1L << 20)) return VRL_INT4_ESHAPE;
                const size_t lds = (size_t)std::min(rows, max_m) * ((size_t)sc_pass * PP_SC + XPAD) * 2 + red;
                hipStream_t s32 = reinterpret_cast<hipStream_t>(hip_stream);
                args.rounds = 1;
                if (!whole) return launch_rows32<false, 8, 2, 1>(args, (int)wgs, lds, s32);
                return fused_any ? launch_rows32<true, 4, 4, 2>(args, (int)wgs, lds, s32)
                                 : launch_rows32<false, 4, 4, 2>(args, (int)wgs, lds, s32);
            }
        }
    }
    long workgroups = 0;
    size_t x_bytes = 0;
    for (int i = 0; i < n_problems; ++i) {
        const vrl_int4_problem &q = problems[i];
        const int kc = pp_nsc(q.K) * PP_SC;
        const size_t row_bytes = (size_t)(kc + XPAD) * 2;
        long rows = xg ? MAX_TILE_M : (long)((DIRECT_LDS_CAP - red) / row_bytes);
        if (rows > MAX_TILE_M) rows = MAX_TILE_M;
        if (rows < 1) return VRL_INT4_ESHAPE;
        const int out_cols = q.fused_gate_up ? q.N / 2 : q.N;
        const int tiles = (out_cols + 15) / 16;
        for (int m0 = 0; m0 < q.M; m0 += (int)rows) {
            if (args.n == DIRECT_MAX) return VRL_INT4_ESHAPE;  // too many slabs for one launch: use a plan
            DevProblem &p = args.recs[args.n++];
            p.x = static_cast<const uint16_t *>(q.x) + (long)m0 * q.K;
            p.qweight = static_cast<const uint32_t *>(q.qweight);
            p.y = static_cast<uint16_t *>(q.y) + (long)m0 * out_cols;
            p.M = std::min<int>((int)rows, q.M - m0);
            p.N = q.N; p.K = q.K; p.G = q.G;
            p.fused = q.fused_gate_up ? 1 : 0;
            p.prepacked = 1 | (norm && i == 0 ? PP_WRITE_H : 0);  // the first problem's slabs write h
            p.kc = kc;
            p.tile_begin = (int)workgroups;  // first workgroup of the record
            workgroups += (tiles + tw - 1) / tw;
            x_bytes = std::max(x_bytes, (size_t)p.M * row_bytes);
        }
    }
    if (workgroups > (1L << 20)) return VRL_INT4_ESHAPE;
    // padding rows of the A operand read a staged row of zeros where LDS is plentiful
    size_t xz_bytes = x_bytes;
    for (int i = 0; i < args.n; ++i) {
        DevProblem &p = args.recs[i];
        const size_t need = (size_t)(p.M + 1) * (p.kc + XPAD) * 2;
        if (!xg && p.M < MAX_TILE_M && need + red <= 32 * 1024) {
            p.prepacked |= PP_ZERO_ROW;
            xz_bytes = std::max(xz_bytes, need);
        }
    }
    size_t lds = xg ? red : xz_bytes + red;
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    // More workgroups than the device holds at once (16 waves and 160 KB of LDS per CU) would run in
    // waves of workgroups, each staging x and ramping up again: a workgroup then walks several sets of
    // TW tiles, the next set's first loads issued under the current one's last.
    // (a register-fed launch with an epilogue keeps one tile per workgroup: its build walks no second set)
    args.rounds = 1;
    if (!lora_up && !(xg && args.epi.enabled)) {
        const long per_cu = std::max<long>(1, std::min<long>(16 / (ks * tw), (long)(160 * 1024 / std::max<size_t>(lds, 1024))));
        const long capacity = per_cu * device_cu_count();
        args.rounds = (int)std::min<long>(8, (workgroups + capacity - 1) / capacity);
        if (args.rounds > 1) {
            workgroups = 0;
            for (int i = 0; i < args.n; ++i) {
                DevProblem &p = args.recs[i];
                const int tiles = ((p.fused ? p.N / 2 : p.N) + 15) / 16;
                p.tile_begin = (int)workgroups;
                workgroups += (tiles + tw * args.rounds - 1) / (tw * args.rounds);
            }
        }
    }
    if (lora_up) {
        // the launch's one problem carries one adapter: y = base + scaling * t . B^T
        const vrl_int4_problem &q0 = problems[0];
        const vrl_lora_adapter &ad = lora->adapters[0];
        if (!lora->t || !ad.B) return VRL_INT4_ENULL;
        if (n_problems != 1 || lora->n_adapters != 1 || fused_any || ad.N != q0.N || ad.r < 8 || ad.r % 8 != 0 ||
            ad.r > LORA_MAX_RANK || lora->t_parts < 1 || lora->t_parts > 256)
            return VRL_INT4_ESHAPE;
        if ((reinterpret_cast<uintptr_t>(lora->t) | reinterpret_cast<uintptr_t>(ad.B)) & 15u) return VRL_INT4_EALIGN;
        args.up.t = lora->t;
        args.up.B = ad.B;
        args.up.x0 = static_cast<const uint16_t *>(q0.x);
        args.up.parts = lora->t_parts;
        args.up.r = ad.r;
        args.up.fp32 = ad.weights_fp32 != 0;
        args.up.scaling = ad.scaling;
        lds += (size_t)(MAX_TILE_M + 16) * (ad.r + 4) * sizeof(float);
        return launch_direct_up(args, ks, xg, (int)workgroups, lds, stream);
    }
    if (lora_down) {
        // the adapters read the input every problem of the launch reads
        const vrl_int4_problem &q0 = problems[0];
        if (fused_any || !lora->t) return fused_any ? VRL_INT4_ESHAPE : VRL_INT4_ENULL;
        if (reinterpret_cast<uintptr_t>(lora->t) & 15u) return VRL_INT4_EALIGN;
        for (int i = 1; i < n_problems; ++i)
            if (problems[i].x != q0.x || problems[i].M != q0.M || problems[i].K != q0.K) return VRL_INT4_ESHAPE;
        const int rc = lora_args(args.ld.a, q0.M, q0.K, lora->adapters, lora->n_adapters, false);
        if (rc != VRL_INT4_OK) return rc;
        // with a norm the adapters' workgroups normalise the rows themselves, a lane holding one piece of each
        if (norm && (q0.K > NORM_MAX_K / 2 || ks != 4 || q0.M > MAX_TILE_M)) return VRL_INT4_ESHAPE;
        args.ld.x = static_cast<const uint16_t *>(q0.x);
        args.ld.t = lora->t;
        args.ld.fp32 = args.ld.a.ad[0].weights_fp32 != 0;
        args.ld.wgs = lora_down_workgroups(args.ld.a, ks * tw);
        workgroups += args.ld.wgs;
        lds = std::max(lds, (size_t)ks * tw * 16 * sizeof(float));
        return norm ? launch_direct_lora_norm(args, ks, tw, (int)workgroups, lds, stream)
                    : launch_direct_lora(args, ks, tw, (int)workgroups, lds, stream);
    }
    if (args.epi.enabled)
        return norm ? launch_direct_epilogue<true>(args, ks, tw, false, (int)workgroups, lds, stream)
                    : launch_direct_epilogue<false>(args, ks, tw, xg, (int)workgroups, lds, stream);
    if (norm)
        return fused_any ? launch_direct_shape<true, true>(args, ks, tw, false, (int)workgroups, lds, stream)
                         : launch_direct_shape<false, true>(args, ks, tw, false, (int)workgroups, lds, stream);
    return fused_any ? launch_direct_shape<true, false>(args, ks, tw, xg, (int)workgroups, lds, stream)
                     : launch_direct_shape<false, false>(args, ks, tw, xg, (int)workgroups, lds, stream);
}

int vrl_int4_gemv_prepacked_bf16(const vrl_int4_problem *problems, int n_problems, void *hip_stream) {
    return direct_launch(problems, n_problems, nullptr, nullptr, hip_stream);
}

int vrl_int4_gemv_prepacked_lora_bf16(const vrl_int4_problem *problems, int n_problems,
                                      const vrl_lora_adapter *adapters, int n_adapters, float *t,
                                      void *hip_stream) {
    if (!adapters) return VRL_INT4_ENULL;
    const DirectLora lora{adapters, n_adapters, t, false, 1};
    return direct_launch(problems, n_problems, nullptr, &lora, hip_stream);
}

int vrl_int4_gemv_prepacked_norm_lora_bf16(const vrl_int4_problem *problems, int n_problems,
                                           const vrl_int4_norm *norm, const vrl_lora_adapter *adapters,
                                           int n_adapters, float *t, void *hip_stream) {
    if (!norm || !adapters) return VRL_INT4_ENULL;
    const DirectLora lora{adapters, n_adapters, t, false, 1};
    return direct_launch(problems, n_problems, norm, &lora, hip_stream);
}

int vrl_int4_gemv_prepacked_lora_up_bf16(const vrl_int4_problem *problem, const vrl_lora_adapter *adapter,
                                         const float *t, int t_parts, void *hip_stream) {
    if (!adapter) return VRL_INT4_ENULL;
    const DirectLora lora{adapter, 1, const_cast<float *>(t), true, t_parts};
    return direct_launch(problem, 1, nullptr, &lora, hip_stream);
}

int vrl_int4_gemv_prepacked_norm_bf16(const vrl_int4_problem *problems, int n_problems,
                                      const vrl_int4_norm *norm, void *hip_stream) {
    if (!norm) return VRL_INT4_ENULL;
    return direct_launch(problems, n_problems, norm, nullptr, hip_stream);
}

int vrl_int4_gemv_prepacked_epilogue_bf16(const vrl_int4_problem *problem, const vrl_int4_norm *norm,
                                          const vrl_int4_epilogue *epilogue, void *hip_stream) {
    if (!epilogue) return VRL_INT4_ENULL;
    return direct_launch(problem, 1, norm, nullptr, hip_stream, epilogue);
}

size_t vrl_int4_grouped_plan_size(int n_problems) {
    if (n_problems < 1) return 0;
    return plan_bytes_for(n_problems);
}

int vrl_int4_grouped_plan_build(const vrl_int4_problem *problems, int n_problems, void *plan_host,
                                size_t plan_bytes, vrl_int4_plan_info *info) {
    if (!problems || !plan_host || !info) return VRL_INT4_ENULL;
    if (n_problems < 1 || plan_bytes < vrl_int4_grouped_plan_size(n_problems)) return VRL_INT4_EPLAN;
    uint8_t *base = static_cast<uint8_t *>(plan_host);
    DevProblem *recs = reinterpret_cast<DevProblem *>(base + sizeof(PlanHeader));
    int2 *block_tab = reinterpret_cast<int2 *>(recs + n_problems);
    std::vector<int32_t> block_begin((size_t)MAX_PLAN_GRID + 1, 0);

    long tiles = 0;
    double total_cost = 0.0;
    int variant = 0;
    int pp_group_size = 0;      // group size of the prepacked records, -1 if they differ
    size_t x_need = 0;  // bytes the largest activation matrix needs if staged whole
    for (int i = 0; i < n_problems; ++i) {
        const vrl_int4_problem &q = problems[i];
        variant |= (q.prepacked ? VARIANT_PP : VARIANT_CANON) | (q.fused_gate_up ? VARIANT_FUSED : 0);
        int rc;
        if (q.prepacked)
            rc = check_problem(q.x, q.qweight, q.qweight, q.qweight, q.y, q.M, q.N, q.K, q.G);
        else
            rc = check_problem(q.x, q.qweight, q.scales, q.qzeros, q.y, q.M, q.N, q.K, q.G);
        if (rc != VRL_INT4_OK) return rc;
        if (q.fused_gate_up && q.N % 2 != 0) return VRL_INT4_ESHAPE;
        DevProblem p;
        memset(&p, 0, sizeof p);
        p.x = static_cast<const uint16_t *>(q.x);
        p.qweight = static_cast<const uint32_t *>(q.qweight);
        p.scales = static_cast<const uint16_t *>(q.scales);
        p.qzeros = static_cast<const uint32_t *>(q.qzeros);
        p.y = static_cast<uint16_t *>(q.y);
        p.M = q.M; p.N = q.N; p.K = q.K; p.G = q.G;
        p.fused = q.fused_gate_up ? 1 : 0;
        p.prepacked = q.prepacked ? 1 : 0;
        if (!tile_path_ok(p)) return VRL_INT4_ESHAPE;  // grouped launches take MFMA-path shapes only
        if (p.prepacked && (!prepack_ok(p.N, p.K, p.G) || (p.fused && (p.N / 2) % 16 != 0)))
            return VRL_INT4_ESHAPE;
        if (p.prepacked) pp_group_size = (pp_group_size == 0 || pp_group_size == p.G) ? p.G : -1;
        if (p.M > MAX_TILE_M) variant |= VARIANT_MB2;
        p.tile_begin = (int)tiles;
        const int out_cols = p.fused ? p.N / 2 : p.N;
        const long nt = (out_cols + 15) / 16;
        tiles += nt;
        if (tiles >= (1L << 30)) return VRL_INT4_ESHAPE;
        const int kfull = p.prepacked ? pp_nsc(p.K) * PP_SC : p.K;
        const size_t need = (size_t)p.M * (kfull + XPAD) * 2;
        if (need > x_need) x_need = need;
        recs[i] = p;
    }
    // Records go into the blob longest tiles first (the kernel only needs tile_begin to ascend
    // with the record index): the ranges that start last then hold the shortest tiles.
    {
        std::stable_sort(recs, recs + n_problems, [](const DevProblem &a, const DevProblem &b) {
            return (long)a.K * (a.fused ? 2 : 1) > (long)b.K * (b.fused ? 2 : 1);
        });
        long t = 0;
        for (int i = 0; i < n_problems; ++i) {
            recs[i].tile_begin = (int)t;
            t += ((recs[i].fused ? recs[i].N / 2 : recs[i].N) + 15) / 16;
        }
    }
    // more than 16 activation rows per record: prepacked-only plans (two A operands per tile)
    if ((variant & VARIANT_MB2) && (variant & VARIANT_CANON)) return VRL_INT4_ESHAPE;

    // workgroup shape: the narrowest whose LDS holds the largest activation matrix whole
    // (plans with canonical or 32-row records have no 8-wave build); the widest one otherwise,
    // walking K in staged passes
    int shape = 2;
    for (int i = 0; i < 3; ++i) {
        if (x_need > STREAM_SHAPES[i].lds) continue;
        if (i == 1 && (variant & VARIANT_CANON)) continue;
        shape = i;
        break;
    }
    if (variant & VARIANT_MB2) shape = 2;
    const StreamShape sh = STREAM_SHAPES[shape];
    size_t smem = 0;
    for (int i = 0; i < n_problems; ++i) {
        DevProblem &p = recs[i];
        p.kc = p.prepacked ? pp_staged_k(p.M, p.K, sh.lds) : stream_staged_k(p.M, p.K, sh.lds);
        const size_t need = (size_t)p.M * (p.kc + XPAD) * 2;
        if (need > smem) smem = need;
        if (p.prepacked && p.kc < pp_nsc(p.K) * PP_SC) variant |= VARIANT_PASSES;
    }
    int wpb = sh.wpb;  // waves per workgroup of the launch
    // How many workgroups of this build a CU holds at a given LDS size (0: the runtime cannot say).
    auto resident_per_cu = [&](size_t lds_bytes) {
        vrl_int4_plan_info probe;
        memset(&probe, 0, sizeof probe);
        probe.block_threads = wpb * WAVE;
        probe.lds_bytes = (int)lds_bytes;
        probe.variant = variant;
        if (dispatch_stream(&probe, nullptr, nullptr, nullptr) != VRL_INT4_OK) return 0;
        return probe.grid;
    };
    // One contiguous tile range per workgroup, balanced by streamed bytes.  The grid is what the
    // device holds at once (every workgroup runs from start to end, no second round of
    // prologues: measured 1 % faster than a grid twice as deep); if the runtime cannot say how
    // many fit, the table's deeper grid is used and the dispatcher evens out the tail.
    // Plans with fewer tiles than the device has workgroup slots take the latency mode: one
    // workgroup per tile, its waves splitting K (gemv_split_kernel); the partial tiles need LDS
    // behind the staged activations.
    // As many waves share a tile as it has super-chunks (4, 8 or 16), fewer if the plan would
    // not fit the device at that width.
    size_t red_bytes = 0;
    if (shape == 0 && !(variant & (VARIANT_CANON | VARIANT_MB2 | VARIANT_PASSES))) {
        int max_nsc = 1;
        for (int i = 0; i < n_problems; ++i) max_nsc = std::max(max_nsc, pp_nsc(recs[i].K));
        variant |= VARIANT_SPLIT;
        for (int w = max_nsc > 8 ? 16 : (max_nsc > 4 ? 8 : 4); w >= 4; w /= 2) {
            const size_t rb = (size_t)(w - 1) * ((variant & VARIANT_FUSED) ? 2 : 1) * WAVE * sizeof(f32x4_t);
            wpb = w;
            const int slots = resident_per_cu(smem + rb);
            if (slots >= 1 && tiles <= (long)device_cu_count() * slots && tiles <= MAX_PLAN_GRID) {
                red_bytes = rb;
                break;
            }
        }
        if (red_bytes == 0) {
            variant &= ~VARIANT_SPLIT;
            wpb = sh.wpb;
        }
    }
    // The throughput kernel is built per group size: its prepacked records share one, and only
    // 128 goes together with canonical records.  (The latency kernel takes them mixed.)
    if (!(variant & VARIANT_SPLIT) && pp_group_size != 0) {
        if (pp_group_size < 0 || ((variant & VARIANT_CANON) && pp_group_size != 128)) return VRL_INT4_ESHAPE;
        variant |= pp_group_size == 64 ? VARIANT_G64 : (pp_group_size == 32 ? VARIANT_G32 : 0);
    }
    long per_cu = sh.per_cu;
    const int resident = resident_per_cu(smem + red_bytes);
    if (resident >= 1) per_cu = resident;
    // Prepacked records with unused A-operand rows stage one more row, of zeros, for those
    // rows to read, if that costs no residency.
    if (resident >= 1) {
        const int rows_per_record = (variant & VARIANT_MB2) ? 32 : 16;
        size_t smem_z = smem;
        for (int i = 0; i < n_problems; ++i) {
            const DevProblem &p = recs[i];
            const size_t need = (size_t)(p.M + 1) * (p.kc + XPAD) * 2;
            if (p.prepacked && p.M < rows_per_record && need <= sh.lds && need > smem_z) smem_z = need;
        }
        if (smem_z == smem || resident_per_cu(smem_z + red_bytes) == resident) {
            for (int i = 0; i < n_problems; ++i) {
                DevProblem &p = recs[i];
                if (p.prepacked && p.M < rows_per_record && (size_t)(p.M + 1) * (p.kc + XPAD) * 2 <= smem_z)
                    p.prepacked |= PP_ZERO_ROW;
            }
            smem = smem_z;
        }
    }
    smem += red_bytes;
    long grid = (long)device_cu_count() * per_cu;
    if (grid > MAX_PLAN_GRID) grid = MAX_PLAN_GRID;
    const long max_useful = (tiles + sh.wpb - 1) / sh.wpb;
    if (grid > max_useful) grid = max_useful;
    if (variant & VARIANT_SPLIT) {
        grid = tiles;
        for (long k = 0; k <= grid; ++k) block_begin[(size_t)k] = (int)k;
        int rec = 0;
        for (long k = 0; k <= grid; ++k) {
            while (rec + 1 < n_problems && recs[rec + 1].tile_begin <= block_begin[(size_t)k]) ++rec;
            block_tab[k] = make_int2(block_begin[(size_t)k], rec);
        }
    } else
    {
        // what a tile costs: its k extent plus a fixed part; a record walked in staged passes
        // pays for its stagings and barriers on top (measured: the workgroups that hold such tiles
        // ended 28 % after the others at equal weight; 1.45 is the best of a sweep from 1.0 to 2.4 on
        // the 1B set at 32 rows, and is worth 7-8 % on the 7B-class sets at 8 and 16 rows)
        const double pass_factor = 1.45;
        auto tile_cost = [&](const DevProblem &p) {
            const bool passes = p.prepacked && p.kc < pp_nsc(p.K) * PP_SC;
            return ((double)p.K * (p.fused ? 2 : 1) + 512.0) * (passes ? pass_factor : 1.0);
        };
        for (int i = 0; i < n_problems; ++i) {
            const DevProblem &p = recs[i];
            total_cost += (double)(((p.fused ? p.N / 2 : p.N) + 15) / 16) * tile_cost(p);
        }
        int b = 0;
        double acc_cost = 0.0;
        block_begin[0] = 0;
        for (int i = 0; i < n_problems; ++i) {
            const DevProblem &p = recs[i];
            const int out_cols = p.fused ? p.N / 2 : p.N;
            const int nt = (out_cols + 15) / 16;
            const double c = tile_cost(p);
            // a record walked in staged passes deals its tiles to the waves in lock-step, one per
            // wave at a time: a range inside it is cut at a multiple of the workgroup's waves
            const int cut = (p.prepacked && p.kc < pp_nsc(p.K) * PP_SC) ? wpb : 1;
            for (int t = 0; t < nt; ++t) {
                // tile (p.tile_begin + t) starts block b+1 once the blocks so far hold their share
                while (b + 1 < grid && t % cut == 0 && acc_cost >= total_cost * (b + 1) / (double)grid) {
                    ++b;
                    block_begin[b] = p.tile_begin + t;
                }
                acc_cost += c;
            }
        }
        while (b < grid) {
            ++b;
            block_begin[b] = (int)tiles;
        }
        int rec = 0;
        for (long k = 0; k <= grid; ++k) {
            while (rec + 1 < n_problems && recs[rec + 1].tile_begin <= block_begin[(size_t)k]) ++rec;
            block_tab[k] = make_int2(block_begin[(size_t)k], rec);
        }
    }

    PlanHeader hdr;
    hdr.magic = PLAN_MAGIC;
    hdr.n_records = n_problems;
    hdr.total_tiles = (int)tiles;
    hdr.grid = (int)grid;
    memcpy(plan_host, &hdr, sizeof hdr);
    memset(info, 0, sizeof *info);
    info->n_problems = n_problems;
    info->total_tiles = (int)tiles;
    info->grid = (int)grid;
    info->block_threads = wpb * WAVE;
    info->lds_bytes = (int)smem;
    info->variant = variant;
    return VRL_INT4_OK;
}

int vrl_int4_gemv_grouped_bf16(const void *plan_dev, const vrl_int4_plan_info *info,
                               void *hip_stream) {
    if (!plan_dev || !info) return VRL_INT4_ENULL;
    if (info->n_problems < 1 || info->total_tiles < 1 || info->grid < 1 ||
        info->grid > MAX_PLAN_GRID || info->lds_bytes < 0 || (size_t)info->lds_bytes > STREAM_LDS_CAP ||
        !aligned16(plan_dev))
        return VRL_INT4_EPLAN;
    const uint8_t *base = static_cast<const uint8_t *>(plan_dev);
    const DevProblem *recs = reinterpret_cast<const DevProblem *>(base + sizeof(PlanHeader));
    const int2 *block_begin = reinterpret_cast<const int2 *>(recs + info->n_problems);
    vrl_int4_plan_info launch = *info;
    return dispatch_stream(&launch, recs, block_begin, reinterpret_cast<hipStream_t>(hip_stream));
}

}  // extern "C"

// extern "C" entry points of libfalkon_amd: argument checks, workspace carving, launch plans.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <utility>
#include <vector>

#include "flk_common.h"
#include "split_common.h"

namespace flk {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Optional instrumentation: HIP events around every launch of the product kernel, recorded on
// the stream the kernel runs on.  Off by default; a benchmark switches it on to obtain the
// kernel's own duration without an external profiler.
static std::mutex g_timing_mu;
static bool g_timing_on = false;
static std::vector<std::pair<hipEvent_t, hipEvent_t>> g_timing_events;

static void timing_clear_locked() {
    for (auto &e : g_timing_events) {
        (void)hipEventDestroy(e.first);
        (void)hipEventDestroy(e.second);
    }
    g_timing_events.clear();
}

struct ScopedKernelTimer {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipStream_t st;
    explicit ScopedKernelTimer(hipStream_t s) : st(s) {
        std::lock_guard<std::mutex> g(g_timing_mu);
        if (!g_timing_on) return;
        // a launch that is being captured into a graph is not timed: events recorded during capture become graph
        // nodes, and asking them for a time afterwards is an error
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return;
        }
        if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { e0 = e1 = nullptr; return; }
        (void)hipEventRecord(e0, st);
    }
    ~ScopedKernelTimer() {
        if (!e0) return;
        (void)hipEventRecord(e1, st);
        std::lock_guard<std::mutex> g(g_timing_mu);
        g_timing_events.emplace_back(e0, e1);
    }
};

constexpr int64_t kTargetWgs = 8192;  // workgroups wanted per launch: 256 CUs x 2 resident x 16 rounds, so that
                                      // the partly filled last round costs a few percent at most
constexpr int64_t kMinChunkBlocks = 16;
constexpr int kMaxSplits = 4096;
constexpr int64_t kL2ChunkBytes = 2 << 20;
constexpr int64_t kL2PartialBytes = 128 << 20;
constexpr int64_t kWideChunkBlocks = 64;  // column chunks wider than 4 accumulate in one fp32 level: keep the chunks short
// A launch of fewer workgroups than this leaves compute units idle or unevenly loaded: its reduction chunks are then
// chosen by the estimated makespan (all workgroups are resident at once, a compute unit works through the ones it was
// given) instead of the rules for large problems; kTinyChunkBlocks is the shortest chunk that is worth a workgroup's
// prologue and its partial result, whose cost is counted as kWgOverheadPercent / 100 of a block step.
constexpr int64_t kComputeUnits = 256;
constexpr int64_t kMinRounds = 10;
constexpr int64_t kWgOverheadBlocks = 5;
constexpr int64_t kUnderfilledWgs = 4 * kComputeUnits;
constexpr int64_t kTinyChunkBlocks = 2;
constexpr int64_t kWgOverheadPercent = 50;

struct Plan {
    bool large;            // LDS-tiled kernel (d beyond the register-resident kernel's range)
    int64_t chunk;         // reduction-side work per workgroup: A blocks (small) or A tiles (large)
    int splits;            // grid.y
    int partials;          // partial results the finalize kernel sums (= splits x partials per split)
    int col_chunk;         // right-hand sides per pass
    int a_tile_blocks = 0; // LDS-tiled kernel: reduction blocks per tile that chunk counts in
    int64_t dpad = 0;      // padded feature count of the operands (register-resident kernels)
};

constexpr int64_t kTargetWgsLarge = 16384;  // two 256-thread workgroups per CU: 8 rounds

// Plan of a register-resident product kernel: per_wg output blocks per workgroup, a_block_bytes per packed
// reduction block of blk rows, col_chunk right-hand sides per pass, results of elem_bytes per element.
// wgs_per_cu: workgroups of the kernel that a compute unit holds at once.
static void plan_register_resident(Plan &p, int64_t na_blocks, int64_t nb_blocks, int64_t per_wg, int64_t a_block_bytes,
                                   int64_t blk, int col_chunk, int64_t t, int64_t elem_bytes, int wgs_per_cu = 2) {
    p.large = false;
    const int64_t kResidentWgs = wgs_per_cu * kComputeUnits;
    const int64_t b_tiles = (nb_blocks + per_wg - 1) / per_wg;
    int64_t splits = (kTargetWgs + b_tiles - 1) / (b_tiles > 0 ? b_tiles : 1);
    int64_t max_splits = na_blocks / kMinChunkBlocks;
    if (max_splits < 1) max_splits = 1;
    if (splits > max_splits) splits = max_splits;
    p.col_chunk = col_chunk;
    int64_t min_splits = 1;            // what the chunk caps below ask for
    if (t > 4 && p.col_chunk > 4 && elem_bytes == 4) {     // (fp64 sums need no such cap: C2's shape with 64 columns
        int64_t want = (na_blocks + kWideChunkBlocks - 1) / kWideChunkBlocks;   // would write 10 GB of partial sums)
        if (splits < want) splits = want;
        if (min_splits < want) min_splits = want;
    }
    // a reduction chunk is streamed by every output tile that shares it: keep it within half of one XCD's
    // 4 MB L2 so that those re-reads hit L2 instead of HBM (only where there is more than one output tile)
    // ... as long as the partial results this creates stay small (kL2PartialBytes per pass)
    if (b_tiles > 1) {
        int64_t chunk_cap = kL2ChunkBytes / a_block_bytes;
        if (chunk_cap < 1) chunk_cap = 1;
        int64_t want = (na_blocks + chunk_cap - 1) / chunk_cap;
        const int64_t tc = t < p.col_chunk ? (t > 0 ? t : 1) : p.col_chunk;
        const int64_t per_split = tc * nb_blocks * blk * elem_bytes;
        const int64_t affordable = kL2PartialBytes / (per_split > 0 ? per_split : 1);
        if (want > affordable) want = affordable;
        if (splits < want) splits = want;
        if (min_splits < want) min_splits = want;
    }
    if (splits > kMaxSplits) splits = kMaxSplits;
    if (splits < 1) splits = 1;
    if (b_tiles * splits >= kUnderfilledWgs && na_blocks > 0 && b_tiles > 0) {
        // Large problem: between the split count that gives kMinRounds rounds of resident workgroups and the one chosen so
        // far, take the one with the shortest estimated run.  A workgroup costs its chunk plus a fixed overhead
        // (dispatch, loading its resident blocks, its partial result: about kWgOverheadBlocks block steps), so fewer,
        // longer workgroups are cheaper, as long as there are enough rounds for the workgroups to drift apart and
        // the last, partly filled round is not nearly empty: that round is counted as 0.35 + 0.65 x of a full one
        // when a fraction x of the slots is used.  Measured on config 2 (fp32): K v with 5 splits (9770 workgroups)
        // -> 3 (5862): 9.46 -> 9.35 ms per launch; K^T u with 203 splits (8120) -> 128 (5120): 9.44 -> 9.40 ms, while
        // 104 splits (4160 = 8.1 rounds) take 9.60 ms.  The lower bounds set above (chunk caps) are kept.
        int64_t lo = (kMinRounds * kResidentWgs + b_tiles - 1) / b_tiles;
        if (lo < 1) lo = 1;
        if (lo < splits) {
            if (min_splits > lo) lo = min_splits;
            int64_t best = splits, best_cost = -1;
            for (int64_t s = lo; s <= splits; s++) {
                int64_t c = (na_blocks + s - 1) / s;
                if (t == 1 && c > 1 && (c & 1)) c += 1;
                const int64_t wgs = b_tiles * ((na_blocks + c - 1) / c);
                const int64_t full = wgs / kResidentWgs, rem = wgs % kResidentWgs;
                const int64_t rounds_milli = full * 1000 + (rem ? 350 + 650 * rem / kResidentWgs : 0);
                const int64_t cost = rounds_milli * (c + kWgOverheadBlocks);
                if (best_cost < 0 || cost < best_cost) { best = s; best_cost = cost; }
            }
            splits = best;
        }
    }
    if (b_tiles * splits < kUnderfilledWgs && na_blocks > 0 && b_tiles > 0) {
        // small problem: the split count with the shortest estimated makespan, at least the one chosen so far (the
        // chunk caps above still hold); ties go to fewer splits
        int64_t best = splits, best_cost = -1;
        const int64_t most = na_blocks / kTinyChunkBlocks;
        for (int64_t s = splits; s <= most && b_tiles * s <= 2 * kUnderfilledWgs; s++) {
            int64_t c = (na_blocks + s - 1) / s;
            if (t == 1 && c > 1 && (c & 1)) c += 1;
            const int64_t wgs = b_tiles * ((na_blocks + c - 1) / c);
            const int64_t deep = (wgs + kComputeUnits - 1) / kComputeUnits;     // workgroups on the busiest compute unit
            // fp64: a second wave on a SIMD hides the latency of the exponential's table reads (measured, N = 2e4,
            // M = 1e3, d = 8: 0.95 us per block step with one wave per SIMD, 0.60 with two or three); fp32: no gain
            const int64_t per_block = (elem_bytes == 8 && deep >= 2) ? 65 : 100;
            const int64_t cost = deep * (c * per_block + kWgOverheadPercent);
            if (best_cost < 0 || cost < best_cost) { best = s; best_cost = cost; }
        }
        splits = best;
    }
    p.chunk = (na_blocks + splits - 1) / splits;
    if (p.chunk < 1) p.chunk = 1;
    // even chunks for one right-hand side: the single-column fp32 kernel's loop handles two blocks per trip and
    // processes the last block of an odd chunk twice (the second time against zeros), which then happens in the last
    // chunk at most
    if (t == 1 && p.chunk > 1 && (p.chunk & 1)) p.chunk += 1;
    p.splits = (int)((na_blocks + p.chunk - 1) / p.chunk);
    if (p.splits < 1) p.splits = 1;
    p.partials = p.splits;
}

template <typename T>
static Plan make_plan(int64_t na_blocks, int64_t nb_blocks, int64_t d, int64_t dpad, int64_t t) {
    Plan p;
    p.dpad = dpad;
    p.large = !mmv_small_serves<T>(d, t);
    if (!p.large) {
        plan_register_resident(p, na_blocks, nb_blocks, mmv_small_b_blocks_per_wg<T>(dpad, t),
                               dpad * Geo<T>::BLK * (int64_t)sizeof(T), Geo<T>::BLK, mmv_small_max_cols<T>(dpad, t), t,
                               (int64_t)sizeof(T), mmv_small_wgs_per_cu<T>(dpad, t));
    } else {
        p.a_tile_blocks = mmv_large_a_tile_blocks<T>(t);
        const int64_t a_tiles = (na_blocks + p.a_tile_blocks - 1) / p.a_tile_blocks;
        const int64_t b_tiles = (nb_blocks + mmv_large_b_tile_blocks<T>(t) - 1) / mmv_large_b_tile_blocks<T>(t);
        int64_t splits = (kTargetWgsLarge + b_tiles - 1) / (b_tiles > 0 ? b_tiles : 1);
        if (splits > a_tiles) splits = a_tiles;
        if (splits > kMaxSplits) splits = kMaxSplits;
        if (splits < 1) splits = 1;
        p.chunk = (a_tiles + splits - 1) / splits;
        if (p.chunk < 1) p.chunk = 1;
        p.splits = (int)((a_tiles + p.chunk - 1) / p.chunk);
        if (p.splits < 1) p.splits = 1;
        p.partials = p.splits * mmv_large_partials_per_split<T>();
        p.col_chunk = mmv_large_max_cols<T>(t);
    }
    return p;
}

// Width of the kernel instantiation that serves a column chunk of tc right-hand sides: the kernels read
// that many planes of the planar right-hand side, so the planes past the caller's columns must be zero.
template <typename T>
static int instantiated_cols(const Plan &p, int tc) {
    static const int large[] = {1, 2, 4, 8, 16, 32, 48, 64};     // 8 columns: an instantiation of fp64 only
    if (p.large) {
        for (int w : large) if (tc <= w && (w != 8 || sizeof(T) == 8)) return w;
        return tc;
    }
    return mmv_small_width<T>(p.dpad, tc);
}
template <typename T>
static int64_t zero_planes_needed(const Plan &p, int64_t t) {
    if (t <= 0) return 0;
    int tc_last = (int)(t % p.col_chunk == 0 ? p.col_chunk : t % p.col_chunk);
    return instantiated_cols<T>(p, tc_last) - tc_last;
}

// Bytes of the planar copy [t + zero planes][n_a padded] of a right-hand side that multiplies the n_a rows of the
// reduction side in a product whose output side has n_b rows.
template <typename T>
static size_t planar_bytes(int64_t n_a, int64_t n_b, int64_t d, int64_t t) {
    PackedView A = packed_view<T>(nullptr, n_a, d), B = packed_view<T>(nullptr, n_b, d);
    Plan p = make_plan<T>(A.nblk, B.nblk, d, A.dpad, t);
    return align256((size_t)(t + zero_planes_needed<T>(p, t)) * A.npad * sizeof(T));
}

template <typename T>
static size_t partial_bytes(int64_t n_a, int64_t n_b, int64_t d, int64_t t) {
    PackedView A = packed_view<T>(nullptr, n_a, d), B = packed_view<T>(nullptr, n_b, d);
    Plan p = make_plan<T>(A.nblk, B.nblk, d, A.dpad, t);
    int64_t tc = t < p.col_chunk ? t : p.col_chunk;
    return align256((size_t)p.partials * tc * B.npad * sizeof(T));
}

static int check_matrix(const char *name, const void *p, int64_t rows, int64_t cols, int64_t rs, int64_t cs) {
    if (rows < 0 || cols < 0) return fail(FLK_EINVAL, "%s: negative shape", name);
    if (rows > 0 && cols > 0 && p == nullptr) return fail(FLK_EINVAL, "%s: null pointer", name);
    if (rows > 1 && cols > 1 && rs != 1 && cs != 1)
        return fail(FLK_EINVAL, "%s: neither stride is one (row stride %lld, column stride %lld)", name, (long long)rs,
                    (long long)cs);
    return FLK_OK;
}

// out[b,t] = sum_a K(A_a,B_b) vecp[t][a] (+ addend).  vecp is planar [t][A.npad].
template <typename T>
static int mmv_packed_planar(int kf, const PackedView &A, const PackedView &B, const T *vecp, int64_t t, const T *addend,
                             int64_t add_rs, int64_t add_cs, T *out, int64_t out_rs, int64_t out_cs, bool zero_pad,
                             T *partial, size_t partial_avail, hipStream_t st) {
    if (B.n == 0 || t == 0) return FLK_OK;
    Plan p = make_plan<T>(A.nblk, B.nblk, A.d, A.dpad, t);
    for (int64_t t0 = 0; t0 < t; t0 += p.col_chunk) {
        int tc = (int)(t - t0 < p.col_chunk ? t - t0 : p.col_chunk);
        if ((size_t)p.partials * tc * B.npad * sizeof(T) > partial_avail)
            return fail(FLK_ENOMEM, "workspace too small for %d partial sums of %lld x %d", p.partials,
                        (long long)B.npad, tc);
        int partials = p.partials;
        if (A.nblk == 0) {
            partials = 0;  // empty reduction: finalize sums nothing and writes the addend (or zero)
        } else {
            ScopedKernelTimer timer(st);
            int rc = p.large ? launch_mmv_large<T>(kf, A, B, vecp + t0 * A.npad, A.npad, tc, p.a_tile_blocks, p.chunk, p.splits, partial, st)
                             : launch_mmv_small<T>(kf, A, B, vecp + t0 * A.npad, A.npad, tc, p.chunk, p.splits, partial, st);
            if (rc != FLK_OK) return rc;
        }
        int rc = launch_finalize<T>(partial, partials, tc, B.n, B.npad, addend ? addend + t0 * add_cs : nullptr,
                                    add_rs, add_cs, out + t0 * out_cs, out_rs, out_cs, zero_pad, (const T *)B.hnorm, st);
        if (rc != FLK_OK) return rc;
    }
    return FLK_OK;
}

template <typename T>
static int pack_impl(int kf, const void *X, int64_t n, int64_t d, int64_t rs, int64_t cs, const void *sigma, int64_t n_sigma,
                     void *packed, size_t bytes, hipStream_t st) {
    int rc = check_matrix("X", X, n, d, rs, cs);
    if (rc) return rc;
    if (d < 1) return fail(FLK_EINVAL, "feature dimension must be positive");
    if (d > flk_max_d(0)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(0));
    if (sigma == nullptr) return fail(FLK_EINVAL, "sigma: null pointer");
    if (n_sigma != 1 && n_sigma != d)
        return fail(FLK_EINVAL, "The size of sigma (%lld) must match the number of features (%lld) or be 1",
                    (long long)n_sigma, (long long)d);
    if (bytes < packed_bytes<T>(n, d)) return fail(FLK_ENOMEM, "packed buffer too small");
    if (n > 0 && packed == nullptr) return fail(FLK_EINVAL, "packed: null pointer");
    PackedView v = packed_view<T>(packed, n, d);
    // odd-d fp32 operands of the register-resident kernel carry 1.0 in their one padding feature
    const bool one_pad = sizeof(T) == 4 && f32_fold_applies(d);
    return launch_pack<T, T>((const T *)X, n, d, rs, cs, (const T *)sigma, n_sigma, operand_scale(kf, sizeof(T) == 8), (T *)v.data,
                             (T *)v.hnorm, v.dpad, v.nblk, one_pad, st);
}

// Prologue of a one-shot product in one launch: X1 packed into p1 (the output side of the first product), X2 into p2
// and v, which multiplies the rows of X2, as planes in vp (zero_planes cleared planes after the t-th).
template <typename T>
static int pack_pair_impl(int kf, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, void *p1, const void *X2,
                          int64_t m, int64_t x2_rs, int64_t x2_cs, void *p2, int64_t d, const void *sigma,
                          int64_t n_sigma, const void *v, int64_t v_rs, int64_t v_cs, int64_t t, T *vp,
                          int64_t zero_planes, hipStream_t st) {
    int rc;
    if ((rc = check_matrix("X", X1, n, d, x1_rs, x1_cs))) return rc;
    if ((rc = check_matrix("X", X2, m, d, x2_rs, x2_cs))) return rc;
    if (sigma == nullptr) return fail(FLK_EINVAL, "sigma: null pointer");
    if (n_sigma != 1 && n_sigma != d)
        return fail(FLK_EINVAL, "The size of sigma (%lld) must match the number of features (%lld) or be 1",
                    (long long)n_sigma, (long long)d);
    PackedView P1 = packed_view<T>(p1, n, d), P2 = packed_view<T>(p2, m, d);
    const bool one_pad = sizeof(T) == 4 && f32_fold_applies(d);
    return launch_pack_pair<T>((const T *)X1, n, x1_rs, x1_cs, (T *)P1.data, (T *)P1.hnorm, P1.nblk, (const T *)X2, m,
                               x2_rs, x2_cs, (T *)P2.data, (T *)P2.hnorm, P2.nblk, d, (const T *)sigma, n_sigma,
                               operand_scale(kf, sizeof(T) == 8), P1.dpad, one_pad, (const T *)v, v_rs, v_cs, vp, t, zero_planes, st);
}

template <typename T>
static int mmv_packed_impl(int kf, const void *pa, int64_t n_a, const void *pb, int64_t n_b, int64_t d, const void *vec,
                           int64_t vec_rs, int64_t vec_cs, int64_t t, const void *addend, int64_t add_rs,
                           int64_t add_cs, void *out, int64_t out_rs, int64_t out_cs, void *ws, size_t ws_bytes,
                           hipStream_t st) {
    if (n_a < 0 || n_b < 0 || d < 1 || t < 0) return fail(FLK_EINVAL, "bad shape");
    if (d > flk_max_d(0)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(0));
    if (t > flk_max_t()) return fail(FLK_EUNSUPPORTED, "more than %lld right-hand sides", (long long)flk_max_t());
    if (n_b == 0 || t == 0) return FLK_OK;
    if (out == nullptr) return fail(FLK_EINVAL, "out: null pointer");
    if (n_a > 0 && vec == nullptr) return fail(FLK_EINVAL, "vec: null pointer");
    PackedView A = packed_view<T>(pa, n_a, d), B = packed_view<T>(pb, n_b, d);
    size_t vec_bytes = planar_bytes<T>(n_a, n_b, d, t);
    size_t need = vec_bytes + partial_bytes<T>(n_a, n_b, d, t);
    if (ws_bytes < need || (need > 0 && ws == nullptr))
        return fail(FLK_ENOMEM, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    T *vecp = (T *)ws;
    T *partial = (T *)((char *)ws + vec_bytes);
    Plan plan = make_plan<T>(A.nblk, B.nblk, A.d, A.dpad, t);
    int rc = launch_vec_planar<T>((const T *)vec, n_a, t, vec_rs, vec_cs, vecp, A.npad, zero_planes_needed<T>(plan, t),
                                  (const T *)A.hnorm, st);
    if (rc) return rc;
    return mmv_packed_planar<T>(kf, A, B, vecp, t, (const T *)addend, add_rs, add_cs, (T *)out, out_rs, out_cs, false,
                                partial, ws_bytes - vec_bytes, st);
}

template <typename T>
static size_t fmmv_ws_bytes(int64_t n, int64_t m, int64_t d, int64_t t) {
    return packed_bytes<T>(n, d) + packed_bytes<T>(m, d) + planar_bytes<T>(m, n, d, t) + partial_bytes<T>(m, n, d, t);
}

template <typename T>
static size_t fdmmv_ws_bytes(int64_t n, int64_t m, int64_t d, int64_t t) {
    size_t p1 = partial_bytes<T>(m, n, d, t), p2 = partial_bytes<T>(n, m, d, t);
    return packed_bytes<T>(n, d) + packed_bytes<T>(m, d) + planar_bytes<T>(m, n, d, t) + planar_bytes<T>(n, m, d, t) +
           (p1 > p2 ? p1 : p2);
}

template <typename T>
static int fmmv_impl(int kf, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m, int64_t x2_rs,
                     int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v, int64_t v_rs,
                     int64_t v_cs, int64_t t, void *out, int64_t out_rs, int64_t out_cs, void *ws, size_t ws_bytes,
                     hipStream_t st) {
    if (n < 0 || m < 0 || d < 1 || t < 0) return fail(FLK_EINVAL, "bad shape");
    if (d > flk_max_d(0)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(0));
    if (t > flk_max_t()) return fail(FLK_EUNSUPPORTED, "more than %lld right-hand sides", (long long)flk_max_t());
    int rc;
    if ((rc = check_matrix("v", v, m, t, v_rs, v_cs))) return rc;
    if ((rc = check_matrix("out", out, n, t, out_rs, out_cs))) return rc;
    size_t need = fmmv_ws_bytes<T>(n, m, d, t);
    if (ws_bytes < need || (need > 0 && ws == nullptr))
        return fail(FLK_ENOMEM, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    char *p = (char *)ws;
    void *px = p; p += packed_bytes<T>(n, d);
    void *pc = p; p += packed_bytes<T>(m, d);
    T *vecp = (T *)p; p += planar_bytes<T>(m, n, d, t);
    PackedView X = packed_view<T>(px, n, d), C = packed_view<T>(pc, m, d);
    Plan plan = make_plan<T>(C.nblk, X.nblk, d, C.dpad, t);
    if ((rc = pack_pair_impl<T>(kf, X1, n, x1_rs, x1_cs, px, X2, m, x2_rs, x2_cs, pc, d, sigma, n_sigma, v, v_rs, v_cs, t,
                                vecp, zero_planes_needed<T>(plan, t), st)))
        return rc;
    if (n == 0 || t == 0) return FLK_OK;
    return mmv_packed_planar<T>(kf, C, X, vecp, t, nullptr, 0, 0, (T *)out, out_rs, out_cs, false, (T *)p,
                                ws_bytes - (size_t)(p - (char *)ws), st);
}

template <typename T>
static int fdmmv_impl(int kf, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m,
                      int64_t x2_rs, int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v,
                      int64_t v_rs, int64_t v_cs, const void *w, int64_t w_rs, int64_t w_cs, int64_t t, void *out,
                      int64_t out_rs, int64_t out_cs, void *ws, size_t ws_bytes, hipStream_t st) {
    if (n < 0 || m < 0 || d < 1 || t < 0) return fail(FLK_EINVAL, "bad shape");
    if (d > flk_max_d(0)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(0));
    if (t > flk_max_t()) return fail(FLK_EUNSUPPORTED, "more than %lld right-hand sides", (long long)flk_max_t());
    int rc;
    if (v == nullptr && m > 0 && t > 0) return fail(FLK_EINVAL, "v: null pointer (v is required)");
    if ((rc = check_matrix("v", v, m, t, v_rs, v_cs))) return rc;
    if (w && (rc = check_matrix("w", w, n, t, w_rs, w_cs))) return rc;
    if ((rc = check_matrix("out", out, m, t, out_rs, out_cs))) return rc;
    size_t need = fdmmv_ws_bytes<T>(n, m, d, t);
    if (ws_bytes < need || (need > 0 && ws == nullptr))
        return fail(FLK_ENOMEM, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    PackedView X = packed_view<T>(nullptr, n, d), C = packed_view<T>(nullptr, m, d);
    char *p = (char *)ws;
    void *px = p; p += packed_bytes<T>(n, d);
    void *pc = p; p += packed_bytes<T>(m, d);
    T *vp = (T *)p; p += planar_bytes<T>(m, n, d, t);     // v multiplies the rows of C in K v
    T *up = (T *)p; p += planar_bytes<T>(n, m, d, t);     // u multiplies the rows of X in K^T u
    T *partial = (T *)p;
    size_t partial_avail = ws_bytes - (size_t)(p - (char *)ws);
    X = packed_view<T>(px, n, d);
    C = packed_view<T>(pc, m, d);
    Plan plan1 = make_plan<T>(C.nblk, X.nblk, d, C.dpad, t), plan2 = make_plan<T>(X.nblk, C.nblk, d, X.dpad, t);
    if ((rc = pack_pair_impl<T>(kf, X1, n, x1_rs, x1_cs, px, X2, m, x2_rs, x2_cs, pc, d, sigma, n_sigma, v, v_rs, v_cs, t,
                                vp, zero_planes_needed<T>(plan1, t), st)))
        return rc;
    // u = K v + w, planar [t][X.npad] with zeroed padding (rows and the spare planes) so it can feed the
    // second product directly
    if ((rc = launch_zero_fill<T>(up + t * X.npad, zero_planes_needed<T>(plan2, t) * X.npad, st))) return rc;
    if ((rc = mmv_packed_planar<T>(kf, C, X, vp, t, (const T *)w, w_rs, w_cs, up, 1, X.npad, true, partial, partial_avail,
                                   st)))
        return rc;
    // out = K^T u
    return mmv_packed_planar<T>(kf, X, C, up, t, nullptr, 0, 0, (T *)out, out_rs, out_cs, false, partial, partial_avail,
                                st);
}

// TI: element type of X1, X2, sigma and out; T: type the kernel values are computed in.
template <typename TI, typename T>
static int fmm_impl(int kf, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m, int64_t x2_rs,
                    int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, void *out, int64_t out_rs,
                    int64_t out_cs, void *ws, size_t ws_bytes, hipStream_t st) {
    if (n < 0 || m < 0 || d < 1) return fail(FLK_EINVAL, "bad shape");
    if (d > flk_max_d(0)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(0));
    int rc;
    if ((rc = check_matrix("X1", X1, n, d, x1_rs, x1_cs))) return rc;
    if ((rc = check_matrix("X2", X2, m, d, x2_rs, x2_cs))) return rc;
    if ((rc = check_matrix("out", out, n, m, out_rs, out_cs))) return rc;
    if (sigma == nullptr) return fail(FLK_EINVAL, "sigma: null pointer");
    if (n_sigma != 1 && n_sigma != d)
        return fail(FLK_EINVAL, "The size of sigma (%lld) must match the number of features (%lld) or be 1",
                    (long long)n_sigma, (long long)d);
    if (n == 0 || m == 0) return FLK_OK;
    const size_t need = packed_bytes<T>(n, d) + packed_bytes<T>(m, d);
    if (ws_bytes < need || ws == nullptr)
        return fail(FLK_ENOMEM, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    PackedView P1 = packed_view<T>(ws, n, d), P2 = packed_view<T>((char *)ws + packed_bytes<T>(n, d), m, d);
    if ((rc = launch_pack<TI, T>((const TI *)X1, n, d, x1_rs, x1_cs, (const TI *)sigma, n_sigma, operand_scale(kf, sizeof(T) == 8),
                                 (T *)P1.data,
                                 (T *)P1.hnorm, P1.dpad, P1.nblk, false, st)))
        return rc;
    if ((rc = launch_pack<TI, T>((const TI *)X2, m, d, x2_rs, x2_cs, (const TI *)sigma, n_sigma, operand_scale(kf, sizeof(T) == 8),
                                 (T *)P2.data,
                                 (T *)P2.hnorm, P2.dpad, P2.nblk, false, st)))
        return rc;
    // lanes run along the B operand: make that the dimension of out with the unit stride (a dimension of
    // extent one never has its stride applied, so it can take either role)
    if (out_cs == 1 || m == 1) return launch_fmm<T, TI>(kf, P1, P2, (TI *)out, out_rs, st);
    return launch_fmm<T, TI>(kf, P2, P1, (TI *)out, out_cs, st);
}

// ---------------------------------------------------------------------------
// bf16x3 mode of the fp32 products (split_common.h): same drivers on the split operands; register-resident kernel
// up to kSplitMaxD features, LDS-tiled kernel beyond.
// ---------------------------------------------------------------------------
constexpr int64_t kTargetWgsSplitLarge = 8192;  // one 512-thread workgroup per CU: 32 rounds

// Where the bf16x3 kernels are the faster route to the same result.  Measured at N = 5e5, M = 2e4, dfmmv, against the
// fp32 MFMA kernels.  Up to four right-hand sides (register-resident kernel, up to four columns per pass): d = 9 / 28 /
// 60, 4 columns: 5.0 / 7.3 / 12.5 ms against 6.2 / 11.3 / 21.6.  5 to 16 (LDS-tiled kernel, sixteen columns per pass on
// the matrix cores; the fp32 kernels contract 8 or 16 columns with narrow MFMA steps): d = 9 / 16 / 28 / 32: 11.4 / 13.5 /
// 13.4 / 15.6 against 6.7 / 8.8 / 12.3 / 13.5 with 5 columns and 8.8 / 11.0 / 14.6 / 15.9 with 9; d = 40 / 48 / 60: 15.7 /
// 17.8 / 17.9 against 16.8 / 19.0 / 23.6 with 5 columns and 18.4 / 20.7 / 25.0 with 9 (two passes of the register-resident
// kernel for 5 to 8 columns: 17.8 / 22.2 / 23.2).  17 and more: the fp32 kernels contract 32 or 64 columns per pass.  So:
// every feature count beyond the register-resident kernels; at small feature counts 1 to 4 right-hand sides, 5 to 16
// beyond 32 features and 9 to 16 from 25 features on; otherwise the fp32 MFMA kernels serve the mode.
// The register-resident bf16x3 kernel for many right-hand sides (mmv_split_wide.hip) serves the column counts beyond
// four at every feature count of the register-resident kernels.  N = 5e5, M = 2e4, 8 / 16 / 32 / 64 columns against the fp32
// kernels: d = 28 8.3 / 10.4 / 14.7 / 25.3 ms against 12.4 / 15.1 / 19.9 / 29.4; d = 56 13.5 / 15.7 / 19.7 / 30.2 against 21.7 /
// 23.5 / 28.3 / 38.0 (and 17.9 for up to 16 columns on the LDS-tiled bf16x3 kernel); d = 9 5.8 / 7.9 / 12.6 / 23.0 against
// 6.9 / 9.0 / 13.8 / 23.9; d = 4 5.6 / 7.7 / 12.6 / 23.0 against 5.7 / 7.8 / 12.4 / 22.1 (the fp32 kernels keep four resident blocks
// per wave there): below 9 features up to 16 columns only, the fp32 kernels beyond.
// Beyond the register-resident kernels the LDS-tiled bf16x3 kernel contracts 16, 32 or 64 columns per pass, as the fp32
// one does, and its cross term is the shorter one at every column count (N = 2.5e5, M = 2e4, 16 / 32 / 64 columns: d = 63
// 10.8 / 13.5 / 19.1 ms against 12.8 / 15.2 / 21.3, d = 100 13.6 / 16.3 / 21.5 against 20.3 / 24.4 / 32.2, d = 300 30.6 / 34.2 /
// 39.6 against 49.2 / 54.5 / 62.8; N = 5e5, M = 1e4, d = 784: 73.1 / 82.2 / 87.1 against 120.3 / 129.3 / 138.3; the one
// exception found, 33 to 40 columns just beyond 62 features, is 18.3 against 17.5).
// Up to four features the fp32 kernels are the faster ones at every column count (their cross term is one or two MFMA steps;
// one right-hand side at d = 2 / 4 / 5 / 6: 2.6 / 3.0 / 3.8 / 3.7 ms against 3.4 / 3.5 / 3.5 / 3.6).
static bool split_applies(int64_t d, int64_t t) {
    if (d <= 4) return false;
    if (t <= kSplitMaxCols) return true;
    if (d > kSplitMaxD) return true;
    return d > 8 || (t <= 16 && d > 5);
}

static Plan make_plan_split(int64_t na_blocks, int64_t nb_blocks, int64_t ks, int64_t t) {
    Plan p;
    // up to four right-hand sides the register-resident kernel with per-lane FMAs
    if (ks * 16 <= kSplitMaxD + 2 && t <= kSplitMaxCols) {
        plan_register_resident(p, na_blocks, nb_blocks, split_b_blocks_per_wg(ks, t), ks * 3 * 64 * 16, 32, kSplitMaxCols,
                               t, (int64_t)sizeof(float));
        return p;
    }
    // more right-hand sides: the register-resident kernel that contracts on the matrix cores
    if (ks * 16 <= kSplitWideMaxD + 2) {
        plan_register_resident(p, na_blocks, nb_blocks, 4 * kSplitWideBlocksPerWave, ks * 3 * 64 * 16, 32,
                               kSplitWideMaxCols, t, (int64_t)sizeof(float));
        return p;
    }
    p.large = true;
    const int64_t a_tiles = (na_blocks + split_large_a_tile_blocks() - 1) / split_large_a_tile_blocks();
    const int64_t b_tiles = (nb_blocks + split_large_b_tile_blocks() - 1) / split_large_b_tile_blocks();
    int64_t splits = (kTargetWgsSplitLarge + b_tiles - 1) / (b_tiles > 0 ? b_tiles : 1);
    if (splits > a_tiles) splits = a_tiles;
    if (splits > kMaxSplits) splits = kMaxSplits;
    if (splits < 1) splits = 1;
    p.chunk = (a_tiles + splits - 1) / splits;
    if (p.chunk < 1) p.chunk = 1;
    p.splits = (int)((a_tiles + p.chunk - 1) / p.chunk);
    if (p.splits < 1) p.splits = 1;
    p.partials = p.splits * split_large_partials_per_split();
    p.col_chunk = split_large_max_cols();
    return p;
}
static size_t split_planar_bytes(int64_t n_a, int64_t t) {
    return align256((size_t)t * (size_t)((n_a + 31) / 32 * 32) * sizeof(float));
}
static size_t split_partial_bytes(int64_t n_a, int64_t n_b, int64_t d, int64_t t) {
    SplitView A = split_view(nullptr, n_a, d), B = split_view(nullptr, n_b, d);
    Plan p = make_plan_split(A.nblk, B.nblk, A.ks, t);
    int64_t tc = t < p.col_chunk ? t : p.col_chunk;
    return align256((size_t)p.partials * tc * B.npad * sizeof(float));
}

// out[b,t] = sum_a K(A_a,B_b) vecp[t][a] (+ addend).  vecp is planar [t][A.npad].
static int mmv_split_planar(int kf, const SplitView &A, const SplitView &B, const float *vecp, int64_t t,
                            const float *addend, int64_t add_rs, int64_t add_cs, float *out, int64_t out_rs,
                            int64_t out_cs, bool zero_pad, float *partial, size_t partial_avail, hipStream_t st) {
    if (B.n == 0 || t == 0) return FLK_OK;
    Plan p = make_plan_split(A.nblk, B.nblk, A.ks, t);
    for (int64_t t0 = 0; t0 < t; t0 += p.col_chunk) {
        int tc = (int)(t - t0 < p.col_chunk ? t - t0 : p.col_chunk);
        if ((size_t)p.partials * tc * B.npad * sizeof(float) > partial_avail)
            return fail(FLK_ENOMEM, "workspace too small for %d partial sums of %lld x %d", p.partials,
                        (long long)B.npad, tc);
        int partials = p.partials;
        if (A.nblk == 0) {
            partials = 0;
        } else {
            ScopedKernelTimer timer(st);
            int rc;
            if (p.large)
                rc = launch_mmv_split_large(kf, A, B, vecp + t0 * A.npad, A.npad, tc, p.chunk, p.splits, partial, st);
            else if (tc > kSplitMaxCols)
                rc = launch_mmv_split_wide(kf, A, B, vecp + t0 * A.npad, A.npad, tc, p.chunk, p.splits, partial, st);
            else
                rc = launch_mmv_split(kf, A, B, vecp + t0 * A.npad, A.npad, tc, p.chunk, p.splits, partial, st);
            if (rc != FLK_OK) return rc;
        }
        int rc = launch_finalize<float>(partial, partials, tc, B.n, B.npad, addend ? addend + t0 * add_cs : nullptr,
                                        add_rs, add_cs, out + t0 * out_cs, out_rs, out_cs, zero_pad, B.hnorm, st);
        if (rc != FLK_OK) return rc;
    }
    return FLK_OK;
}

static int pack_split_impl(int kf, const char *name, const void *X, int64_t n, int64_t d, int64_t rs, int64_t cs,
                           const void *sigma, int64_t n_sigma, void *packed, hipStream_t st) {
    int rc = check_matrix(name, X, n, d, rs, cs);
    if (rc) return rc;
    if (sigma == nullptr) return fail(FLK_EINVAL, "sigma: null pointer");
    if (n_sigma != 1 && n_sigma != d)
        return fail(FLK_EINVAL, "The size of sigma (%lld) must match the number of features (%lld) or be 1",
                    (long long)n_sigma, (long long)d);
    return launch_pack_split((const float *)X, n, d, rs, cs, (const float *)sigma, n_sigma, operand_scale(kf, false), packed, st);
}

static size_t fmmv_split_ws_bytes(int64_t n, int64_t m, int64_t d, int64_t t) {
    return split_packed_bytes(n, d) + split_packed_bytes(m, d) + split_planar_bytes(m, t) +
           split_partial_bytes(m, n, d, t);
}
static size_t fdmmv_split_ws_bytes(int64_t n, int64_t m, int64_t d, int64_t t) {
    size_t p1 = split_partial_bytes(m, n, d, t), p2 = split_partial_bytes(n, m, d, t);
    return split_packed_bytes(n, d) + split_packed_bytes(m, d) + split_planar_bytes(m, t) + split_planar_bytes(n, t) +
           (p1 > p2 ? p1 : p2);
}

static int fmmv_split_impl(int kf, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m,
                           int64_t x2_rs, int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v,
                           int64_t v_rs, int64_t v_cs, int64_t t, void *out, int64_t out_rs, int64_t out_cs, void *ws,
                           size_t ws_bytes, hipStream_t st) {
    if (n < 0 || m < 0 || d < 1 || t < 0) return fail(FLK_EINVAL, "bad shape");
    if (d > flk_max_d(0)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(0));
    if (t > flk_max_t()) return fail(FLK_EUNSUPPORTED, "more than %lld right-hand sides", (long long)flk_max_t());
    int rc;
    if ((rc = check_matrix("v", v, m, t, v_rs, v_cs))) return rc;
    if ((rc = check_matrix("out", out, n, t, out_rs, out_cs))) return rc;
    size_t need = fmmv_split_ws_bytes(n, m, d, t);
    if (ws_bytes < need || (need > 0 && ws == nullptr))
        return fail(FLK_ENOMEM, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    char *p = (char *)ws;
    void *px = p; p += split_packed_bytes(n, d);
    void *pc = p; p += split_packed_bytes(m, d);
    float *vp = (float *)p; p += split_planar_bytes(m, t);
    float *partial = (float *)p;
    if ((rc = pack_split_impl(kf, "X1", X1, n, d, x1_rs, x1_cs, sigma, n_sigma, px, st))) return rc;
    if ((rc = pack_split_impl(kf, "X2", X2, m, d, x2_rs, x2_cs, sigma, n_sigma, pc, st))) return rc;
    SplitView X = split_view(px, n, d), C = split_view(pc, m, d);
    if (n == 0 || t == 0) return FLK_OK;
    if ((rc = launch_vec_planar<float>((const float *)v, m, t, v_rs, v_cs, vp, C.npad, 0, C.hnorm, st))) return rc;
    return mmv_split_planar(kf, C, X, vp, t, nullptr, 0, 0, (float *)out, out_rs, out_cs, false, partial,
                            ws_bytes - (size_t)(p - (char *)ws), st);
}

static int fdmmv_split_impl(int kf, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m,
                            int64_t x2_rs, int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v,
                            int64_t v_rs, int64_t v_cs, const void *w, int64_t w_rs, int64_t w_cs, int64_t t, void *out,
                            int64_t out_rs, int64_t out_cs, void *ws, size_t ws_bytes, hipStream_t st) {
    if (n < 0 || m < 0 || d < 1 || t < 0) return fail(FLK_EINVAL, "bad shape");
    if (d > flk_max_d(0)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(0));
    if (t > flk_max_t()) return fail(FLK_EUNSUPPORTED, "more than %lld right-hand sides", (long long)flk_max_t());
    int rc;
    if (v == nullptr && m > 0 && t > 0) return fail(FLK_EINVAL, "v: null pointer (v is required)");
    if ((rc = check_matrix("v", v, m, t, v_rs, v_cs))) return rc;
    if (w && (rc = check_matrix("w", w, n, t, w_rs, w_cs))) return rc;
    if ((rc = check_matrix("out", out, m, t, out_rs, out_cs))) return rc;
    size_t need = fdmmv_split_ws_bytes(n, m, d, t);
    if (ws_bytes < need || (need > 0 && ws == nullptr))
        return fail(FLK_ENOMEM, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    char *p = (char *)ws;
    void *px = p; p += split_packed_bytes(n, d);
    void *pc = p; p += split_packed_bytes(m, d);
    float *vp = (float *)p; p += split_planar_bytes(m, t);     // v multiplies the rows of C in K v
    float *up = (float *)p; p += split_planar_bytes(n, t);     // u multiplies the rows of X in K^T u
    float *partial = (float *)p;
    size_t partial_avail = ws_bytes - (size_t)(p - (char *)ws);
    if ((rc = pack_split_impl(kf, "X1", X1, n, d, x1_rs, x1_cs, sigma, n_sigma, px, st))) return rc;
    if ((rc = pack_split_impl(kf, "X2", X2, m, d, x2_rs, x2_cs, sigma, n_sigma, pc, st))) return rc;
    SplitView X = split_view(px, n, d), C = split_view(pc, m, d);
    if (m == 0 || t == 0) return FLK_OK;
    if ((rc = launch_vec_planar<float>((const float *)v, m, t, v_rs, v_cs, vp, C.npad, 0, C.hnorm, st))) return rc;
    // u = K v + w, planar [t][X.npad] with zeroed padding rows so it can feed the second product directly
    if ((rc = mmv_split_planar(kf, C, X, vp, t, (const float *)w, w_rs, w_cs, up, 1, X.npad, true, partial,
                               partial_avail, st)))
        return rc;
    return mmv_split_planar(kf, X, C, up, t, nullptr, 0, 0, (float *)out, out_rs, out_cs, false, partial, partial_avail,
                            st);
}

// bf16x3 mode of the kernel matrix: beyond the register-resident feature counts, fp32 arithmetic only (the fp64
// evaluation of fp32 data, compute_f64, keeps its own kernels).
static bool fmm_split_applies(int64_t d, int dtype, int compute_f64) {
    return dtype == FLK_F32_BF16X3 && !compute_f64 && d > kSmallMaxD;
}

static int fmm_split_impl(int kf, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m,
                          int64_t x2_rs, int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, void *out,
                          int64_t out_rs, int64_t out_cs, void *ws, size_t ws_bytes, hipStream_t st) {
    if (n < 0 || m < 0 || d < 1) return fail(FLK_EINVAL, "bad shape");
    if (d > flk_max_d(0)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(0));
    int rc;
    if ((rc = check_matrix("out", out, n, m, out_rs, out_cs))) return rc;
    if (n == 0 || m == 0) return FLK_OK;
    const size_t need = split_packed_bytes(n, d) + split_packed_bytes(m, d);
    if (ws_bytes < need || ws == nullptr)
        return fail(FLK_ENOMEM, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    void *p1 = ws, *p2 = (char *)ws + split_packed_bytes(n, d);
    if ((rc = pack_split_impl(kf, "X1", X1, n, d, x1_rs, x1_cs, sigma, n_sigma, p1, st))) return rc;
    if ((rc = pack_split_impl(kf, "X2", X2, m, d, x2_rs, x2_cs, sigma, n_sigma, p2, st))) return rc;
    SplitView P1 = split_view(p1, n, d), P2 = split_view(p2, m, d);
    // lanes run along the B operand: make that the dimension of out with the unit stride
    if (out_cs == 1 || m == 1) return launch_fmm_split_large(kf, P1, P2, (float *)out, out_rs, st);
    return launch_fmm_split_large(kf, P2, P1, (float *)out, out_cs, st);
}

// ---------------------------------------------------------------------------
// Scratch memory of the entry point that allocates nothing (flk_gauss_fdmmv_noalloc): one array per GPU, part of the
// loaded code object, held until the process ends.  `scratch` is only a host-side handle of the symbol: the device
// address comes from hipGetSymbolAddress, once per device, and only that address is ever handed to kernels.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[FLK_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void *g_scratch_ptr[kMaxDevices] = {};

// Device address of the current device's copy of `scratch` (looked up on the first call on that device).
static int scratch_address(void **ptr) {
    int dev = -1;
    FLK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(FLK_EUNSUPPORTED, "device ordinal %d beyond %d", dev, kMaxDevices - 1);
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        FLK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr) return fail(FLK_EHIP, "hipGetSymbolAddress returned a null address for the scratch array");
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return FLK_OK;
}

}  // namespace flk

using namespace flk;

extern "C" {

int flk_version(void) { return 100; }
const char *flk_last_error(void) { return g_err; }
int64_t flk_max_d(int dtype) { (void)dtype; return (int64_t)1 << 20; }
int64_t flk_max_t(void) { return 65535 - kColPad; }   // the planar right-hand sides (t + spare planes) index grid.y

int flk_kernel_timing_enable(int on) {
    std::lock_guard<std::mutex> g(g_timing_mu);
    timing_clear_locked();
    g_timing_on = on != 0;
    return FLK_OK;
}

int flk_kernel_timing_read(double *total_ms, int64_t *launches) {
    g_err[0] = 0;
    if (!total_ms || !launches) return fail(FLK_EINVAL, "null output pointer");
    std::lock_guard<std::mutex> g(g_timing_mu);
    double tot = 0.0;
    for (auto &e : g_timing_events) {
        float ms = 0.f;
        hipError_t err = hipEventSynchronize(e.second);
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, e.first, e.second);
        if (err != hipSuccess) {
            (void)hipGetLastError();       // do not leave the error for the next launch check to find
            timing_clear_locked();
            return fail(FLK_EHIP, "reading a kernel timing event failed: %s", hipGetErrorString(err));
        }
        tot += ms;
    }
    *total_ms = tot;
    *launches = (int64_t)g_timing_events.size();
    timing_clear_locked();
    return FLK_OK;
}

static bool known_dtype(int dtype, bool with_split) {
    return dtype == FLK_F32 || dtype == FLK_F64 || (with_split && dtype == FLK_F32_BF16X3);
}

size_t flk_gauss_packed_bytes(int64_t n, int64_t d, int dtype) {
    if (n < 0 || d < 1 || d > flk_max_d(dtype) || !known_dtype(dtype, false)) return 0;
    return dtype == FLK_F64 ? packed_bytes<double>(n, d) : packed_bytes<float>(n, d);
}

#define FLK_CHECK_KERNEL(kernel) \
    if (!valid_kernel_fn(kernel)) return fail(FLK_EINVAL, "unknown kernel function %d", kernel)

int flk_kernel_pack(int kernel, const void *X, int64_t n, int64_t d, int64_t x_rs, int64_t x_cs, const void *sigma,
                    int64_t n_sigma, int dtype, void *packed, size_t packed_bytes_, void *stream) {
    g_err[0] = 0;
    FLK_CHECK_KERNEL(kernel);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == FLK_F32) return pack_impl<float>(kernel, X, n, d, x_rs, x_cs, sigma, n_sigma, packed, packed_bytes_, st);
    if (dtype == FLK_F64) return pack_impl<double>(kernel, X, n, d, x_rs, x_cs, sigma, n_sigma, packed, packed_bytes_, st);
    return fail(FLK_EINVAL, "unknown dtype %d", dtype);
}

int flk_gauss_pack(const void *X, int64_t n, int64_t d, int64_t x_rs, int64_t x_cs, const void *sigma,
                   int64_t n_sigma, int dtype, void *packed, size_t packed_bytes_, void *stream) {
    return flk_kernel_pack(FLK_GAUSSIAN, X, n, d, x_rs, x_cs, sigma, n_sigma, dtype, packed, packed_bytes_, stream);
}

size_t flk_gauss_mmv_packed_workspace_bytes(int64_t n_a, int64_t n_b, int64_t d, int64_t t, int dtype) {
    if (n_a < 0 || n_b < 0 || d < 1 || t < 0 || d > flk_max_d(dtype) || t > flk_max_t() || !known_dtype(dtype, false))
        return 0;
    if (dtype == FLK_F64)
        return planar_bytes<double>(n_a, n_b, d, t) + partial_bytes<double>(n_a, n_b, d, t);
    return planar_bytes<float>(n_a, n_b, d, t) + partial_bytes<float>(n_a, n_b, d, t);
}

int flk_kernel_mmv_packed(int kernel, const void *packed_a, int64_t n_a, const void *packed_b, int64_t n_b, int64_t d,
                          const void *vec, int64_t vec_rs, int64_t vec_cs, int64_t t, const void *addend,
                          int64_t add_rs, int64_t add_cs, void *out, int64_t out_rs, int64_t out_cs, int dtype,
                          void *workspace, size_t workspace_bytes, void *stream) {
    g_err[0] = 0;
    FLK_CHECK_KERNEL(kernel);
    if (dtype == FLK_F32)
        return mmv_packed_impl<float>(kernel, packed_a, n_a, packed_b, n_b, d, vec, vec_rs, vec_cs, t, addend, add_rs,
                                      add_cs, out, out_rs, out_cs, workspace, workspace_bytes, (hipStream_t)stream);
    if (dtype == FLK_F64)
        return mmv_packed_impl<double>(kernel, packed_a, n_a, packed_b, n_b, d, vec, vec_rs, vec_cs, t, addend, add_rs,
                                       add_cs, out, out_rs, out_cs, workspace, workspace_bytes, (hipStream_t)stream);
    return fail(FLK_EINVAL, "unknown dtype %d", dtype);
}

int flk_gauss_mmv_packed(const void *packed_a, int64_t n_a, const void *packed_b, int64_t n_b, int64_t d,
                         const void *vec, int64_t vec_rs, int64_t vec_cs, int64_t t, const void *addend,
                         int64_t add_rs, int64_t add_cs, void *out, int64_t out_rs, int64_t out_cs, int dtype,
                         void *workspace, size_t workspace_bytes, void *stream) {
    return flk_kernel_mmv_packed(FLK_GAUSSIAN, packed_a, n_a, packed_b, n_b, d, vec, vec_rs, vec_cs, t, addend, add_rs,
                                 add_cs, out, out_rs, out_cs, dtype, workspace, workspace_bytes, stream);
}

size_t flk_gauss_fmmv_workspace_bytes(int64_t n, int64_t m, int64_t d, int64_t t, int dtype) {
    if (n < 0 || m < 0 || d < 1 || t < 0 || d > flk_max_d(dtype) || t > flk_max_t() || !known_dtype(dtype, true))
        return 0;
    if (dtype == FLK_F32_BF16X3 && split_applies(d, t)) return fmmv_split_ws_bytes(n, m, d, t);
    return dtype == FLK_F64 ? fmmv_ws_bytes<double>(n, m, d, t) : fmmv_ws_bytes<float>(n, m, d, t);
}

int flk_kernel_fmmv(int kernel, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m,
                    int64_t x2_rs, int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v,
                    int64_t v_rs, int64_t v_cs, int64_t t, void *out, int64_t out_rs, int64_t out_cs, int dtype,
                    void *workspace, size_t workspace_bytes, void *stream) {
    g_err[0] = 0;
    FLK_CHECK_KERNEL(kernel);
    if (dtype == FLK_F32_BF16X3 && split_applies(d, t))
        return fmmv_split_impl(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, t, out,
                               out_rs, out_cs, workspace, workspace_bytes, (hipStream_t)stream);
    if (dtype == FLK_F32 || dtype == FLK_F32_BF16X3)
        return fmmv_impl<float>(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, t,
                                out, out_rs, out_cs, workspace, workspace_bytes, (hipStream_t)stream);
    if (dtype == FLK_F64)
        return fmmv_impl<double>(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, t,
                                 out, out_rs, out_cs, workspace, workspace_bytes, (hipStream_t)stream);
    return fail(FLK_EINVAL, "unknown dtype %d", dtype);
}

int flk_gauss_fmmv(const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m, int64_t x2_rs,
                   int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v, int64_t v_rs,
                   int64_t v_cs, int64_t t, void *out, int64_t out_rs, int64_t out_cs, int dtype, void *workspace,
                   size_t workspace_bytes, void *stream) {
    return flk_kernel_fmmv(FLK_GAUSSIAN, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, t,
                           out, out_rs, out_cs, dtype, workspace, workspace_bytes, stream);
}

size_t flk_gauss_fdmmv_workspace_bytes(int64_t n, int64_t m, int64_t d, int64_t t, int dtype) {
    if (n < 0 || m < 0 || d < 1 || t < 0 || d > flk_max_d(dtype) || t > flk_max_t() || !known_dtype(dtype, true))
        return 0;
    if (dtype == FLK_F32_BF16X3 && split_applies(d, t)) return fdmmv_split_ws_bytes(n, m, d, t);
    return dtype == FLK_F64 ? fdmmv_ws_bytes<double>(n, m, d, t) : fdmmv_ws_bytes<float>(n, m, d, t);
}

int flk_kernel_fdmmv(int kernel, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m,
                     int64_t x2_rs, int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v,
                     int64_t v_rs, int64_t v_cs, const void *w, int64_t w_rs, int64_t w_cs, int64_t t, void *out,
                     int64_t out_rs, int64_t out_cs, int dtype, void *workspace, size_t workspace_bytes,
                     void *stream) {
    g_err[0] = 0;
    FLK_CHECK_KERNEL(kernel);
    if (dtype == FLK_F32_BF16X3 && split_applies(d, t))
        return fdmmv_split_impl(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, w,
                                w_rs, w_cs, t, out, out_rs, out_cs, workspace, workspace_bytes, (hipStream_t)stream);
    if (dtype == FLK_F32 || dtype == FLK_F32_BF16X3)
        return fdmmv_impl<float>(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, w,
                                 w_rs, w_cs, t, out, out_rs, out_cs, workspace, workspace_bytes, (hipStream_t)stream);
    if (dtype == FLK_F64)
        return fdmmv_impl<double>(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, w,
                                  w_rs, w_cs, t, out, out_rs, out_cs, workspace, workspace_bytes, (hipStream_t)stream);
    return fail(FLK_EINVAL, "unknown dtype %d", dtype);
}

int flk_gauss_fdmmv(const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m, int64_t x2_rs,
                    int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v, int64_t v_rs,
                    int64_t v_cs, const void *w, int64_t w_rs, int64_t w_cs, int64_t t, void *out, int64_t out_rs,
                    int64_t out_cs, int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    return flk_kernel_fdmmv(FLK_GAUSSIAN, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, w,
                            w_rs, w_cs, t, out, out_rs, out_cs, dtype, workspace, workspace_bytes, stream);
}

int flk_gauss_fdmmv_noalloc(const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m,
                            int64_t x2_rs, int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, const void *v,
                            int64_t v_rs, int64_t v_cs, const void *w, int64_t w_rs, int64_t w_cs, int64_t t, void *out,
                            int64_t out_rs, int64_t out_cs, int dtype, void *stream) {
    g_err[0] = 0;
    if (n < 0 || m < 0 || d < 1 || t < 0) return fail(FLK_EINVAL, "bad shape");
    if (!known_dtype(dtype, true)) return fail(FLK_EINVAL, "unknown dtype %d", dtype);
    if (d > flk_max_d(dtype)) return fail(FLK_EUNSUPPORTED, "more than %lld features", (long long)flk_max_d(dtype));
    if (t > flk_max_t()) return fail(FLK_EUNSUPPORTED, "more than %lld right-hand sides", (long long)flk_max_t());
    const size_t need = flk_gauss_fdmmv_workspace_bytes(n, m, d, t, dtype);
    if (need > (size_t)FLK_NOALLOC_SCRATCH_BYTES)
        return fail(FLK_ENOMEM,
                    "flk_gauss_fdmmv_noalloc: this problem (n=%lld, m=%lld, d=%lld, t=%lld) needs %zu bytes of scratch "
                    "memory, the built-in array holds %zu; use flk_gauss_fdmmv with a workspace of the caller's",
                    (long long)n, (long long)m, (long long)d, (long long)t, need, (size_t)FLK_NOALLOC_SCRATCH_BYTES);
    void *ws = nullptr;
    int rc = scratch_address(&ws);
    if (rc != FLK_OK) return rc;
    // every byte of the workspace a product reads it has written before in the same call (packed operands, planar
    // vectors including their zero planes, partial sums), so what the previous call left behind needs no clearing
    return flk_kernel_fdmmv(FLK_GAUSSIAN, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, v, v_rs, v_cs, w,
                            w_rs, w_cs, t, out, out_rs, out_cs, dtype, ws, (size_t)FLK_NOALLOC_SCRATCH_BYTES, stream);
}

int64_t flk_cg_state_ints(int64_t t) { return t < 0 ? 0 : 2 + 3 * t; }

int flk_cg_update(int mode, void *X, void *R, void *P, const void *Q, const void *B, int64_t m, int64_t t, int64_t rs,
                  int64_t cs, void *rsold, int32_t *state, int64_t iteration, double eps, double tol2, int differential,
                  int dtype, void *stream) {
    g_err[0] = 0;
    if (mode < 0 || mode > 2) return fail(FLK_EINVAL, "flk_cg_update: mode %d (0: whole iteration, 1 / 2: its halves)", mode);
    if (m < 0 || t < 0 || iteration < 0) return fail(FLK_EINVAL, "flk_cg_update: negative size or iteration");
    if (t > 65535) return fail(FLK_EUNSUPPORTED, "flk_cg_update: more than 65535 right-hand sides");
    if (m == 0 || t == 0) return FLK_OK;
    if (!X || !P || !Q || !rsold || !state || (mode != 1 && !R) || (mode == 2 && !B))
        return fail(FLK_EINVAL, "flk_cg_update: null pointer");
    if (m > 1 && t > 1 && rs != 1 && cs != 1) return fail(FLK_EINVAL, "flk_cg_update: neither stride is one");
    const int parity = (int)(iteration & 1);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == FLK_F32)
        return launch_cg_update<float>(mode, (float *)X, (float *)R, (float *)P, (const float *)Q, (const float *)B, m, t, rs,
                                       cs, (float *)rsold, state, parity, eps, tol2, differential, st);
    if (dtype == FLK_F64)
        return launch_cg_update<double>(mode, (double *)X, (double *)R, (double *)P, (const double *)Q, (const double *)B,
                                        m, t, rs, cs, (double *)rsold, state, parity, eps, tol2, differential, st);
    return fail(FLK_EINVAL, "unknown dtype %d", dtype);
}

int64_t flk_tri_solve_work_elems(int64_t m, int64_t t, int64_t block) {
    if (m < 0 || t < 0 || block < 1) return 0;
    return tri_solve_work_elems(m, t, block);
}

int flk_tri_solve(int dtype, int transposed, const void *L, int64_t m, int64_t ld, int row_major, const void *dinv,
                  const void *dinv_t, int64_t block, const void *b, int64_t ldb, void *x, int64_t ldx, int64_t t,
                  void *work, void *stream) {
    g_err[0] = 0;
    if (m < 0 || t < 0) return fail(FLK_EINVAL, "flk_tri_solve: negative size");
    if (m == 0 || t == 0) return FLK_OK;
    if (block < 4 || block % 4 != 0) return fail(FLK_EINVAL, "flk_tri_solve: block size %lld (a positive multiple of 4)", (long long)block);
    if (ld < m || ldb < m || ldx < m) return fail(FLK_EINVAL, "flk_tri_solve: leading dimension below m");
    if (!L || !dinv || !dinv_t || !b || !x || !work) return fail(FLK_EINVAL, "flk_tri_solve: null pointer");
    if (x == b || work == b || work == x) return fail(FLK_EINVAL, "flk_tri_solve: b, x and work must be distinct buffers");
    if (t > 4) return fail(FLK_EUNSUPPORTED, "flk_tri_solve: %lld right-hand sides (1 .. 4 per call)", (long long)t);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == FLK_F32)
        return launch_tri_solve<float>((const float *)L, m, ld, row_major, (const float *)dinv, (const float *)dinv_t, block,
                                       transposed, (const float *)b, ldb, (float *)x, ldx, t, (float *)work, st);
    if (dtype == FLK_F64)
        return launch_tri_solve<double>((const double *)L, m, ld, row_major, (const double *)dinv, (const double *)dinv_t,
                                        block, transposed, (const double *)b, ldb, (double *)x, ldx, t, (double *)work, st);
    return fail(FLK_EINVAL, "unknown dtype %d", dtype);
}

int64_t flk_potrf_tile_rows(int dtype) { return known_dtype(dtype, false) ? potrf_tile_rows(dtype) : 0; }

int flk_potrf_tile(int dtype, void *A, int64_t n, int64_t lda, void *inv, int64_t ldinv, int *info, int64_t info_base,
                   void *stream) {
    g_err[0] = 0;
    if (n < 0) return fail(FLK_EINVAL, "flk_potrf_tile: negative size");
    if (n == 0) return FLK_OK;
    if (!A || !inv || !info) return fail(FLK_EINVAL, "flk_potrf_tile: null pointer");
    if (lda < n || ldinv < n) return fail(FLK_EINVAL, "flk_potrf_tile: leading dimension below n");
    if (A == inv) return fail(FLK_EINVAL, "flk_potrf_tile: A and inv must be distinct buffers");
    if (info_base < 0 || info_base + n > 0x7fffffff) return fail(FLK_EINVAL, "flk_potrf_tile: info_base out of range");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == FLK_F32) return launch_potrf_tile<float>((float *)A, n, lda, (float *)inv, ldinv, info, (int)info_base, st);
    if (dtype == FLK_F64) return launch_potrf_tile<double>((double *)A, n, lda, (double *)inv, ldinv, info, (int)info_base, st);
    return fail(FLK_EINVAL, "unknown dtype %d", dtype);
}

size_t flk_gauss_fmm_workspace_bytes(int64_t n, int64_t m, int64_t d, int dtype, int compute_f64) {
    if (n < 0 || m < 0 || d < 1 || d > flk_max_d(dtype) || !known_dtype(dtype, true)) return 0;
    if (fmm_split_applies(d, dtype, compute_f64)) return split_packed_bytes(n, d) + split_packed_bytes(m, d);
    if (dtype == FLK_F64 || compute_f64) return packed_bytes<double>(n, d) + packed_bytes<double>(m, d);
    return packed_bytes<float>(n, d) + packed_bytes<float>(m, d);
}

int flk_kernel_fmm(int kernel, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m,
                   int64_t x2_rs, int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, void *out,
                   int64_t out_rs, int64_t out_cs, int dtype, int compute_f64, void *workspace, size_t workspace_bytes,
                   void *stream) {
    g_err[0] = 0;
    FLK_CHECK_KERNEL(kernel);
    hipStream_t st = (hipStream_t)stream;
    if (fmm_split_applies(d, dtype, compute_f64))
        return fmm_split_impl(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, out, out_rs, out_cs,
                              workspace, workspace_bytes, st);
    if (dtype == FLK_F32_BF16X3) dtype = FLK_F32;      // where the mode has no kernel of its own: the fp32 kernels
    if (dtype == FLK_F64)
        return fmm_impl<double, double>(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, out, out_rs,
                                        out_cs, workspace, workspace_bytes, st);
    if (dtype == FLK_F32 && compute_f64)
        return fmm_impl<float, double>(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, out, out_rs,
                                       out_cs, workspace, workspace_bytes, st);
    if (dtype == FLK_F32)
        return fmm_impl<float, float>(kernel, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, out, out_rs,
                                      out_cs, workspace, workspace_bytes, st);
    return fail(FLK_EINVAL, "unknown dtype %d", dtype);
}

int flk_gauss_fmm(const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs, const void *X2, int64_t m, int64_t x2_rs,
                  int64_t x2_cs, int64_t d, const void *sigma, int64_t n_sigma, void *out, int64_t out_rs,
                  int64_t out_cs, int dtype, int compute_f64, void *workspace, size_t workspace_bytes, void *stream) {
    return flk_kernel_fmm(FLK_GAUSSIAN, X1, n, x1_rs, x1_cs, X2, m, x2_rs, x2_cs, d, sigma, n_sigma, out, out_rs, out_cs,
                          dtype, compute_f64, workspace, workspace_bytes, stream);
}

}  // extern "C"

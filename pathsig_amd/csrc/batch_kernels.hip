// Signature backward for word projections with lanes on paths.
//
// The kernels in words_kernels.hip put one lane on each requested word, so every increment ends in a
// sum over lanes per letter.  With a batch of paths there is a cheaper arrangement: a group of G lanes
// holds G paths that all work on the same word, so a lane's per-position gradients go straight into its
// own (increment, letter) cell: no cross-lane sum at all.  A wave carries 64/G such groups side by side,
// each with its own words, and every lane sweeps several words at once.  Every wave has a private slab
// of cells in LDS, [increment of the tile][letter][lane], updated with plain read-add-write (LDS float
// atomics run at a small fraction of the plain LDS rate); the waves of a block share the G paths and
// the staged increments, and after each tile the slabs are added up and flushed to the per-increment
// gradient with one global atomic per (path, increment, letter) and block.  (Two entries of a lane may carry the
// same letter, so the read-add-writes of an increment form a chain, each waiting for the LDS round trip of the one
// before.  Measured alternative: 64 paths to a group, so that a wave's letters are uniform and sit in scalar
// registers, with the per-letter sums formed in sixteen vector registers indexed by those scalars and every cell
// stored once: gfx950 has no relative register moves, the compiler brackets every indexed access with a switch
// of the register-index mode, and the sweep of 2320 words over sixteen letters took 1077 us against 959 us.)
// The arithmetic per word is
// the same chain roll-back and chain adjoint as in words_kernels.hip
// (reference: src/pathsig/backward/sig_backward_kernels.cu:120-342).
#include <cstdlib>

#include "common.hpp"
#include "words_common.hpp"

namespace psig {

namespace {

constexpr int kBatchWaves = 8;
constexpr int kBatchBlock = kBatchWaves * kWave;
constexpr int kBatchStride = kWave + 1;
constexpr int kBatchChunks = 2;  // a tile holds at most kBatchChunks * 64 increments x letters per path

// words swept at once by one lane: chosen so that a wave has about the same work at every word length.  Every
// block pays the same fixed cost per increment (staging, slab flush, barriers), whatever its words cost, and the
// slabs allow one block per CU: the short words of levels 1 and 2 are therefore packed sixteen to a lane, which
// keeps a projection like "two full levels + a few thousand words" within one round of blocks on 256 CUs.
constexpr int batch_words(int deg) {
    return deg <= 2 ? 16 : deg == 3 ? 8 : deg == 4 ? 6 : deg == 5 ? 4 : deg == 6 ? 3 : deg <= 8 ? 2 : 1;
}

// level of block `blk` when the levels are laid out from the deepest down: level k owns
// [block_begin[k], block_begin[k-1]), block_begin[0] being the total
__device__ __forceinline__ int find_level_descending(const LevelPlan &plan, int64_t blk) {
    int deg = plan.depth;
    while (deg > 1 && blk >= plan.block_begin[deg - 1]) --deg;
    return deg;
}

template <typename T, int DEG, int G, typename ACC>
__device__ void batch_backward_body(const T *__restrict__ path, const T *__restrict__ sig,
                                    const T *__restrict__ grad_sig, ACC *__restrict__ grad_inc, const SigShape &shape,
                                    const LevelPlan &plan, const int64_t *__restrict__ codes, int64_t blk_in_level,
                                    int tile, T *sdx, T *slabs) {
    constexpr int WPL = batch_words(DEG);
    constexpr int kSlots = kWave / G;
    // LDS rows hold one value per lane (the increments of a path are repeated for every group of the
    // wave); the odd row stride spreads lanes along the row and lanes along time over the banks
    constexpr int kStride = kBatchStride;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int slot = lane / G, pl = lane % G;
    const int d = (int)shape.d;
    const int64_t group = (int64_t)blockIdx.y / shape.W, w = (int64_t)blockIdx.y - group * shape.W;
    const int64_t b0 = group * G;
    const bool path_ok = b0 + pl < shape.B;
    const int64_t b = path_ok ? b0 + pl : shape.B - 1;
    const WindowSpan span = window_span(shape, w);
    const int64_t row = b * shape.W + w;
    const T *srow = sig + row * plan.sig_size;
    const T *grow = grad_sig + row * plan.sig_size;

    // per word: LDS offsets of the lane's increments, chain at the right end of the window, chain adjoint
    const bool kept_chain = DEG > 1 && !plan.from_saved[DEG] && plan.keep != nullptr && plan.keep_off[DEG] >= 0;
    int aoff[WPL][DEG];
    T p[WPL][DEG + 1], h[WPL][DEG + 1];
#pragma unroll
    for (int i = 0; i < WPL; ++i) {
        const int64_t word_idx = ((blk_in_level * kBatchWaves + wave) * kSlots + slot) * WPL + i;
        const bool have = word_idx < plan.size[DEG];
        uint64_t code = 0;
        if (have) code = plan.code_off[DEG] >= 0 ? (uint64_t)codes[plan.code_off[DEG] + word_idx] : (uint64_t)word_idx;
        int l[DEG];
        decode_letters<DEG>(code, (uint64_t)d, l);
        p[i][0] = T(1);
#pragma unroll
        for (int k = 0; k < DEG; ++k) {
            aoff[i][k] = l[k] * kStride + lane;
            p[i][k + 1] = T(0);
            h[i][k] = T(0);
        }
        h[i][DEG] = (have && path_ok) ? grow[plan.out_off[DEG] + word_idx] : T(0);
        if (plan.from_saved[DEG] && have) {
            uint64_t off = 0, width = (uint64_t)d, pref = 0;
#pragma unroll
            for (int k = 1; k < DEG; ++k) {
                pref = pref * (uint64_t)d + (uint64_t)l[k - 1];
                p[i][k] = srow[off + pref];
                off += width;
                width *= (uint64_t)d;
            }
        } else if (kept_chain && have && path_ok) {
            // the forward of this call kept the chain
            const T *kept = (const T *)plan.keep + row * plan.keep_size + plan.keep_off[DEG] + word_idx * (DEG - 1);
#pragma unroll
            for (int k = 1; k < DEG; ++k) p[i][k] = kept[k - 1];
        }
    }

    // Every wave stages (and later flushes) the paths wave, wave + kBatchWaves, ...; lanes run along time.
    // The path points of the next tile are fetched into registers before the current tile is worked on
    // and turned into increments in LDS after it, so the memory latency hides behind the arithmetic
    // (the loaded values are first touched in commit()).
    constexpr int kPaths = G / kBatchWaves;
    static_assert(G % kBatchWaves == 0, "paths of a group are dealt out evenly to the waves");
    T fetched_hi[kPaths][kBatchChunks], fetched_lo[kPaths][kBatchChunks];
    auto fetch = [&](int64_t t0, int nt) {
#pragma unroll
        for (int pp = 0; pp < kPaths; ++pp) {
            const int q = wave + pp * kBatchWaves;
            const bool ok = b0 + q < shape.B;
            const T *xq = path + ((ok ? b0 + q : 0) * shape.L + span.start + t0) * d;
#pragma unroll
            for (int c = 0; c < kBatchChunks; ++c) {
                const int j = lane + c * kWave;
                const int jc = j < nt * d ? j : 0;
                fetched_hi[pp][c] = xq[jc + d];
                fetched_lo[pp][c] = xq[jc];
            }
        }
    };
    auto commit = [&](int nt) {
#pragma unroll
        for (int pp = 0; pp < kPaths; ++pp) {
            const int q = wave + pp * kBatchWaves;
            const bool ok = b0 + q < shape.B;
#pragma unroll
            for (int c = 0; c < kBatchChunks; ++c) {
                const int j = lane + c * kWave;
                if (j < nt * d) {
                    const T v = ok ? fetched_hi[pp][c] - fetched_lo[pp][c] : T(0);
#pragma unroll
                    for (int g = 0; g < kSlots; ++g) sdx[j * kStride + g * G + q] = v;
                }
            }
        }
    };
    const int slab_size = tile * d * kStride;
    T *slab = slabs + wave * slab_size;
    for (int idx = lane; idx < slab_size; idx += kWave) slab[idx] = T(0);
    const int64_t ntiles = (span.steps + tile - 1) / tile;
    auto tile_steps = [&](int64_t ti) {
        const int64_t left = span.steps - ti * tile;
        return (int)(left < tile ? left : tile);
    };

    if (!plan.from_saved[DEG] && DEG > 1 && ntiles > 0 && !kept_chain) {
        // chain at the right end of the window by a forward sweep (levels < DEG)
        fetch(0, tile_steps(0));
        commit(tile_steps(0));
        for (int64_t ti = 0; ti < ntiles; ++ti) {
            const int nt = tile_steps(ti);
            lds_barrier();
            if (ti + 1 < ntiles) fetch((ti + 1) * tile, tile_steps(ti + 1));
            for (int tt = 0; tt < nt; ++tt) {
                const T *dxr = sdx + tt * d * kStride;
#pragma unroll
                for (int i = 0; i < WPL; ++i) {
                    T dl[DEG];
#pragma unroll
                    for (int k = 0; k < DEG; ++k) dl[k] = dxr[aoff[i][k]];
                    T dq[DEG][DEG];
                    scale_letters<T, DEG>(dl, dq);
                    chain_step<T, DEG, DEG - 1, true>(p[i], dq);
                }
            }
            lds_barrier();
            if (ti + 1 < ntiles) commit(tile_steps(ti + 1));
        }
    }

    if (ntiles > 0) {
        lds_barrier();
        fetch((ntiles - 1) * tile, tile_steps(ntiles - 1));
        commit(tile_steps(ntiles - 1));
    }
    for (int64_t ti = ntiles - 1; ti >= 0; --ti) {
        const int64_t t0 = ti * tile;
        const int nt = tile_steps(ti);
        lds_barrier();
        if (ti > 0) fetch((ti - 1) * tile, tile_steps(ti - 1));
        for (int tt = nt - 1; tt >= 0; --tt) {
            const T *dxr = sdx + tt * d * kStride;
            T *acc = slab + tt * d * kStride;
#pragma unroll
            for (int i = 0; i < WPL; ++i) {
                T dl[DEG], gl[DEG];
#pragma unroll
                for (int k = 0; k < DEG; ++k) dl[k] = dxr[aoff[i][k]];
                // S_t = S_{t+1} (x) exp(-dx_t) on the chain (levels < DEG are all the adjoint needs)
                T dq[DEG][DEG];
                scale_letters<T, DEG>(dl, dq);
                chain_step<T, DEG, DEG - 1, false>(p[i], dq);
                chain_step_adjoint<T, DEG>(p[i], h[i], dl, dq, gl);
                // cells of this lane only, so no atomics; two entries may share a cell (same letter), which
                // keeps the read-add-writes in program order
#pragma unroll
                for (int k = 0; k < DEG; ++k) acc[aoff[i][k]] += gl[k];
            }
        }
        lds_barrier();
        // sum of the slabs (all waves, all groups of a wave) per (path, increment, letter); the cells are
        // cleared by the thread that read them, for the next tile
#pragma unroll
        for (int pp = 0; pp < kPaths; ++pp) {
            const int q = wave + pp * kBatchWaves;
            const bool ok = b0 + q < shape.B;
            ACC *gq = grad_inc + ((ok ? b0 + q : 0) * (shape.L - 1) + span.start + t0) * d;
            for (int j = lane; j < nt * d; j += kWave) {
                // all reads first, so their latencies overlap
                T *cell = slabs + j * kStride + q;
                T part[kBatchWaves * kSlots];
#pragma unroll
                for (int wv = 0; wv < kBatchWaves; ++wv)
#pragma unroll
                    for (int g = 0; g < kSlots; ++g) part[wv * kSlots + g] = cell[wv * slab_size + g * G];
#pragma unroll
                for (int wv = 0; wv < kBatchWaves; ++wv)
#pragma unroll
                    for (int g = 0; g < kSlots; ++g) cell[wv * slab_size + g * G] = T(0);
                T v = T(0);
#pragma unroll
                for (int i = 0; i < kBatchWaves * kSlots; ++i) v += part[i];
                if (ok && v != T(0)) atomicAdd(&gq[j], (ACC)v);
            }
        }
        if (ti > 0) commit(tile_steps(ti - 1));
    }
}

template <typename T, int MAXDEG, int G, typename ACC>
__global__ void __launch_bounds__(kBatchBlock) batch_backward_kernel(const T *__restrict__ path,
                                                                     const T *__restrict__ sig,
                                                                     const T *__restrict__ grad_sig,
                                                                     ACC *__restrict__ grad_inc, SigShape shape,
                                                                     LevelPlan plan, const int64_t *__restrict__ codes,
                                                                     int tile) {
    extern __shared__ __align__(16) unsigned char smem[];
    T *sdx = reinterpret_cast<T *>(smem);
    T *slabs = sdx + (int64_t)tile * shape.d * kBatchStride;
    const int64_t blk = blockIdx.x;
    const int deg = find_level_descending(plan, blk);
    const int64_t bl = blk - plan.block_begin[deg];
    switch (deg) {
#define PSIG_CASE(N)                                                                                                \
    case N:                                                                                                         \
        if constexpr (N <= MAXDEG)                                                                                  \
            batch_backward_body<T, N, G, ACC>(path, sig, grad_sig, grad_inc, shape, plan, codes, bl, tile, sdx, slabs); \
        break;
        PSIG_CASE(1) PSIG_CASE(2) PSIG_CASE(3) PSIG_CASE(4) PSIG_CASE(5) PSIG_CASE(6)
        PSIG_CASE(7) PSIG_CASE(8) PSIG_CASE(9) PSIG_CASE(10) PSIG_CASE(11) PSIG_CASE(12)
#undef PSIG_CASE
        default: break;
    }
}

// LDS bytes of one increment of a tile: the staged increments plus one slab per wave
int64_t batch_lds_per_step(int64_t d, size_t elem) { return (int64_t)(1 + kBatchWaves) * d * kBatchStride * (int64_t)elem; }

// largest dynamic LDS allocation of a block on the current device (64 KB when the query fails)
int64_t max_block_lds() {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 64 * 1024;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || v <= 0) return 64 * 1024;
    return v;
}

template <typename T>
int batch_group(int64_t B) {
    // 32 paths per group when that wastes at most a quarter of the lanes, else 16
    const int64_t padded = (B + 31) / 32 * 32;
    return (B >= 24 && 4 * B >= 3 * padded) ? 32 : 16;
}

}  // namespace

bool batch_backward_usable(size_t elem, int64_t B, int64_t d, int64_t W) {
    if (B < 12) return false;  // too few paths to fill the lanes: the word-per-lane kernel does better
    if (d > kBatchChunks * kWave) return false;  // one increment of a path must fit the staging registers
    if (batch_lds_per_step(d, elem) > max_block_lds()) return false;  // one increment of every slab must fit in LDS
    const int64_t groups = (B + 15) / 16;
    return groups * W <= 65535;
}

template <typename T, typename ACC>
hipError_t launch_batch_backward(const T *path, const T *sig, const T *grad_sig, ACC *grad_inc, const SigShape &shape,
                                 const LevelPlan &plan_in, const int64_t *codes, hipStream_t stream) {
    const int G = batch_group<T>(shape.B);
    LevelPlan plan = plan_in;
    int64_t blocks = 0;
    for (int k = plan.depth; k >= 1; --k) {
        const int64_t per_block = (int64_t)kBatchWaves * (kWave / G) * batch_words(k);
        plan.block_begin[k] = blocks;
        blocks += (plan.size[k] + per_block - 1) / per_block;
    }
    plan.block_begin[0] = blocks;
    const int64_t groups = (shape.B + G - 1) / G;
    if (blocks == 0 || groups * shape.W == 0) return hipSuccess;
    if (blocks >= (int64_t(1) << 31) || groups * shape.W > 65535) return hipErrorInvalidValue;
    const int64_t per_step = batch_lds_per_step(shape.d, sizeof(T));
    int64_t tile = max_block_lds() / per_step;
    if (tile > 8) tile = 8;
    if (tile * shape.d > kBatchChunks * kWave) tile = kBatchChunks * kWave / shape.d;
    if (const int64_t forced = options().batch_tile; forced >= 1 && forced < tile) tile = forced;
    if (tile > shape.L - 1) tile = shape.L - 1;
    if (tile < 1) return hipErrorInvalidValue;
    const size_t lds = (size_t)(tile * per_step);
    const dim3 grid((unsigned)blocks, (unsigned)(groups * shape.W));
    hipError_t attr = hipSuccess;
#define PSIG_LAUNCH(MAXDEG, GG)                                                                                    \
    do {                                                                                                           \
        if (lds > 64 * 1024) attr = allow_dynamic_lds<batch_backward_kernel<T, MAXDEG, GG, ACC>>(lds);             \
        if (attr != hipSuccess) return attr;                                                                       \
        hipLaunchKernelGGL((batch_backward_kernel<T, MAXDEG, GG, ACC>), grid, dim3(kBatchBlock), lds, stream, path, \
                           sig, grad_sig, grad_inc, shape, plan, codes, (int)tile);                                \
    } while (0)
#define PSIG_PICK(GG)                          \
    if (plan.depth <= 3) PSIG_LAUNCH(3, GG);   \
    else if (plan.depth <= 4) PSIG_LAUNCH(4, GG); \
    else if (plan.depth <= 6) PSIG_LAUNCH(6, GG); \
    else if (plan.depth <= 8) PSIG_LAUNCH(8, GG); \
    else PSIG_LAUNCH(12, GG)
    if (G == 32) {
        PSIG_PICK(32);
    } else {
        PSIG_PICK(16);
    }
#undef PSIG_PICK
#undef PSIG_LAUNCH
    return hipGetLastError();
}

// The flush adds one term per block (a slice of the words) to every (path, increment, letter) cell.  On dense levels of
// a million words and more an fp32 cell collects tens of thousands of terms of mixed sign; such calls keep the
// per-increment sums in fp64.
bool batch_wide_sums(size_t elem, const LevelPlan &plan) { return elem == 4 && plan.sig_size >= 65536; }

template hipError_t launch_batch_backward<float, float>(const float *, const float *, const float *, float *,
                                                        const SigShape &, const LevelPlan &, const int64_t *,
                                                        hipStream_t);
template hipError_t launch_batch_backward<float, double>(const float *, const float *, const float *, double *,
                                                         const SigShape &, const LevelPlan &, const int64_t *,
                                                         hipStream_t);
template hipError_t launch_batch_backward<double, double>(const double *, const double *, const double *, double *,
                                                          const SigShape &, const LevelPlan &, const int64_t *,
                                                          hipStream_t);

}  // namespace psig

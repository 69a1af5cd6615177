// Register-tiled kernels for the dense signature (every word up to depth N over D letters).
//
// Work decomposition.  The update S <- S (x) exp(dx) of a word only reads the word's own prefixes, so
// the sub-trie below any prefix u evolves on its own once the chain S(u_1), S(u_1 u_2), .. S(u) is
// known.  A lane owns one prefix u of length P: it keeps the P chain values (recomputed redundantly by
// every lane that shares them) and the whole sub-trie below u (levels P+1..N, sum_k D^k values) in
// registers.  All letters below u are compile-time constants, so every state access is a fixed
// register and the increment of the step is the same for all lanes of the unit: there is no
// inter-lane traffic and no barrier inside the time loop.  One "unit" = one (path, window, time chunk); its
// D^P lanes fill ceil(D^P / 64) wavefronts of one workgroup (of several for the largest shapes), each of
// which stages a tile of increments in LDS.  For the widest alphabets the D children of a prefix (and their
// sub-tries) are dealt to several lanes, K to a lane, so that a lane's state still fits the register file
// (split_children); the letters of a lane's children are then the same for every row of sixteen lanes.
//
// Horner form of one step for target level m (every node is one FMA):
//     tmp_j[w a] = S_j[w a] + (tmp_{j-1}[w] / (m - j + 1)) * dx[a],   j = 1..m-1,   tmp_0 = 1
//     S_m[w a]  += tmp_{m-1}[w] * dx[a]
// evaluated depth-first below the lane's prefix, targets descending so lower levels are still old.
//
// Backward.  With A_t = S_{0,t} and H_t = dL/dS_{0,t}: a reverse sweep rolls A back with exp(-dx_t)
// (levels < N only: the top level of A is never read), back-propagates through the Horner chains of the
// step (which yields H_{t-1} and dL/d(dx_t)), and keeps the top level of H equal to the upstream
// gradient.  Adjoint values of the shared chain nodes stay lane-private partial sums (everything they
// feed is linear in them), so the only cross-lane operation is the final sum of D numbers per step.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdlib>
#include <type_traits>

#include "dense.hpp"

// This file is compiled once per group of shapes (-DPSIG_GROUP=g, g = 0 .. kDenseGroups-1: the kernels of the
// shapes whose index is g modulo kDenseGroups and their launch sequences) and once without a group (the table
// of shapes, the choice of a shape for a call, and the dispatch to the groups), so that the shapes compile in
// parallel.
#ifndef PSIG_GROUP
#define PSIG_GROUP -1
#endif

namespace psig {

namespace {

// compile-time loop: f(std::integral_constant<int, I>) for I in [Begin, End)
template <int Begin, int End, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (Begin < End) {
        f(std::integral_constant<int, Begin>{});
        static_for<Begin + 1, End>(f);
    }
}

// f(std::integral_constant<int, v>) for the one v in [Begin, End] equal to `value` (End when none below it is)
template <int Begin, int End, typename F>
__device__ __forceinline__ void dispatch_value(int value, F &&f) {
    if constexpr (Begin >= End) {
        f(std::integral_constant<int, End>{});
    } else {
        if (value == Begin) f(std::integral_constant<int, Begin>{});
        else dispatch_value<Begin + 1, End>(value, f);
    }
}

constexpr int ipow(int b, int e) { return e <= 0 ? 1 : b * ipow(b, e - 1); }
// number of sub-trie values in levels 1..k below a prefix
constexpr int trie_size(int D, int k) { return k <= 0 ? 0 : ipow(D, k) + trie_size(D, k - 1); }
// values on the first k levels below a lane's prefix when the lane holds K children of the prefix (all D of them
// unless the first level is split between several lanes) and every child's complete sub-trie
constexpr int sub_size(int D, int K, int k) { return k <= 0 ? 0 : K * ipow(D, k - 1) + sub_size(D, K, k - 1); }
// Children of the prefix that one lane holds.  The widest alphabets (d = 28..48 at depth 3, 16..32 at depth 4, 12..16
// at depth 5) split
// them between lanes: with all D children a lane would hold D + D^2 = 156 to 1056 values, with the next longer
// prefix only D.
// Chosen by an estimate of the useful share of a lane's instructions: K / (K + 1.5) for the chain, the per-letter
// sums and the reduction that every lane pays whatever K is, times the share of child slots in use (the last lane
// of a prefix may hold fewer than K), within K * (D + 1) <= 136 values.
constexpr int split_children(int D, int N, int P) {
    // (d = 13 at depth 5 measured slower split, 24.7 against 32.3 TFLOP/s, and keeps all its children in one lane)
    if (!(P == N - 2 && ((N == 3 && D >= 28 && D <= 48) || (N == 4 && D >= 16 && D <= 32) ||
                         (N == 5 && D >= 12 && D <= 16 && D != 13))))
        return D;
    int best = 2;
    long best_num = 0, best_den = 1;
    for (int k = 2; k * (D + 1) <= 136 && k <= 8; ++k) {
        const int parts = (D + k - 1) / k;
        // D / (parts * k) * k / (k + 1.5)  =  2 D / (parts * (2 k + 3))
        const long num = 2L * D, den = (long)parts * (2 * k + 3);
        if (num * best_den >= best_num * den) {
            best = k;
            best_num = num;
            best_den = den;
        }
    }
    return best;
}

template <typename T>
__device__ __forceinline__ constexpr T rcp(int k) { return T(1) / T(k); }

template <typename T>
__device__ __forceinline__ T fmad(T a, T b, T c);
template <>
__device__ __forceinline__ float fmad<float>(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
template <>
__device__ __forceinline__ double fmad<double>(double a, double b, double c) { return __builtin_fma(a, b, c); }

// ---------------------------------------------------------------------------------------------
// one Chen step on a lane's state: chain a[1..P] and sub-trie levels P+1..TOP (TOP <= N)
//
// Below the prefix the division by (m - j + 1) is carried by the increment: dxs[q][a] = dx[a] / (q + 1)
// is staged once per tile, so a sub-trie node is exactly one FMA, tmp_j[w a] = S_j[w a] + tmp_{j-1}[w] * dxs.
// On the chain (P nodes per target) the parent is scaled instead.
// ---------------------------------------------------------------------------------------------
// LO: letters below LO are left out below the prefix (their words are not wanted; see LetterBounds).
// K: children of the prefix held by the lane (D, or fewer when the first level is split between lanes: then dxf
// holds the scaled increments of the lane's own K letters; otherwise dxf is dxs).
template <typename T, int D, int P, int M, int J, bool NEG, int LO = 0, int K = D>
struct StepDescend {
    // children (level J > P) of a node with Horner value pt; idx0 = index of the first child within level J
    template <int SUB, int KS>
    static __device__ __forceinline__ void run(T pt, int idx0, T (&sub)[SUB], const T (&dxs)[KS][D],
                                               const T (&dxf)[KS][K]) {
        constexpr int off = sub_size(D, K, J - P - 1);
        constexpr bool kFirst = J == P + 1;
#pragma unroll
        for (int a = LO; a < (kFirst ? K : D); ++a) {
            T inc;
            if constexpr (kFirst) inc = NEG ? -dxf[M - J][a] : dxf[M - J][a];
            else inc = NEG ? -dxs[M - J][a] : dxs[M - J][a];
            if constexpr (J == M) {
                sub[off + idx0 + a] = fmad<T>(pt, inc, sub[off + idx0 + a]);
            } else {
                const T tmp = fmad<T>(pt, inc, sub[off + idx0 + a]);
                StepDescend<T, D, P, M, J + 1, NEG, LO, K>::template run<SUB, KS>(tmp, (idx0 + a) * D, sub, dxs, dxf);
            }
        }
    }
};

// LO applies to the top target only (the first M of the recursion); the targets below are complete.
template <typename T, int D, int P, int M, bool NEG, int LO = 0, int K = D>
struct StepTargets {
    template <int SUB, int KS>
    static __device__ __forceinline__ void run(T (&a)[P + 1], T (&sub)[SUB], const T (&dxs)[KS][D],
                                               const T (&dxf)[KS][K], const T (&dxp)[P]) {
        T ps = rcp<T>(M);
        T tmp = T(1);
        constexpr int JP = (M - 1 < P) ? (M - 1) : P;
#pragma unroll
        for (int j = 1; j <= JP; ++j) {
            tmp = fmad<T>(ps, NEG ? -dxp[j - 1] : dxp[j - 1], a[j]);
            ps = tmp * rcp<T>(M - j);
        }
        if constexpr (M <= P) {
            a[M] = fmad<T>(ps, NEG ? -dxp[M - 1] : dxp[M - 1], a[M]);
        } else {
            StepDescend<T, D, P, M, P + 1, NEG, LO, K>::template run<SUB, KS>(tmp, 0, sub, dxs, dxf);
        }
        if constexpr (M > 1) StepTargets<T, D, P, M - 1, NEG, 0, K>::template run<SUB, KS>(a, sub, dxs, dxf, dxp);
    }
};

// ---------------------------------------------------------------------------------------------
// adjoint of one Chen step
// ---------------------------------------------------------------------------------------------
template <typename T, int D, int P, int M, int J, int LO = 0, int K = D>
struct AdjDescend {
    // pt = Horner value of the parent; returns its adjoint.  gdxk[q][a] collects the gradient with respect
    // to dxs[q][a]; the caller folds the 1/(q+1) back in.
    template <int ASUB, int HSUB, int KS>
    // (with the first level split between lanes: dxf / gdxf are the increments of the lane's own K letters and
    // their gradients; otherwise they are dxs / gdxk themselves)
    static __device__ __forceinline__ T run(T pt, int idx0, const T (&asub)[ASUB], T (&hsub)[HSUB],
                                            const T (&dxs)[KS][D], const T (&dxf)[KS][K], T (&gdxk)[KS][D],
                                            T (&gdxf)[KS][K]) {
        constexpr int off = sub_size(D, K, J - P - 1);
        constexpr bool kFirst = J == P + 1;
        T gpt = T(0);
#pragma unroll
        for (int a = LO; a < (kFirst ? K : D); ++a) {
            T inc;
            if constexpr (kFirst) inc = dxf[M - J][a];
            else inc = dxs[M - J][a];
            T g;
            if constexpr (J == M) {
                g = hsub[off + idx0 + a];
            } else {
                const T tmp = fmad<T>(pt, inc, asub[off + idx0 + a]);
                g = AdjDescend<T, D, P, M, J + 1, LO, K>::template run<ASUB, HSUB, KS>(tmp, (idx0 + a) * D, asub, hsub,
                                                                                       dxs, dxf, gdxk, gdxf);
                hsub[off + idx0 + a] += g;
            }
            if constexpr (kFirst) gdxf[M - J][a] = fmad<T>(g, pt, gdxf[M - J][a]);
            else gdxk[M - J][a] = fmad<T>(g, pt, gdxk[M - J][a]);
            gpt = fmad<T>(g, inc, gpt);
        }
        return gpt;
    }
};

template <typename T, int D, int N, int P, int M, int LO = 0, int K = D>
struct AdjTargets {
    // targets ascending: the seed of target M (adjoint of level M) is only changed by targets above M;
    // LO applies to the top target (M = N), whose left-out words have a zero upstream gradient
    template <int ASUB, int HSUB, int KS>
    static __device__ __forceinline__ void run(const T (&a)[P + 1], const T (&asub)[ASUB], T (&hc)[P + 1],
                                               T (&hsub)[HSUB], const T (&dxs)[KS][D], const T (&dxf)[KS][K],
                                               const T (&dxp)[P], T (&gdxk)[KS][D], T (&gdxf)[KS][K],
                                               T (&gpre)[P]) {
        constexpr int JP = (M - 1 < P) ? (M - 1) : P;
        T ps[P + 2];
        T tmp = T(1);
        ps[1] = rcp<T>(M);
#pragma unroll
        for (int j = 1; j <= JP; ++j) {
            tmp = fmad<T>(ps[j], dxp[j - 1], a[j]);
            ps[j + 1] = tmp * rcp<T>(M - j);
        }
        T g;
        constexpr int JS = (M <= P) ? M : P;  // chain level where the walk back starts
        if constexpr (M <= P) {
            g = hc[M];
        } else {
            g = AdjDescend<T, D, P, M, P + 1, (M == N ? LO : 0), K>::template run<ASUB, HSUB, KS>(
                tmp, 0, asub, hsub, dxs, dxf, gdxk, gdxf);
            hc[P] += g;
        }
#pragma unroll
        for (int j = JS; j >= 1; --j) {
            gpre[j - 1] = fmad<T>(g, ps[j], gpre[j - 1]);
            if (j > 1) {
                g = g * dxp[j - 1] * rcp<T>(M - j + 1);
                hc[j - 1] += g;
            }
        }
        if constexpr (M < N)
            AdjTargets<T, D, N, P, M + 1, LO, K>::template run<ASUB, HSUB, KS>(a, asub, hc, hsub, dxs, dxf, dxp, gdxk,
                                                                                 gdxf, gpre);
    }
};

// sums over the 16 lanes of a DPP row; every lane of the row ends with the row's sum
__device__ __forceinline__ float row_total(float v) {
    v = dpp_add_c<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v = dpp_add_c<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v = dpp_add_c<0x141, 0xF>(v);  // row_half_mirror
    v = dpp_add_c<0x140, 0xF>(v);  // row_mirror
    return v;
}

__device__ __forceinline__ double row_total(double v) {
    v = dpp_add_c<0xB1, 0xF>(v);
    v = dpp_add_c<0x4E, 0xF>(v);
    v = dpp_add_c<0x141, 0xF>(v);
    v = dpp_add_c<0x140, 0xF>(v);
    return v;
}

// Sums of D values (D = 2, 4, 8 or 16) over the 16 lanes of a DPP row, all at once: the first
// log2(D) exchange steps halve the number of values a lane carries (a lane keeps the half selected by one
// of its index bits and adds its partner's copy of that half), the remaining steps add single values.
// Exchange partners are lane^1, lane^2, lane^8, lane^4, in that order.  Afterwards every lane holds the
// row total of letter row_letter<D>(lane); the lanes with row_writer<D>(lane) cover each letter once.
template <typename T>
__device__ __forceinline__ T dpp_take_xor4(T v) {
    // lane^4: banks 0 and 2 of the row read four lanes up, banks 1 and 3 four lanes down
    if constexpr (sizeof(T) == 4) {
        int x = __builtin_bit_cast(int, v);
        int r = __builtin_amdgcn_update_dpp(0, x, 0x104, 0xF, 0x5, false);   // row_shl:4
        r = __builtin_amdgcn_update_dpp(r, x, 0x114, 0xF, 0xA, false);       // row_shr:4
        return __builtin_bit_cast(T, r);
    } else {
        const long long bits = __builtin_bit_cast(long long, v);
        const int xl = (int)(bits & 0xffffffffll), xh = (int)(bits >> 32);
        int rl = __builtin_amdgcn_update_dpp(0, xl, 0x104, 0xF, 0x5, false);
        rl = __builtin_amdgcn_update_dpp(rl, xl, 0x114, 0xF, 0xA, false);
        int rh = __builtin_amdgcn_update_dpp(0, xh, 0x104, 0xF, 0x5, false);
        rh = __builtin_amdgcn_update_dpp(rh, xh, 0x114, 0xF, 0xA, false);
        return __builtin_bit_cast(T, ((long long)rh << 32) | (long long)(unsigned)rl);
    }
}

template <int CTRL, typename T>
__device__ __forceinline__ T dpp_take(T v) {
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
    } else {
        const long long bits = __builtin_bit_cast(long long, v);
        const int lo = __builtin_amdgcn_update_dpp(0, (int)(bits & 0xffffffffll), CTRL, 0xF, 0xF, false);
        const int hi = __builtin_amdgcn_update_dpp(0, (int)(bits >> 32), CTRL, 0xF, 0xF, false);
        return __builtin_bit_cast(T, ((long long)hi << 32) | (long long)(unsigned)lo);
    }
}

// partner's value for exchange step S (0: lane^1, 1: lane^2, 2: lane^8, 3: lane^4)
template <int S, typename T>
__device__ __forceinline__ T row_partner(T v) {
    if constexpr (S == 0) return dpp_take<0xB1>(v);        // quad_perm [1,0,3,2]
    else if constexpr (S == 1) return dpp_take<0x4E>(v);   // quad_perm [2,3,0,1]
    else if constexpr (S == 2) return dpp_take<0x128>(v);  // row_ror:8
    else return dpp_take_xor4(v);
}

// lane bit that selects the kept half in exchange step S
__device__ __forceinline__ constexpr int row_step_bit(int S) { return S == 0 ? 1 : S == 1 ? 2 : S == 2 ? 8 : 4; }

template <int D>
constexpr int log2_of() { return D == 1 ? 0 : 1 + log2_of<D / 2>(); }

template <int D>
__device__ __forceinline__ int row_letter(int lane) {
    int k = 0;
#pragma unroll
    for (int s = 0; s < log2_of<D>(); ++s) k += (lane & row_step_bit(s)) ? (D >> (s + 1)) : 0;
    return k;
}

template <int D>
__device__ __forceinline__ bool row_writer(int lane) {
    bool w = true;
#pragma unroll
    for (int s = log2_of<D>(); s < 4; ++s) w = w && !(lane & row_step_bit(s));
    return w;
}

template <typename T, int D, int S = 0, int LIVE = D>
__device__ __forceinline__ T row_totals(T (&v)[D], int lane) {
    if constexpr (S == 4) {
        return v[0];
    } else if constexpr (LIVE > 1) {
        const bool upper = (lane & row_step_bit(S)) != 0;
#pragma unroll
        for (int i = 0; i < LIVE / 2; ++i) {
            const T keep = upper ? v[i + LIVE / 2] : v[i];
            const T send = upper ? v[i] : v[i + LIVE / 2];
            v[i] = keep + row_partner<S>(send);
        }
        return row_totals<T, D, S + 1, LIVE / 2>(v, lane);
    } else {
        v[0] += row_partner<S>(v[0]);
        return row_totals<T, D, S + 1, 1>(v, lane);
    }
}

// Letter bounds of a set of top-level words: bounds[a] = the smallest letter that occurs after the first
// letter in any wanted word that starts with a (D when no word starts with a).  A word a w_2 .. w_N with
// some w_j < bounds[a] is therefore not wanted, and the sweeps leave its sub-trie node out.  The bound has
// to be the same for all lanes of a wave, which holds when the lanes of a wave share their first letter.
template <int D, int P>
struct LetterBounds {
    static constexpr int kPerLetter = ipow(D, P - 1);  // lanes that share a first letter
    // (units of more than 1024 lanes take several blocks and are swept without bounds)
    static constexpr bool kUsable = P >= 1 && kPerLetter % kWave == 0 && ipow(D, P) <= 1024;
    static __device__ __forceinline__ int of_wave(const int *__restrict__ bounds, int pu) {
        const int first = __builtin_amdgcn_readfirstlane(pu / kPerLetter);
        const int lo = bounds[first];
        return lo < 0 ? 0 : (lo > D ? D : lo);
    }
    // Prefix of thread tid.  The first letters are dealt to the waves in the order 0, 1, .., D/2-1, D-1, .., D/2:
    // bounds tend to grow with the first letter (Lyndon words), and waves that are four apart tend to share a
    // SIMD, so this pairs a long sweep with a short one.
    static __device__ __forceinline__ int prefix_of_thread(int tid) {
        const int first = tid / kPerLetter;
        const int dealt = first < D / 2 ? first : D - 1 - (first - D / 2);
        return dealt * kPerLetter + (tid - first * kPerLetter);
    }
};

// bounds[0..d) from the codes of the top-level words (one block; d <= 16)
template <typename C>
__device__ __forceinline__ void least_later_letter(C c, C d, int depth, int &first, int &least) {
    least = (int)d;
    for (int j = 1; j < depth; ++j) {
        const C q = c / d;
        const int letter = (int)(c - q * d);
        c = q;
        least = letter < least ? letter : least;
    }
    first = (int)(c % d);
}

__device__ __forceinline__ void letter_bounds_block(const int64_t *__restrict__ codes, int64_t count, int d,
                                                    int depth, bool narrow, int *__restrict__ bounds) {
    __shared__ int lo[16];
    if (threadIdx.x < 16) lo[threadIdx.x] = d;
    __syncthreads();
    for (int64_t i = threadIdx.x; i < count; i += blockDim.x) {
        int first, least;
        // codes below 2^32 are taken apart with 32-bit divisions
        if (narrow) least_later_letter<uint32_t>((uint32_t)codes[i], (uint32_t)d, depth, first, least);
        else least_later_letter<uint64_t>((uint64_t)codes[i], (uint64_t)d, depth, first, least);
        if (least < lo[first]) atomicMin(&lo[first], least);
    }
    __syncthreads();
    if ((int)threadIdx.x < d) bounds[threadIdx.x] = lo[threadIdx.x];
}

__global__ void __launch_bounds__(1024)
    letter_bounds_kernel(const int64_t *__restrict__ codes, int64_t count, int d, int depth, bool narrow,
                         int *__restrict__ bounds) {
    letter_bounds_block(codes, count, d, depth, narrow, bounds);
}

// The last block computes the letter bounds (when asked for: bounds != nullptr), the others clear ptr[0..n).
template <typename T>
__global__ void __launch_bounds__(1024)
    zero_and_bounds_kernel(T *__restrict__ ptr, int64_t n, const int64_t *__restrict__ codes, int64_t count, int d,
                           int depth, bool narrow, int *__restrict__ bounds) {
    if (blockIdx.x + 1 == gridDim.x) {
        if (bounds) letter_bounds_block(codes, count, d, depth, narrow, bounds);
        return;
    }
    zero_span<T>(ptr, n, (int64_t)blockIdx.x * blockDim.x + threadIdx.x, (int64_t)(gridDim.x - 1) * blockDim.x);
}

struct Span {
    int64_t start, steps;
};

__device__ __forceinline__ Span unit_span(const SigShape &shape, int64_t w) {
    int64_t start = 0, end = shape.L;
    if (shape.windows) {
        start = shape.windows[2 * w];
        end = shape.windows[2 * w + 1];
        start = start < 0 ? 0 : (start > shape.L ? shape.L : start);
        end = end < 0 ? 0 : (end > shape.L ? shape.L : end);
    }
    int64_t steps = end - start - 1;
    return {start, steps < 0 ? 0 : steps};
}

// chunk c of `chunks` equal parts of a span: steps [begin, end)
// (64-bit divisions are some thirty scalar instructions each, in front of every unit's first load: spans of less
// than 2^31 steps, that is all spans met in practice, take one 32-bit division and small ones for the remainder)
__device__ __forceinline__ void chunk_range(int64_t steps, int chunks, int c, int64_t &begin, int64_t &end) {
    if (steps < (int64_t(1) << 31) && chunks <= 32768) {
        // floor(steps * c / chunks) = q * c + floor(r * c / chunks) with steps = q * chunks + r
        const unsigned q = (unsigned)steps / (unsigned)chunks, r = (unsigned)steps - q * (unsigned)chunks;
        begin = (int64_t)q * c + (r * (unsigned)c) / (unsigned)chunks;
        end = (int64_t)q * (c + 1) + (r * (unsigned)(c + 1)) / (unsigned)chunks;
    } else {
        begin = steps * c / chunks;
        end = steps * (c + 1) / chunks;
    }
}

// quotient and remainder of a block or row index (always below 2^31: a grid dimension) by a small positive divisor
__device__ __forceinline__ void divide_index(int64_t index, int64_t by, int64_t &quotient, int64_t &remainder) {
    if (index < (int64_t(1) << 31) && by < (int64_t(1) << 31)) {
        const unsigned q = (unsigned)index / (unsigned)by;
        quotient = q;
        remainder = (unsigned)index - q * (unsigned)by;
    } else {
        quotient = index / by;
        remainder = index - quotient * by;
    }
}

constexpr int kTile = 64;  // increments staged in LDS at a time

// Place of letter a in a staged row of increments.  The vector register file has two banks (register parity), and
// an instruction whose two multiplicands sit in the same bank takes 2.5 times as long.  The increments of a step
// arrive in registers by 16-byte LDS reads, the leaves of a lane's sub-trie and their adjoints by 16-byte loads:
// both land in aligned runs of registers, letter a in a register of parity a % 2, and the leaf updates multiply
// exactly those pairs (adjoint of the leaf with letter a times increment a: 90 % of them were conflicts, a third
// of all conflicts of the reverse sweep).  For fp32 alphabets of whole 16-byte rows the increments are therefore
// staged with every two neighbours swapped and read back in whole rows, which puts increment a into a register of
// the other parity (c2 reverse sweep 77.1 -> 74.8 us on one box; its forward sweep 37.2 -> 37.6).
template <typename T, int D>
__device__ __forceinline__ constexpr int inc_slot(int a) { return (D % 4 == 0 && sizeof(T) == 4) ? (a ^ 1) : a; }

// Stages nt increments as sdx[(tt * KS + q) * D + inc_slot(a)] = (x[tt+1][a] - x[tt][a]) / (q + 1).
// (the loads of four rounds are issued before the first of them is waited for: the points come from memory, and a
// chunk of 64 increments over four letters is four rounds of a wave)
template <typename T, int D, int KS, int BLOCK>
__device__ __forceinline__ void stage_increments(T *sdx, const T *__restrict__ xw, int nt, int tid) {
    constexpr int kRounds = 4;
    const int count = nt * D;
    for (int first = 0; first < count; first += kRounds * BLOCK) {
        T later[kRounds], earlier[kRounds];
#pragma unroll
        for (int i = 0; i < kRounds; ++i) {
            // (an index beyond the end reads the last element again: loads under a condition would be branches,
            // and a load the compiler cannot see consumed on every path is waited for at its register's next
            // use, together with every store issued since)
            const int idx = first + i * BLOCK + tid;
            const int at = idx < count ? idx : count - 1;
            later[i] = xw[at + D];
            earlier[i] = xw[at];
        }
#pragma unroll
        for (int i = 0; i < kRounds; ++i) {
            const int idx = first + i * BLOCK + tid;
            if (idx < count) {
                const T inc = later[i] - earlier[i];
                const int tt = idx / D, a = idx - tt * D;
#pragma unroll
                for (int q = 0; q < KS; ++q) sdx[(tt * KS + q) * D + inc_slot<T, D>(a)] = inc * rcp<T>(q + 1);
            }
        }
    }
    // Every load above has been consumed.  Saying so (s_waitcnt vmcnt(0), which waits for nothing here) keeps the
    // compiler from waiting later, where it cannot tell any more and global stores are in flight that the wait
    // would include.
    __builtin_amdgcn_s_waitcnt(0x0F70);
}

template <typename T, int D, int P, int KS>
__device__ __forceinline__ void read_increments(const T *sdx, int tt, const int (&u)[P], T (&dxs)[KS][D], T (&dxp)[P]) {
    if constexpr (sizeof(T) == 4 && D % 4 == 0) {
        // whole 16-byte reads, so that the swapped neighbours land in one aligned run of four registers
        typedef T V4 __attribute__((ext_vector_type(4)));
        const V4 *rows = reinterpret_cast<const V4 *>(sdx + tt * KS * D);
#pragma unroll
        for (int q = 0; q < KS; ++q)
#pragma unroll
            for (int g = 0; g < D / 4; ++g) {
                const V4 v = rows[q * (D / 4) + g];
#pragma unroll
                for (int e = 0; e < 4; ++e) dxs[q][4 * g + e] = v[inc_slot<T, D>(e)];
            }
    } else {
#pragma unroll
        for (int q = 0; q < KS; ++q)
#pragma unroll
            for (int k = 0; k < D; ++k) dxs[q][k] = sdx[(tt * KS + q) * D + inc_slot<T, D>(k)];
    }
#pragma unroll
    for (int j = 0; j < P; ++j) dxp[j] = sdx[tt * KS * D + inc_slot<T, D>(u[j])];
}

// scaled increments of the K letters a0 .. a0 + K - 1 (zero beyond the alphabet); a0 is the same for a whole wave
template <typename T, int D, int K, int KS, int FQ, int FK>
__device__ __forceinline__ void read_first_level(const T *sdx, int tt, int a0, T (&dxf)[FQ][FK]) {
    static_assert(FQ == KS && FK == K, "only called where the first level is split");
#pragma unroll
    for (int q = 0; q < KS; ++q)
#pragma unroll
        for (int i = 0; i < K; ++i) dxf[q][i] = a0 + i < D ? sdx[(tt * KS + q) * D + inc_slot<T, D>(a0 + i)] : T(0);
}

constexpr int pow2_divisor(int d) { return (d % 2 == 0) ? 2 * pow2_divisor(d / 2) : 1; }

template <int D, int N, int P, int ELEM = 4, int MAXW = 0>
struct Geometry {
    // A lane holds kK children of its prefix: all D, or fewer where the first level below the prefix is split
    // between kParts lanes (split_children).  The lanes of a part are padded to whole rows of sixteen lanes (the unit
    // of the per-letter sums), so the part, and with it the letters of the lane's children, is the same for all lanes
    // of such a row.
    static constexpr int kK = split_children(D, N, P);
    static constexpr bool kSplit = kK < D;
    static constexpr int kParts = (D + kK - 1) / kK;
    static constexpr int kPrefixes = ipow(D, P);
    static constexpr int kPartLanes = kSplit ? (kPrefixes + 15) / 16 * 16 : kPrefixes;
    static constexpr int kLanes = kSplit ? kParts * kPartLanes : kPrefixes;
    // A unit needs kUnitWaves waves.  Up to sixteen of them form one block; a larger unit is spread over
    // kUnitBlocks blocks (its lanes never talk to each other inside a sweep; the per-increment sums of the
    // backward then meet in memory).  Such shapes are swept in one piece, without time chunks.
    static constexpr int kUnitWaves = (kLanes + kWave - 1) / kWave;
    // waves of one block: sixteen at most, eight when the lane's sub-trie is large (a block of sixteen waves leaves
    // each lane 128 registers, which the reverse sweep of such a shape overflows), four from 160 values on (one
    // wave per SIMD: 512 registers, the upper half reached through copies); a unit that needs several blocks
    // anyway takes the smaller block from a smaller sub-trie on
    static constexpr int kSubTrie = sub_size(D, kK, N - P);
    static constexpr int kMaxWaves32 =
        (kSubTrie > 160 || (kSplit && kSubTrie > 128)) ? 4
        : (kSubTrie > 40 || (kUnitWaves > 16 && kSubTrie > 30)) ? 8 : 16;
    // fp64 doubles the registers of a lane's state.  Where the unit is spread over several blocks anyway (or,
    // with three levels below the prefix, would fill more than eight waves), the blocks shrink until the state
    // fits: the reverse sweeps of these shapes spilled 200 to 400 registers to memory in blocks of eight or
    // sixteen waves.  Units of one block keep their shape (they may be cut into time chunks).
    static constexpr bool kSplit64 = ELEM == 8 && (kUnitWaves > kMaxWaves32 || (N - P >= 3 && kUnitWaves > 8));
    // MAXW > 0: blocks of at most MAXW waves whatever the sub-trie (the sweeps with letter bounds run one wave to
    // a block: see kLetterBlocks)
    static constexpr int kMaxWaves =
        MAXW > 0 ? MAXW
        : !kSplit64 ? kMaxWaves32
        : (kSubTrie >= 72 || N - P >= 3 || (kSubTrie >= 56 && P >= 6)) ? 4
        : kSubTrie >= 30 ? (kMaxWaves32 < 8 ? kMaxWaves32 : 8) : kMaxWaves32;
    // a unit of several blocks deals its waves out evenly (18 waves: three blocks of six, not 8 + 8 + 2 with six
    // waves that sweep nothing)
    static constexpr int kUnitBlocks = (kUnitWaves + kMaxWaves - 1) / kMaxWaves;
    static constexpr int kWaves = (kUnitWaves + kUnitBlocks - 1) / kUnitBlocks;
    static constexpr int kBlock = kWaves * kWave;
    static constexpr int kFwdSub = sub_size(D, kK, N - P);    // sub-trie levels P+1..N
    static constexpr int kASub = sub_size(D, kK, N - 1 - P);  // levels P+1..N-1
    // swept in one piece, never cut into time chunks: units of several blocks, and units with split children (the
    // products of chunk signatures are not written for them)
    static constexpr bool kOnePiece = kUnitBlocks > 1 || kSplit;
    // Sweeps with letter bounds: the waves of a unit differ in the words they leave out, by a factor of ten and
    // more between the first letter 0 and the last, and a wave cannot issue faster than every fourth clock, so
    // inside one block the unit takes as long as its longest wave takes alone.  With MAXW = 1 every wave is a block
    // of its own (the unit's lanes never talk to each other inside a sweep; their per-increment sums meet in
    // memory), the blocks of the longest waves are launched first, and the short ones fill in behind them.
    static constexpr bool kLetterBlocks = MAXW > 0;
    static __host__ __device__ constexpr int64_t level_off(int k) {  // first column of level k in the dense layout
        int64_t o = 0, w = 1;
        for (int i = 1; i < k; ++i) {
            w *= D;
            o += w;
        }
        return o;
    }
    static constexpr int64_t kSigSize = level_off(N + 1);
    static constexpr int64_t kLowSize = level_off(N);  // levels 1..N-1
};

// letters of the lane's prefix, most significant first
template <int D, int P>
__device__ __forceinline__ void prefix_letters(int pu, int (&u)[P]) {
#pragma unroll
    for (int j = P - 1; j >= 0; --j) {
        u[j] = pu % D;
        pu /= D;
    }
}

// Unit of the block, and which of the unit's blocks it is.  The blocks of a unit follow each other in the grid,
// except in a launch of letter blocks: there all first blocks come first, then all second ones, .. (the blocks
// with the smallest first letters, which leave out the fewest words, start first).
template <typename G>
__device__ __forceinline__ int64_t unit_of_block() {
    if constexpr (G::kLetterBlocks) return (int64_t)(blockIdx.x % (gridDim.x / (unsigned)G::kUnitBlocks));
    else return G::kUnitBlocks > 1 ? (int64_t)blockIdx.x / G::kUnitBlocks : (int64_t)blockIdx.x;
}
template <typename G>
__device__ __forceinline__ int part_of_block() {
    if constexpr (G::kLetterBlocks) return (int)(blockIdx.x / (gridDim.x / (unsigned)G::kUnitBlocks));
    else return (int)(blockIdx.x % (unsigned)G::kUnitBlocks);
}

// ---------------------------------------------------------------------------------------------
// Place of the elements of a dense-layout row that lives in LDS.
// The lanes of a wave hold consecutive prefixes, so they touch such a row at addresses D^r elements apart (r = 1,
// 2, ..): for an alphabet that is a power of two these strides are multiples of the 64 LDS banks from D^r = 64 on,
// and all lanes of a 16-byte access meet in four banks (measured on (4, 6): a product of two chunk signatures
// through LDS took 10 000 clocks for 500 multiply-adds per lane).  SKEW rows are therefore stored with four
// elements of padding after every 64, counted from a shifted origin that puts the first element of every level of
// 64 words and more on a multiple of 64: a run of D^r elements that starts at a multiple of D^r within its level
// then lies in one piece (D^r <= 64) or starts a block of 64 (D^r > 64), so its elements keep offsets known at
// compile time, and lanes 64 elements apart are four banks apart.
// ---------------------------------------------------------------------------------------------
template <int D, bool SKEW>
struct RowPlace {
    static constexpr bool kOn = SKEW && D % 4 == 0 && (D & (D - 1)) == 0 && D <= 64;
    static constexpr int shift() {
        if (!kOn) return 0;
        int below = 0, w = D;  // words of the levels whose size is not a multiple of 64
        while (w % 64 != 0) {
            below += w;
            w *= D;
        }
        return (64 - below % 64) % 64;
    }
    static constexpr int kShift = shift();
    static __host__ __device__ constexpr int pos(int idx) {
        if (!kOn) return idx;
        const int j = idx + kShift;
        return j + ((j >> 6) << 2);
    }
    // element iv of a run that starts at pos(first) with first a multiple of the run's length within its level
    static __host__ __device__ constexpr int in_run(int iv) { return kOn ? iv + ((iv >> 6) << 2) : iv; }
    // elements of LDS that a row of `count` elements takes
    static constexpr int size(int count) { return kOn ? (pos(count - 1) + 4) / 4 * 4 : count; }
};

// ---------------------------------------------------------------------------------------------
// lane state <-> dense layout in memory
// ---------------------------------------------------------------------------------------------
// Reads the chain a[1..P] and the sub-trie levels P+1..TOP of prefix pu from a dense-layout row.
// K < D: the lane holds the children a0 .. a0 + K - 1 of its prefix only (those beyond the alphabet read as zero).
// SKEW: the row lives in LDS in the layout of RowPlace (whole sets of children only).
template <typename T, int D, int P, int TOP, int SUB, int K = D, bool SKEW = false>
__device__ __forceinline__ void load_state(const T *__restrict__ row, int pu, bool active, T (&a)[P + 1], T (&sub)[SUB],
                                           int a0 = 0) {
    using G = Geometry<D, TOP, P>;
    using RP = RowPlace<D, SKEW>;
    static_assert(!RP::kOn || K == D, "skewed rows hold whole sets of children");
    int rest = 1;
#pragma unroll
    for (int j = P; j >= 1; --j) {
        a[j] = active ? row[RP::pos((int)G::level_off(j) + pu / rest)] : T(0);
        rest *= D;
    }
    static_for<1, TOP - P + 1>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        constexpr int below = ipow(D, k - 1);  // words of this level below one child
        constexpr int off = sub_size(D, K, k - 1);
        const T *src = RP::kOn ? row + RP::pos((int)G::level_off(P + k) + pu * D * below)
                               : row + G::level_off(P + k) + ((int64_t)pu * D + a0) * below;
#pragma unroll
        for (int i = 0; i < K * below; ++i) {
            const bool have = K == D || a0 + i / below < D;
            sub[off + i] = (active && have) ? src[RP::in_run(i)] : T(0);
        }
    });
}

template <typename T, int D, int P, int TOP, int SUB, int K = D, bool SKEW = false>
__device__ __forceinline__ void store_state(T *__restrict__ row, int pu, const T (&a)[P + 1], const T (&sub)[SUB],
                                            int a0 = 0) {
    using G = Geometry<D, TOP, P>;
    using RP = RowPlace<D, SKEW>;
    static_assert(!RP::kOn || K == D, "skewed rows hold whole sets of children");
    // Every lane writes its chain values: lanes that share a chain node computed it with the same
    // operations, so they store identical bits, and no branch is needed.
    int rest = 1;
#pragma unroll
    for (int j = P; j >= 1; --j) {
        row[RP::pos((int)G::level_off(j) + pu / rest)] = a[j];
        rest *= D;
    }
    static_for<1, TOP - P + 1>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        constexpr int below = ipow(D, k - 1);
        constexpr int off = sub_size(D, K, k - 1);
        T *dst = RP::kOn ? row + RP::pos((int)G::level_off(P + k) + pu * D * below)
                         : row + G::level_off(P + k) + ((int64_t)pu * D + a0) * below;
#pragma unroll
        for (int i = 0; i < K * below; ++i)
            if (K == D || a0 + i / below < D) dst[RP::in_run(i)] = sub[off + i];
    });
}

// codes of the sub-words u_{k+1..i} of the lane's prefix, 0 <= k < i <= P
template <int D, int P>
struct SubWords {
    int code[P + 1][P + 1];
    __device__ __forceinline__ explicit SubWords(const int (&u)[P]) {
#pragma unroll
        for (int k = 0; k <= P; ++k) {
            int c = 0;
#pragma unroll
            for (int i = 0; i <= P; ++i) {
                if (i > k) c = c * D + u[i - 1];
                code[k][i] = c;
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------
// A <- A (x) B on a lane's state (chain + sub-trie levels P+1..TOP); B is a dense-layout row.
//   (A (x) B)(u v) = sum_{k<=P} A(u_1..u_k) B(u_{k+1}..u_P v) + sum_{j<|v|} A(u v_1..v_j) B(v_{j+1}..) + A(u v)
// Sub-trie levels go top-down and the chain last, so everything read is still the old A.
// ---------------------------------------------------------------------------------------------
template <typename T, int D, int P, int TOP, int SUB, bool SKEW = false>
__device__ __forceinline__ void apply_right(T (&a)[P + 1], T (&sub)[SUB], const T *__restrict__ B,
                                            const SubWords<D, P> &sw) {
    using G = Geometry<D, TOP, P>;
    using RP = RowPlace<D, SKEW>;
    a[0] = T(1);
    static_for<0, TOP - P>([&](auto rc) {
        constexpr int r = TOP - P - decltype(rc)::value;  // TOP-P .. 1
        constexpr int width = ipow(D, r);
        constexpr int off = trie_size(D, r - 1);
        T acc[width];
#pragma unroll
        for (int iv = 0; iv < width; ++iv) acc[iv] = sub[off + iv];
        // own sub-trie values times the low words of B
        static_for<1, r>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            constexpr int tail = ipow(D, r - j);
            constexpr int offj = trie_size(D, j - 1);
#pragma unroll
            for (int iv = 0; iv < width; ++iv)
                acc[iv] = fmad<T>(sub[offj + iv / tail], B[RP::pos((int)G::level_off(r - j) + iv % tail)], acc[iv]);
        });
        // chain values times B at (suffix of the prefix) . v
        static_for<0, P + 1>([&](auto kc) {
            constexpr int k = decltype(kc)::value;
            const T *run = RP::kOn ? B + RP::pos((int)G::level_off(P - k + r) + sw.code[k][P] * width)
                                   : B + G::level_off(P - k + r) + (int64_t)sw.code[k][P] * width;
#pragma unroll
            for (int iv = 0; iv < width; ++iv) acc[iv] = fmad<T>(a[k], run[RP::in_run(iv)], acc[iv]);
        });
#pragma unroll
        for (int iv = 0; iv < width; ++iv) sub[off + iv] = acc[iv];
    });
#pragma unroll
    for (int i = P; i >= 1; --i) {
        T acc = a[i];
#pragma unroll
        for (int k = 0; k < i; ++k) acc = fmad<T>(a[k], B[RP::pos((int)G::level_off(i - k) + sw.code[k][i])], acc);
        a[i] = acc;
    }
}

// ---------------------------------------------------------------------------------------------
// H <- H contracted on the right with B:  H'(w) = sum_s H(w s) B(s),  B(empty) = 1.
// State: lane-private chain partials hc[1..P], sub-trie levels P+1..N (the top level never changes).
// B is a dense-layout row with levels 1..N-1.  The chain goes first (ascending), then the sub-trie
// levels top-down in depth, so everything read is still the old H.
// ---------------------------------------------------------------------------------------------
template <typename T, int D, int N, int P, int HSUB, bool SKEW = false>
__device__ __forceinline__ void contract_right(T (&hc)[P + 1], T (&hsub)[HSUB], const T *__restrict__ B,
                                               const SubWords<D, P> &sw) {
    using G = Geometry<D, N, P>;
    using RP = RowPlace<D, SKEW>;
    constexpr int R = N - P;
#pragma unroll
    for (int i = 1; i <= P; ++i) {
        T acc = hc[i];
#pragma unroll
        for (int i2 = i + 1; i2 <= P; ++i2)
            acc = fmad<T>(hc[i2], B[RP::pos((int)G::level_off(i2 - i) + sw.code[i][i2])], acc);
        static_for<1, R + 1>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            constexpr int width = ipow(D, r);
            constexpr int off = trie_size(D, r - 1);
            const T *run = RP::kOn ? B + RP::pos((int)G::level_off(P - i + r) + sw.code[i][P] * width)
                                   : B + G::level_off(P - i + r) + (int64_t)sw.code[i][P] * width;
#pragma unroll
            for (int iv = 0; iv < width; ++iv) acc = fmad<T>(hsub[off + iv], run[RP::in_run(iv)], acc);
        });
        hc[i] = acc;
    }
    static_for<1, R>([&](auto rc) {
        constexpr int r = decltype(rc)::value;  // 1 .. R-1
        constexpr int width = ipow(D, r);
        constexpr int off = trie_size(D, r - 1);
        static_for<1, R - r + 1>([&](auto qc) {
            constexpr int q = decltype(qc)::value;  // extension length
            constexpr int ext = ipow(D, q);
            constexpr int offq = trie_size(D, r + q - 1);
#pragma unroll
            for (int iv = 0; iv < width; ++iv) {
                T acc = hsub[off + iv];
#pragma unroll
                for (int e = 0; e < ext; ++e)
                    acc = fmad<T>(hsub[offq + iv * ext + e], B[RP::pos((int)G::level_off(q) + e)], acc);
                hsub[off + iv] = acc;
            }
        });
    });
}

// ---------------------------------------------------------------------------------------------
// forward: a block holds GW consecutive time chunks of one row, one chunk per group of kBlock threads.
// Each group sweeps its chunk; the GW chunk signatures are then multiplied together inside the block
// (pairwise, through LDS), so only one dense-layout row per block goes to memory.
// ---------------------------------------------------------------------------------------------
template <int D, int N, int P, int GW, typename T>
constexpr size_t forward_lds_bytes() {
    using G = Geometry<D, N, P, sizeof(T)>;
    return (size_t)GW * kTile * (N - P) * D * sizeof(T) +
           (size_t)(GW / 2) * RowPlace<D, true>::size((int)G::kSigSize) * sizeof(T);
}

// LDS layout of the forward sweep: staged increments per chunk, and slots for the in-block products
template <typename T, int D, int N, int P, int GW, int MAXW = 0>
struct ForwardShape {
    using G = Geometry<D, N, P, sizeof(T), MAXW>;
    static constexpr int KS = N - P;
    static constexpr int kSlots = GW / 2 > 0 ? GW / 2 : 1;
    static constexpr int kSlotSize = GW > 1 ? RowPlace<D, true>::size((int)G::kSigSize) : 4;  // skewed rows
    static constexpr int kStage = kTile * KS * D;  // staged increments of one chunk
    // Grouped hand-over (blocks of four chunks, fp32): the block also leaves the products of its chunks with the
    // chunks to their left and to their right inside the block (below the top level), which takes one more row below
    // the top level in LDS.
    static constexpr int kLowRow = RowPlace<D, true>::size((int)G::kLowSize);
    static constexpr bool kGrouped =
        GW == 4 && sizeof(T) == 4 && MAXW == 0 && N >= 4 && N - 1 >= P && !G::kOnePiece &&
        ((size_t)GW * kStage + (size_t)kSlots * kSlotSize + kLowRow) * sizeof(T) <= 64 * 1024;
    static constexpr int kLowSlot = kGrouped ? kLowRow : 4;
};

// zero_rows (optional, GW = 1): the block also clears the points of its chunk in a [B, L, D] buffer (the last
// chunk of a row clears the final point too); the backward uses this to prepare the path gradient.
// chunk_low (optional): [rows, chunks, levels below N] receives every chunk's own signature below the top level.
// BOUND: top-level words with a letter below BOUND after the prefix's first letter are left out (they stay zero
// in the output); the LDS arrays belong to the calling kernel.
template <typename T, int D, int N, int P, int GW, int BOUND, int MAXW = 0>
__device__ __forceinline__ void dense_forward_body(const T *__restrict__ path, T *__restrict__ out,
                                                   const SigShape &shape, int chunks, T *__restrict__ zero_rows,
                                                   T *__restrict__ chunk_low,
                                                   const int pu,   // prefix of the thread within its chunk
                                                   const int tid,  // index of the thread within its chunk's block part
                                                   T (&sdx_all)[GW][ForwardShape<T, D, N, P, GW, MAXW>::kStage],
                                                   T (&slot)[ForwardShape<T, D, N, P, GW, MAXW>::kSlots]
                                                            [ForwardShape<T, D, N, P, GW, MAXW>::kSlotSize],
                                                   T (&lowslot)[ForwardShape<T, D, N, P, GW, MAXW>::kLowSlot],
                                                   T *__restrict__ group_suffix) {
    using G = Geometry<D, N, P, sizeof(T), MAXW>;
    using FS = ForwardShape<T, D, N, P, GW, MAXW>;
    constexpr int KS = N - P;
    const int part = (int)threadIdx.x / G::kBlock;  // chunk within the block
    T *sdx = sdx_all[part];
    // first level split between lanes: pu counts (part of the children, prefix); pp is the prefix
    constexpr int KF = G::kK, FQ = G::kSplit ? KS : 1, FK = G::kSplit ? KF : 1;
    const int spart = G::kSplit ? pu / G::kPartLanes : 0;
    const int pp = G::kSplit ? pu - spart * G::kPartLanes : pu;
    const int a0 = spart * KF;
    const bool active = G::kSplit ? (pp < G::kPrefixes && spart < G::kParts)
                                  : ((G::kLanes == G::kBlock) || pu < G::kLanes);
    int u[P];
    prefix_letters<D, P>(active ? pp : 0, u);

    const int groups = chunks / GW;  // blocks per row
    const int64_t blk = unit_of_block<G>();
    int64_t row, group_of_row, b, w;
    divide_index(blk, groups, row, group_of_row);
    const int c = (int)group_of_row * GW + part;
    divide_index(row, shape.W, b, w);
    const Span span = unit_span(shape, w);
    int64_t begin, end;
    chunk_range(span.steps, chunks, c, begin, end);
    const T *x = path + (b * shape.L + span.start) * D;
    // every chunk of the row has floor or ceil of steps/chunks increments: the longest sets the number
    // of tile rounds for the whole block, so all threads meet at the same barriers
    int64_t longest, longest_rest;
    divide_index(span.steps + chunks - 1, chunks, longest, longest_rest);
    if constexpr (GW == 1) {
        if (zero_rows) {
            const int64_t points = end - begin + (c == chunks - 1 ? 1 : 0);
            T *z = zero_rows + (b * shape.L + span.start + begin) * D;
            if (pu == tid)  // the first block of the unit
                for (int64_t idx = tid; idx < points * D; idx += G::kBlock) z[idx] = T(0);
        }
    }

    T a[P + 1];
    T sub[G::kFwdSub];
#pragma unroll
    for (int j = 0; j <= P; ++j) a[j] = T(0);
#pragma unroll
    for (int i = 0; i < G::kFwdSub; ++i) sub[i] = T(0);

    for (int64_t off = 0; off < longest; off += kTile) {
        const int64_t t0 = begin + off;
        const int64_t left = end - t0;
        const int nt = (int)(left < 0 ? 0 : (left < kTile ? left : kTile));
        const T *xw = x + t0 * D;
        lds_barrier();
        stage_increments<T, D, KS, G::kBlock>(sdx, xw, nt, tid);
        lds_barrier();
        if (nt > 0) {
            // two register sets of increments: the LDS reads of the next step are issued before the
            // arithmetic of the current one, so their latency hides behind it
            T dxs0[KS][D], dxp0[P], dxs1[KS][D], dxp1[P];
            T dxf0[FQ][FK], dxf1[FQ][FK];
            auto read = [&](int at, T (&dxs)[KS][D], T (&dxp)[P], T (&dxf)[FQ][FK]) {
                read_increments<T, D, P, KS>(sdx, at, u, dxs, dxp);
                if constexpr (G::kSplit) read_first_level<T, D, KF, KS>(sdx, at, a0, dxf);
            };
            auto step = [&](const T (&dxs)[KS][D], const T (&dxp)[P], const T (&dxf)[FQ][FK]) {
                if constexpr (G::kSplit)
                    StepTargets<T, D, P, N, false, BOUND, KF>::template run<G::kFwdSub, KS>(a, sub, dxs, dxf, dxp);
                else
                    StepTargets<T, D, P, N, false, BOUND>::template run<G::kFwdSub, KS>(a, sub, dxs, dxs, dxp);
            };
            // (one set where two would not fit the register file beside the lane's state: fp64 over the widest
            // alphabets, whose sweep otherwise keeps part of its state in scratch memory)
            // (nor beside the hundred and more children of a lane over the widest alphabets)
            constexpr bool kTwoSets = (sizeof(T) == 4 && D <= 64 && !G::kLetterBlocks) ||
                                      (sizeof(T) == 8 && 2 * (G::kFwdSub + 2 * (KS * D + FQ * FK + P)) <= 384);
            if constexpr (kTwoSets) {
                read(0, dxs0, dxp0, dxf0);
                int tt = 0;
                for (; tt + 1 < nt; tt += 2) {
                    read(tt + 1, dxs1, dxp1, dxf1);
                    step(dxs0, dxp0, dxf0);
                    read(tt + 2 < nt ? tt + 2 : tt + 1, dxs0, dxp0, dxf0);
                    step(dxs1, dxp1, dxf1);
                }
                if (tt < nt) step(dxs0, dxp0, dxf0);
            } else {
                for (int tt = 0; tt < nt; ++tt) {
                    read(tt, dxs0, dxp0, dxf0);
                    step(dxs0, dxp0, dxf0);
                }
            }
        }
    }
    if constexpr (FS::kGrouped) {
        if (group_suffix != nullptr) {
            // Grouped hand-over.  The four chunks of the block are c0 .. c3; chunk_low receives, per chunk j, the
            // product c0 (x) .. (x) cj, group_suffix the product c(j+1) (x) .. (x) c3 (nothing for j = 3: the
            // identity), both below the top level; `out` receives the product of all four as before.  The products
            // that the block's result does not need run on the waves that would otherwise wait:
            //   first    wave 0: c0 (x) c1          wave 2: c2 (x) c3
            //   then     wave 0: (c0 c1) (x) (c2 c3)   wave 1: c1 (x) (c2 c3)   wave 3: (c0 c1) (x) c2   (the last two
            //            below the top level)
            constexpr int kLow = (int)G::kLowSize;
            const SubWords<D, P> sw(u);
            T *prefix_at = chunk_low + (row * chunks + c) * kLow;
            T *suffix_at = group_suffix + (row * chunks + c) * kLow;
            if (part == 0 && active) store_state<T, D, P, N - 1, G::kFwdSub>(prefix_at, pu, a, sub);
            if (part == 3 && active) store_state<T, D, P, N - 1, G::kFwdSub>(suffix_at - kLow, pu, a, sub);
            if (part == 1 && active) store_state<T, D, P, N, G::kFwdSub, D, true>(slot[0], pu, a, sub);
            if (part == 3 && active) store_state<T, D, P, N, G::kFwdSub, D, true>(slot[1], pu, a, sub);
            if (part == 2 && active) store_state<T, D, P, N - 1, G::kFwdSub, D, true>(lowslot, pu, a, sub);
            lds_barrier();
            if (part == 0) apply_right<T, D, P, N, G::kFwdSub, true>(a, sub, slot[0], sw);
            if (part == 2) apply_right<T, D, P, N, G::kFwdSub, true>(a, sub, slot[1], sw);
            lds_barrier();
            if (part == 0 && active) {
                store_state<T, D, P, N - 1, G::kFwdSub>(prefix_at + kLow, pu, a, sub);
                store_state<T, D, P, N - 1, G::kFwdSub, D, true>(slot[1], pu, a, sub);
            }
            if (part == 2 && active) {
                store_state<T, D, P, N - 1, G::kFwdSub>(suffix_at - kLow, pu, a, sub);
                store_state<T, D, P, N, G::kFwdSub, D, true>(slot[0], pu, a, sub);
            }
            lds_barrier();
            if (part == 0) {
                apply_right<T, D, P, N, G::kFwdSub, true>(a, sub, slot[0], sw);
                if (active) {
                    store_state<T, D, P, N - 1, G::kFwdSub>(prefix_at + 3 * kLow, pu, a, sub);
                    store_state<T, D, P, N, G::kFwdSub>(out + blk * G::kSigSize, pu, a, sub);
                }
            }
            if (part == 1) {
                apply_right<T, D, P, N - 1, G::kFwdSub, true>(a, sub, slot[0], sw);
                if (active) store_state<T, D, P, N - 1, G::kFwdSub>(suffix_at - kLow, pu, a, sub);
            }
            if (part == 3) {
                load_state<T, D, P, N - 1, G::kFwdSub, D, true>(slot[1], pu, active, a, sub);
                apply_right<T, D, P, N - 1, G::kFwdSub, true>(a, sub, lowslot, sw);
                if (active) store_state<T, D, P, N - 1, G::kFwdSub>(prefix_at - kLow, pu, a, sub);
            }
            return;
        }
    }
    if constexpr (N - 1 >= P) {
        // the chunk's own signature below the top level, kept for the backward of the same call
        if (chunk_low != nullptr && active)
            store_state<T, D, P, N - 1, G::kFwdSub, KF>(chunk_low + (row * chunks + c) * G::kLowSize, pp, a, sub, a0);
    }
    if constexpr (GW > 1) {
        const SubWords<D, P> sw(u);
#pragma unroll
        for (int stride = 1; stride < GW; stride *= 2) {
            const int pair = part / (2 * stride);
            const bool right = (part % (2 * stride)) == stride;
            const bool left = (part % (2 * stride)) == 0;
            lds_barrier();
            if (right && active) store_state<T, D, P, N, G::kFwdSub, D, true>(slot[pair], pu, a, sub);
            lds_barrier();
            if (left) apply_right<T, D, P, N, G::kFwdSub, true>(a, sub, slot[pair], sw);
        }
        if (part == 0 && active) store_state<T, D, P, N, G::kFwdSub>(out + blk * G::kSigSize, pu, a, sub);
    } else {
        if (active) store_state<T, D, P, N, G::kFwdSub, KF>(out + blk * G::kSigSize, pp, a, sub, a0);
    }
}

// BOUNDED: `bounds` holds the letter bounds of the wanted top-level words (see LetterBounds).  Every wave runs
// the copy of the sweep compiled for its bound; the copies differ in nothing but the sub-trie nodes they leave
// out, so all waves of the block still meet at the same barriers.  MAXW = 1: letter blocks, one wave to a block
// (Geometry::kLetterBlocks).
template <typename T, int D, int N, int P, int GW, bool BOUNDED = false, int MAXW = 0>
__global__ void __launch_bounds__((Geometry<D, N, P, sizeof(T), MAXW>::kBlock * GW))
    dense_forward_kernel(const T *__restrict__ path, T *__restrict__ out, SigShape shape, int chunks,
                         T *__restrict__ zero_rows = nullptr, const int *__restrict__ bounds = nullptr,
                         T *__restrict__ chunk_low = nullptr, T *__restrict__ group_suffix = nullptr) {
    using FS = ForwardShape<T, D, N, P, GW, MAXW>;
    static_assert(!BOUNDED || LetterBounds<D, P>::kUsable, "letter bounds need one first letter per wave");
    __shared__ __align__(16) T sdx_all[GW][FS::kStage];
    __shared__ __align__(16) T slot[FS::kSlots][FS::kSlotSize];
    __shared__ __align__(16) T lowslot[FS::kLowSlot];
    using G = Geometry<D, N, P, sizeof(T), MAXW>;
    static_assert(!G::kOnePiece || (GW == 1 && BOUNDED == G::kLetterBlocks),
                  "a unit of several blocks is swept one chunk to a block; with letter bounds, in letter blocks");
    const int tid = (int)threadIdx.x % G::kBlock;
    if constexpr (BOUNDED) {
        const int pu = G::kLetterBlocks ? tid + part_of_block<G>() * G::kBlock : LetterBounds<D, P>::prefix_of_thread(tid);
        const int lo = LetterBounds<D, P>::of_wave(bounds, pu);
        dispatch_value<0, D>(lo, [&](auto loc) {
            dense_forward_body<T, D, N, P, GW, decltype(loc)::value, MAXW>(path, out, shape, chunks, zero_rows,
                                                                           chunk_low, pu, tid, sdx_all, slot, lowslot,
                                                                           (T *)nullptr);
        });
    } else {
        const int pu = G::kUnitBlocks > 1 ? tid + part_of_block<G>() * G::kBlock : tid;
        dense_forward_body<T, D, N, P, GW, 0, MAXW>(path, out, shape, chunks, zero_rows, chunk_low, pu, tid, sdx_all,
                                                    slot, lowslot, group_suffix);
    }
}

// ---------------------------------------------------------------------------------------------
// staging of one dense-layout row (COUNT elements) through registers into LDS
// ---------------------------------------------------------------------------------------------
// native vector types (the HIP float4 wrappers do not stay in registers as array elements)
template <typename T, int VW>
struct VecOf {
    typedef T type __attribute__((ext_vector_type(VW)));
};
template <typename T>
struct VecOf<T, 1> {
    typedef T type;
};

// Rows start at multiples of COUNT elements from a 256-byte aligned base, so a row can be moved in
// 16-byte pieces exactly when COUNT * sizeof(T) is a multiple of 16.
template <typename T, int COUNT, int BLOCK>
struct RowStager {
    static constexpr int kMaxVW = 16 / (int)sizeof(T);
    static constexpr int kVW = (COUNT % kMaxVW == 0) ? kMaxVW : ((kMaxVW == 4 && COUNT % 2 == 0) ? 2 : 1);
    using V = typename VecOf<T, kVW>::type;
    static constexpr int kVecs = COUNT / kVW;
    static constexpr int kPer = (kVecs + BLOCK - 1) / BLOCK;
    static constexpr int kPadded = kPer * BLOCK * kVW;  // elements an LDS buffer must hold
    V regs[kPer];
    __device__ __forceinline__ void fetch(const T *__restrict__ src) {
        const V *v = reinterpret_cast<const V *>(src);
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int idx = i * BLOCK + (int)threadIdx.x;
            regs[i] = v[idx < kVecs ? idx : kVecs - 1];  // unconditional, so the array stays in registers
        }
    }
    // dst must have room for kPadded elements: the tail of the last pass lands in the padding
    __device__ __forceinline__ void commit(T *dst) const {
        V *v = reinterpret_cast<V *>(dst);
#pragma unroll
        for (int i = 0; i < kPer; ++i) v[i * BLOCK + (int)threadIdx.x] = regs[i];
    }
    // the same into a buffer of exactly COUNT elements
    __device__ __forceinline__ void commit_exact(T *dst) const {
        V *v = reinterpret_cast<V *>(dst);
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int idx = i * BLOCK + (int)threadIdx.x;
            if (idx < kVecs) v[idx] = regs[i];
        }
    }
    // into a row in the skewed layout of RowPlace<D, true>
    template <int D>
    __device__ __forceinline__ void commit_skewed(T *dst) const {
        using RP = RowPlace<D, true>;
        V *v = reinterpret_cast<V *>(dst);
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int idx = i * BLOCK + (int)threadIdx.x;
            if (idx < kVecs) v[RP::pos(idx * kVW) / kVW] = regs[i];
        }
    }
};

// product of the chunk signatures of one row, left to right.  Lanes sit on prefixes of length P (one
// more letter than in the sweep kernels, for more lanes per row).  Chunks are fetched into registers
// kAhead products before they are needed and handed over through a double buffer in LDS.
// BLOCK: threads that work on a row together (all lanes of the row, or a part of them when the row is spread over
// several blocks, each of which stages the whole right factor for itself)
template <typename T, int D, int N, int P, int BLOCK = Geometry<D, N, P>::kBlock>
struct CombineShape {
    using G = Geometry<D, N, P>;
    static constexpr int kStage = RowStager<T, (int)G::kSigSize, BLOCK>::kPadded;
    static constexpr size_t kBytes = 2 * (size_t)kStage * sizeof(T);
};

// (the first BLOCK threads of the block, on the lanes lane_base .. lane_base + BLOCK - 1 of the row; sB: two buffers
// of CombineShape::kStage elements)
// running_low (optional): [rows, chunks, levels below N] receives, at chunk c >= 1, the product of the chunks before
// c below the top level.
template <typename T, int D, int N, int P, int BLOCK = Geometry<D, N, P>::kBlock>
__device__ __forceinline__ void combine_staged(const T *__restrict__ chunk_sig, T *__restrict__ sig, int chunks,
                                               int64_t row, T *sB0, T *sB1, int lane_base = 0,
                                               T *__restrict__ running_low = nullptr) {
    using G = Geometry<D, N, P>;
    constexpr int kAhead = 3;
    const int pu = lane_base + (int)threadIdx.x;
    const bool active = (G::kLanes == G::kBlock) || pu < G::kLanes;
    int u[P];
    prefix_letters<D, P>(active ? pu : 0, u);
    const SubWords<D, P> sw(u);
    const T *rows = chunk_sig + row * chunks * G::kSigSize;
    T a[P + 1];
    T sub[G::kFwdSub];
    load_state<T, D, P, N, G::kFwdSub>(rows, pu, active, a, sub);
    // Register set q holds chunk c with (c - 1) % kAhead == q.  Fetches past the last chunk re-read the
    // last chunk instead of branching, so the waits on them stay exact counts.
    const int last = chunks - 1;
    RowStager<T, (int)G::kSigSize, BLOCK> stager[kAhead];
    static_for<0, kAhead>([&](auto qc) {
        constexpr int q = decltype(qc)::value;
        stager[q].fetch(rows + (int64_t)(1 + q < last ? 1 + q : last) * G::kSigSize);
    });
    stager[0].commit(sB1);
    stager[0].fetch(rows + (int64_t)(1 + kAhead < last ? 1 + kAhead : last) * G::kSigSize);
    lds_barrier();
    for (int base = 1; base < chunks; base += kAhead) {
        static_for<0, kAhead>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            constexpr int qn = (q + 1) % kAhead;  // register set of the next chunk
            const int c = base + q;
            if (c < chunks) {
                if constexpr (N - 1 >= P) {
                    if (running_low != nullptr && active)
                        store_state<T, D, P, N - 1, G::kFwdSub>(running_low + (row * chunks + c) * G::kLowSize, pu, a, sub);
                }
                apply_right<T, D, P, N, G::kFwdSub>(a, sub, (c & 1) ? sB1 : sB0, sw);
                stager[qn].commit(((c + 1) & 1) ? sB1 : sB0);
                const int nxt = c + 1 + kAhead;
                stager[qn].fetch(rows + (int64_t)(nxt < last ? nxt : last) * G::kSigSize);
                lds_barrier();
            }
        });
    }
    if (active) store_state<T, D, P, N, G::kFwdSub>(sig + row * G::kSigSize, pu, a, sub);
}

// bounds (optional, not STAGED): the letter bounds of the sweep that made the chunk signatures.  A lane whose prefix
// has a letter below the bound of its first letter after that first letter can only reach top-level words that the
// sweep has left out: where the lanes sit on prefixes of length N - 1, it multiplies its chain and neither reads nor
// writes anything above it (the row it leaves in `sig` is then undefined at those words, which no wanted word's
// column maps to).
template <typename T, int D, int N, int P, bool STAGED>
__global__ void __launch_bounds__((Geometry<D, N, P>::kBlock))
    dense_combine_kernel(const T *__restrict__ chunk_sig, T *__restrict__ sig, int chunks,
                         const int *__restrict__ bounds = nullptr) {
    using G = Geometry<D, N, P>;
    constexpr int kStage = STAGED ? CombineShape<T, D, N, P>::kStage : 4;
    __shared__ __align__(16) T sB[2][kStage];
    if constexpr (STAGED) {
        combine_staged<T, D, N, P>(chunk_sig, sig, chunks, (int64_t)blockIdx.x, sB[0], sB[1]);
    } else {
        // without staging the lanes are independent: the row is spread over gridDim.y blocks
        const int pu = (int)(blockIdx.y * blockDim.x + threadIdx.x);
        const bool active = (G::kLanes == G::kBlock) || pu < G::kLanes;
        int u[P];
        prefix_letters<D, P>(active ? pu : 0, u);
        const SubWords<D, P> sw(u);
        const int64_t row = blockIdx.x;
        const T *rows = chunk_sig + row * chunks * G::kSigSize;
        T a[P + 1];
        T sub[G::kFwdSub];
        // (only where the sub-trie of a lane is the top level alone: the levels below it are never left out)
        bool above = true;  // the lane's sub-trie holds words that the sweep has not left out
        if (bounds != nullptr && P == N - 1) {
            const int lo = bounds[u[0]];
#pragma unroll
            for (int i = 1; i < P; ++i) above = above && u[i] >= lo;
        }
        if (above) {
            load_state<T, D, P, N, G::kFwdSub>(rows, pu, active, a, sub);
            for (int c = 1; c < chunks; ++c)
                apply_right<T, D, P, N, G::kFwdSub>(a, sub, rows + (int64_t)c * G::kSigSize, sw);
            if (active) store_state<T, D, P, N, G::kFwdSub>(sig + row * G::kSigSize, pu, a, sub);
        } else {
            // the chain alone (same operations as in load_state, apply_right and store_state)
            int rest = 1;
#pragma unroll
            for (int j = P; j >= 1; --j) {
                a[j] = active ? rows[G::level_off(j) + pu / rest] : T(0);
                rest *= D;
            }
            a[0] = T(1);
            for (int c = 1; c < chunks; ++c) {
                const T *B = rows + (int64_t)c * G::kSigSize;
#pragma unroll
                for (int i = P; i >= 1; --i) {
                    T acc = a[i];
#pragma unroll
                    for (int k = 0; k < i; ++k) acc = fmad<T>(a[k], B[G::level_off(i - k) + sw.code[k][i]], acc);
                    a[i] = acc;
                }
            }
            if (active) {
                T *out = sig + row * G::kSigSize;
                rest = 1;
#pragma unroll
                for (int j = P; j >= 1; --j) {
                    out[G::level_off(j) + pu / rest] = a[j];
                    rest *= D;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------------------------
// Adjoint state of a lane at the right end of a row: the upstream gradient (read like a signature state with
// load_state).  Chain entries are lane-private partial sums, so only the lane whose remaining prefix letters are
// zero keeps what it read.
template <typename T, int D, int P>
__device__ __forceinline__ void adjoint_chain_of_lane(int pu, int a0, T (&hc)[P + 1]) {
    int rest = 1;
#pragma unroll
    for (int j = P; j >= 1; --j) {
        // (of the lanes that split the children of one prefix, the first one)
        if (pu % rest != 0 || a0 != 0) hc[j] = T(0);
        rest *= D;
    }
    hc[0] = T(0);
}

// Per row, from the chunk signatures S_c (levels 1..N-1, dense-layout rows): the signature up to the
// right edge of every chunk, and the signature from there to the end of the row.
//   blockIdx.y == 0:  edgeA_c = S_0 (x) .. (x) S_c            (state in registers, multiplied on the right)
//   blockIdx.y == 1:  edgeZ_c = S_{c+1} (x) .. (x) S_{C-1}      (state in LDS, multiplied on the left:
//                     the lanes load S_c as their state and multiply it by the running product)
// Chunk signatures pass through a double buffer in LDS.  The first kBlock threads do the algebra and
// only ever wait on their own prefetches; the results of a round are left in LDS and copied to global
// memory during the next round by kCopyThreads extra threads, whose stores nobody waits for.
constexpr int kCopyThreads = 128;

// Copies one dense-layout row of COUNT elements with THREADS threads, in 16-byte pieces where the row
// size allows; all loads of a thread are issued before its first store.
// SKEW_D > 0: dst is a row in LDS in the layout of RowPlace<SKEW_D, true> (a piece never straddles its padding:
// the pieces are at most four elements, and the layout moves whole groups of four).
template <typename T, int COUNT, int THREADS, int SKEW_D = 0>
__device__ __forceinline__ void copy_row(const T *src, T *dst, int tid) {
    using Stager = RowStager<T, COUNT, THREADS>;
    using V = typename Stager::V;
    using RP = RowPlace<(SKEW_D > 0 ? SKEW_D : 4), (SKEW_D > 0)>;
    const V *s = reinterpret_cast<const V *>(src);
    V *d = reinterpret_cast<V *>(dst);
    V regs[Stager::kPer];
#pragma unroll
    for (int i = 0; i < Stager::kPer; ++i) {
        const int idx = i * THREADS + tid;
        regs[i] = s[idx < Stager::kVecs ? idx : Stager::kVecs - 1];
    }
#pragma unroll
    for (int i = 0; i < Stager::kPer; ++i) {
        const int idx = i * THREADS + tid;
        if (idx < Stager::kVecs) d[RP::kOn ? RP::pos(idx * Stager::kVW) / Stager::kVW : idx] = regs[i];
    }
}

template <typename T, int COUNT>
__device__ __forceinline__ void copy_row_out(const T *src_lds, T *__restrict__ dst, int tid) {
    copy_row<T, COUNT, kCopyThreads>(src_lds, dst, tid);
}

// RESIDENT: all chunk rows of the row are first copied into dynamic LDS in one burst (one memory latency
// for the whole scan); otherwise they stream through a double buffer, one chunk ahead.
template <typename T, int D, int N, int P, bool RESIDENT>
__global__ void __launch_bounds__((Geometry<D, N, P>::kBlock + kCopyThreads))
    dense_scan_kernel(const T *__restrict__ chunk_low, T *__restrict__ edgeA, T *__restrict__ edgeZ, int chunks,
                      T *__restrict__ zero_rows = nullptr, int64_t row_elems = 0) {
    using G = Geometry<D, N, P>;
    using Stager = RowStager<T, (int)G::kLowSize, G::kBlock>;
    constexpr int kAS = G::kASub > 0 ? G::kASub : 1;
    constexpr int kLow = (int)G::kLowSize;
    constexpr int kThreads = G::kBlock + kCopyThreads;
    extern __shared__ __align__(16) unsigned char scan_smem[];
    __shared__ __align__(16) T sB[RESIDENT ? 1 : 2][RESIDENT ? 4 : Stager::kPadded];
    __shared__ __align__(16) T sOut[2][kLow];
    T *sAll = reinterpret_cast<T *>(scan_smem);  // RESIDENT: [chunks][kLow]
    const bool copier = threadIdx.x >= G::kBlock;
    const int ctid = (int)threadIdx.x - G::kBlock;
    const int pu = copier ? 0 : (int)threadIdx.x;
    const bool active = !copier && ((G::kLanes == G::kBlock) || pu < G::kLanes);
    int u[P];
    prefix_letters<D, P>(active ? pu : 0, u);
    const SubWords<D, P> sw(u);
    const int64_t row = blockIdx.x;
    if (zero_rows) {
        // the two blocks of a row clear one half each of the row's row_elems values in a second buffer (the path
        // gradient, which the reverse sweep then accumulates into)
        const int64_t half = (row_elems + 1) / 2;
        const int64_t first = (int64_t)blockIdx.y * half;
        const int64_t last = first + half < row_elems ? first + half : row_elems;
        T *z = zero_rows + row * row_elems;
        for (int64_t i = first + threadIdx.x; i < last; i += kThreads) z[i] = T(0);
    }
    const T *rows = chunk_low + row * chunks * kLow;
    const int last = chunks - 1;
    if constexpr (RESIDENT) {
#pragma unroll 8
        for (int c = 0; c < chunks; ++c)
            copy_row<T, kLow, kThreads>(rows + (int64_t)c * kLow, sAll + (int64_t)c * kLow, (int)threadIdx.x);
    }
    auto chunk_ptr = [&](int c) -> const T * {
        if constexpr (RESIDENT) return sAll + (int64_t)c * kLow;
        else return sB[c & 1];
    };
    Stager stager;
    T a[P + 1];
    T asub[kAS];
    if (blockIdx.y == 0) {
        T *edge = edgeA + row * chunks * kLow;
        if (!copier) {
            load_state<T, D, P, N - 1, kAS>(rows, pu, active, a, asub);
            if constexpr (!RESIDENT) {
                stager.fetch(rows + (int64_t)(1 < last ? 1 : last) * kLow);
                stager.commit(sB[1]);
                stager.fetch(rows + (int64_t)(2 < last ? 2 : last) * kLow);
            }
            if (active) store_state<T, D, P, N - 1, kAS>(sOut[0], pu, a, asub);
        }
        lds_barrier();
        for (int c = 1; c < chunks; ++c) {
            if (!copier) {
                apply_right<T, D, P, N - 1, kAS>(a, asub, chunk_ptr(c), sw);
                if constexpr (!RESIDENT) {
                    stager.commit(sB[(c + 1) & 1]);
                    stager.fetch(rows + (int64_t)(c + 2 < last ? c + 2 : last) * kLow);
                }
                if (active) store_state<T, D, P, N - 1, kAS>(sOut[c & 1], pu, a, asub);
            } else {
                copy_row_out<T, kLow>(sOut[(c - 1) & 1], edge + (int64_t)(c - 1) * kLow, ctid);
            }
            lds_barrier();
        }
        if (copier) copy_row_out<T, kLow>(sOut[last & 1], edge + (int64_t)last * kLow, ctid);
    } else {
        T *edge = edgeZ + row * chunks * kLow;
        // the product to the right of the last chunk is the identity (all coefficients zero)
        if (!copier) {
            for (int idx = threadIdx.x; idx < kLow; idx += G::kBlock) sOut[last & 1][idx] = T(0);
            if constexpr (!RESIDENT) {
                stager.fetch(rows + (int64_t)last * kLow);
                stager.commit(sB[last & 1]);
                stager.fetch(rows + (int64_t)(last - 1 > 0 ? last - 1 : 0) * kLow);
            }
        }
        lds_barrier();
        for (int c = last; c >= 1; --c) {
            if (!copier) {
                // Z_{c-1} = S_c (x) Z_c
                load_state<T, D, P, N - 1, kAS>(chunk_ptr(c), pu, active, a, asub);
                apply_right<T, D, P, N - 1, kAS>(a, asub, sOut[c & 1], sw);
                if (active) store_state<T, D, P, N - 1, kAS>(sOut[(c - 1) & 1], pu, a, asub);
                if constexpr (!RESIDENT) {
                    stager.commit(sB[(c - 1) & 1]);
                    stager.fetch(rows + (int64_t)(c - 2 > 0 ? c - 2 : 0) * kLow);
                }
            } else {
                copy_row_out<T, kLow>(sOut[c & 1], edge + (int64_t)c * kLow, ctid);
            }
            lds_barrier();
        }
        if (copier) copy_row_out<T, kLow>(sOut[0], edge, ctid);
    }
}

// The scan and the product of the partial signatures of the forward sweep in one launch: three chains of dependent
// products per row, in blocks that are small enough for two of them to share a CU, so that they run side by side
// (as launches of their own, the 128 to 256 blocks of each leave most of the device idle, one after the other).
//   blockIdx.y == 0:  edgeA_c = S_0 (x) .. (x) S_c
//   blockIdx.y == 1:  edgeZ_c = S_{c+1} (x) .. (x) S_{C-1}
//   blockIdx.y >= 2:  the signature of the row from its `groups` partial products (combine_staged), the lanes of
//                     the row dealt to one or more blocks
// The scans work like dense_scan_kernel with all rows in LDS, except that only `resident` chunk rows have a place
// there: the up to kEdgeExtra rows that a scan uses last are fetched into registers at the start and take the
// places of the rows used first once those have been read.  (A deeper pipeline of fetches through registers is not
// an option: after the first branch the compiler waits for every outstanding load before it uses any.)
constexpr int kEdgeExtra = 3;

template <typename T, int D, int N, int PS, int PC>
struct EdgesShape {
    using GS = Geometry<D, N, PS>;
    using GC = Geometry<D, N, PC>;
    static constexpr int kLow = (int)GS::kLowSize;
    static constexpr int kScanThreads = GS::kBlock + kCopyThreads;
    // the combine's lanes in blocks of at most 512 threads (two such blocks share a CU whatever their registers)
    static constexpr int kCombineBlock = GC::kBlock <= 512 ? GC::kBlock : 512;
    static constexpr int kCombineParts = GC::kBlock / kCombineBlock;
    static constexpr int kThreads = kCombineBlock > kScanThreads ? kCombineBlock : kScanThreads;
    static constexpr size_t kRowBytes = (size_t)kLow * sizeof(T);
    static constexpr size_t kStaticBytes = 2 * kRowBytes;  // the double buffer of the scans
    static constexpr size_t kCombineBytes = CombineShape<T, D, N, PC, kCombineBlock>::kBytes;  // staging of the combine
    static constexpr size_t kBudget = 78 * 1024;           // two blocks to a CU
    // (compiled for fp32 from depth 4 on: the launch it saves matters where a step takes a hundred microseconds,
    // and every instantiation adds to the library)
    static constexpr bool kUsable = sizeof(T) == 4 && N >= 4 && kThreads <= 512 && GC::kBlock % kCombineBlock == 0 &&
                                    !GS::kOnePiece && kRowBytes % 16 == 0 && kStaticBytes + kCombineBytes <= kBudget;
};

template <typename T, int D, int N, int P, bool ascending>
__device__ __forceinline__ void scan_resident(const T *__restrict__ chunk_low, T *__restrict__ edges, int chunks,
                                              int resident, int64_t row, T *sAll, T *sOut0, T *sOut1) {
    using G = Geometry<D, N, P>;
    using Stager = RowStager<T, (int)G::kLowSize, G::kBlock>;
    constexpr int kAS = G::kASub > 0 ? G::kASub : 1;
    constexpr int kLow = (int)G::kLowSize;
    constexpr int kThreads = G::kBlock + kCopyThreads;
    const bool copier = (int)threadIdx.x >= G::kBlock;
    const int ctid = (int)threadIdx.x - G::kBlock;
    const int pu = copier ? 0 : (int)threadIdx.x;
    const bool active = !copier && ((G::kLanes == G::kBlock) || pu < G::kLanes);
    int u[P];
    prefix_letters<D, P>(active ? pu : 0, u);
    const SubWords<D, P> sw(u);
    const T *rows = chunk_low + row * chunks * kLow;
    T *edge = edges + row * chunks * kLow;
    const int last = chunks - 1;
    // rows in the order of their use: edgeA multiplies the chunks 1, 2, .. onto chunk 0, edgeZ takes the chunks
    // last, last - 1, .., 1 as the left factor of its running product
    const int used = last;
    auto chunk_of = [&](int j) { return ascending ? 1 + j : last - j; };
    const int held = resident < used ? resident : used;
    Stager extra[kEdgeExtra];
    if (!copier) {
        static_for<0, kEdgeExtra>([&](auto ec) {
            constexpr int e = decltype(ec)::value;
            const int j = held + e < used ? held + e : used - 1;
            extra[e].fetch(rows + (int64_t)chunk_of(j) * kLow);
        });
    }
    // (unrolled so that the loads of several rows are in flight together: one memory latency for the burst)
#pragma unroll 8
    for (int j = 0; j < held; ++j)
        copy_row<T, kLow, kThreads>(rows + (int64_t)chunk_of(j) * kLow, sAll + (int64_t)j * kLow, (int)threadIdx.x);
    T a[P + 1];
    T asub[kAS];
    if (!copier) {
        if (ascending) {
            load_state<T, D, P, N - 1, kAS>(rows, pu, active, a, asub);
            if (active) store_state<T, D, P, N - 1, kAS>(sOut0, pu, a, asub);
        } else {
            // the product to the right of the last chunk is the identity (all coefficients zero)
            for (int idx = threadIdx.x; idx < kLow; idx += G::kBlock) ((last & 1) ? sOut1 : sOut0)[idx] = T(0);
        }
    }
    lds_barrier();
    for (int j = 0; j < used; ++j) {
        const int c = chunk_of(j);
        const T *slot = sAll + (int64_t)(j < held ? j : j - held) * kLow;
        if (!copier) {
            // the row of the round before has been read by everyone: its place takes the row that comes `held` later
            static_for<0, kEdgeExtra>([&](auto ec) {
                constexpr int e = decltype(ec)::value;
                if (j == e + 1 && held + e < used) extra[e].commit_exact(sAll + (int64_t)e * kLow);
            });
            if (ascending) {
                apply_right<T, D, P, N - 1, kAS>(a, asub, slot, sw);
                if (active) store_state<T, D, P, N - 1, kAS>((c & 1) ? sOut1 : sOut0, pu, a, asub);
            } else {
                // Z_{c-1} = S_c (x) Z_c
                load_state<T, D, P, N - 1, kAS>(slot, pu, active, a, asub);
                apply_right<T, D, P, N - 1, kAS>(a, asub, (c & 1) ? sOut1 : sOut0, sw);
                if (active) store_state<T, D, P, N - 1, kAS>(((c - 1) & 1) ? sOut1 : sOut0, pu, a, asub);
            }
        } else {
            if (ascending) copy_row_out<T, kLow>(((c - 1) & 1) ? sOut1 : sOut0, edge + (int64_t)(c - 1) * kLow, ctid);
            else copy_row_out<T, kLow>((c & 1) ? sOut1 : sOut0, edge + (int64_t)c * kLow, ctid);
        }
        lds_barrier();
    }
    if (copier) {
        if (ascending) copy_row_out<T, kLow>((last & 1) ? sOut1 : sOut0, edge + (int64_t)last * kLow, ctid);
        else copy_row_out<T, kLow>(sOut0, edge, ctid);
    }
}

template <typename T, int D, int N, int PS, int PC>
__global__ void __launch_bounds__((EdgesShape<T, D, N, PS, PC>::kThreads))
    dense_edges_kernel(const T *__restrict__ chunk_low, T *__restrict__ edgeA, T *__restrict__ edgeZ, int chunks,
                       int resident, const T *__restrict__ partial, T *__restrict__ sig, int groups) {
    using ES = EdgesShape<T, D, N, PS, PC>;
    extern __shared__ __align__(16) unsigned char edges_smem[];
    __shared__ __align__(16) T sOut[2][ES::kLow];
    T *dyn = reinterpret_cast<T *>(edges_smem);
    const int64_t row = blockIdx.x;
    if (blockIdx.y >= 2) {
        if ((int)threadIdx.x >= ES::kCombineBlock) return;
        combine_staged<T, D, N, PC, ES::kCombineBlock>(partial, sig, groups, row, dyn,
                                                       dyn + CombineShape<T, D, N, PC, ES::kCombineBlock>::kStage,
                                                       ((int)blockIdx.y - 2) * ES::kCombineBlock);
        return;
    }
    if ((int)threadIdx.x >= ES::kScanThreads) return;
    if (blockIdx.y == 0) scan_resident<T, D, N, PS, true>(chunk_low, edgeA, chunks, resident, row, dyn, sOut[0], sOut[1]);
    else scan_resident<T, D, N, PS, false>(chunk_low, edgeZ, chunks, resident, row, dyn, sOut[0], sOut[1]);
}

// Grouped hand-over: the products of whole groups of four chunks.  `partial` holds the `groups` group products of
// every row (dense-layout rows, the forward sweep's block results).
//   blockIdx.y == 0:  edgeR_g = Q_{g+1} (x) .. (x) Q_{groups-1} below the top level, g = 0 .. groups - 2
//   blockIdx.y >= 1:  the signature of the row (combine_staged), which on its way leaves
//                     edgeL_g = Q_0 (x) .. (x) Q_{g-1} below the top level, g = 1 .. groups - 1
// (both arrays [rows, groups, levels below N]; the entries not named are never read)
template <typename T, int D, int N, int PS, int PC>
__global__ void __launch_bounds__((EdgesShape<T, D, N, PS, PC>::kThreads))
    dense_group_edges_kernel(const T *__restrict__ partial, T *__restrict__ edgeL, T *__restrict__ edgeR,
                             T *__restrict__ sig, int groups) {
    using ES = EdgesShape<T, D, N, PS, PC>;
    using G = Geometry<D, N, PS>;
    extern __shared__ __align__(16) unsigned char group_smem[];
    __shared__ __align__(16) T sOut[2][ES::kLow];
    T *dyn = reinterpret_cast<T *>(group_smem);
    const int64_t row = blockIdx.x;
    if (blockIdx.y >= 1) {
        if ((int)threadIdx.x >= ES::kCombineBlock) return;
        combine_staged<T, D, N, PC, ES::kCombineBlock>(partial, sig, groups, row, dyn,
                                                       dyn + CombineShape<T, D, N, PC, ES::kCombineBlock>::kStage,
                                                       ((int)blockIdx.y - 1) * ES::kCombineBlock, edgeL);
        return;
    }
    if ((int)threadIdx.x >= G::kBlock) return;
    constexpr int kAS = G::kASub > 0 ? G::kASub : 1;
    constexpr int kLow = ES::kLow;
    const int pu = (int)threadIdx.x;
    const bool active = (G::kLanes == G::kBlock) || pu < G::kLanes;
    int u[PS];
    prefix_letters<D, PS>(active ? pu : 0, u);
    const SubWords<D, PS> sw(u);
    const T *rows = partial + row * groups * G::kSigSize;
    T *edge = edgeR + row * groups * kLow;
    T a[PS + 1];
    T asub[kAS];
    // R_{groups-2} = Q_{groups-1}; R_{g-1} = Q_g (x) R_g
    load_state<T, D, PS, N - 1, kAS>(rows + (int64_t)(groups - 1) * G::kSigSize, pu, active, a, asub);
    if (active) {
        store_state<T, D, PS, N - 1, kAS>(sOut[(groups - 2) & 1], pu, a, asub);
        store_state<T, D, PS, N - 1, kAS>(edge + (int64_t)(groups - 2) * kLow, pu, a, asub);
    }
    for (int g = groups - 2; g >= 1; --g) {
        load_state<T, D, PS, N - 1, kAS>(rows + (int64_t)g * G::kSigSize, pu, active, a, asub);
        lds_barrier();
        apply_right<T, D, PS, N - 1, kAS>(a, asub, sOut[g & 1], sw);
        if (active) {
            store_state<T, D, PS, N - 1, kAS>(sOut[(g - 1) & 1], pu, a, asub);
            store_state<T, D, PS, N - 1, kAS>(edge + (int64_t)(g - 1) * kLow, pu, a, asub);
        }
    }
}

// Depth 2: the signature of a chunk below the top level is its level 1, the sum of its increments.  One block
// per (row, chunk); zero_rows as in dense_forward_kernel (the block also clears the points of its chunk in a
// [B, L, d] buffer, the last chunk of a row the final point too).
template <typename T>
__global__ void __launch_bounds__(kWave) chunk_level1_kernel(const T *__restrict__ path, T *__restrict__ chunk_low,
                                                             SigShape shape, int chunks, T *__restrict__ zero_rows) {
    const int64_t unit = blockIdx.x;
    int64_t row, chunk_of_row, b, w;
    divide_index(unit, chunks, row, chunk_of_row);
    const int c = (int)chunk_of_row;
    divide_index(row, shape.W, b, w);
    const Span span = unit_span(shape, w);
    int64_t begin, end;
    chunk_range(span.steps, chunks, c, begin, end);
    const int64_t d = shape.d;
    const T *x = path + (b * shape.L + span.start) * d;
    for (int64_t a = threadIdx.x; a < d; a += kWave)
        chunk_low[unit * d + a] = end > begin ? x[end * d + a] - x[begin * d + a] : T(0);
    if (zero_rows) {
        const int64_t points = end - begin + (c == chunks - 1 ? 1 : 0);
        T *z = zero_rows + (b * shape.L + span.start + begin) * d;
        for (int64_t idx = threadIdx.x; idx < points * d; idx += kWave) z[idx] = T(0);
    }
}

// LDS layout of the reverse sweep.  Per-increment sums leave a wave as four row sums (eight partial sums where the
// slab below is used); the tile flush adds the parts of all waves in a fixed order.  The tile is shortened until
// the parts fit 48 KB of LDS (128 KB for the widest alphabets, whose parts of sixteen increments would not fit a
// CU at all).
//
// The slab.  Summing a lane's D per-increment terms over the lanes with DPP moves costs more than its dozen
// instructions: a wave with DPP instructions (or lane reads, or lane permutes) in its stream is not overlapped
// with the other wave of its SIMD any more.  Measured on MI355X with two resident waves per SIMD: 0.94 ns per
// vector instruction for a long run of multiply-adds, 1.7 to 1.8 ns as soon as one instruction in sixty-four
// is a DPP move, which is what one wave alone gets; LDS reads, writes and swizzles cost about three instruction
// slots each and leave the overlap alone.  The loop of the depth-6 sweep over four letters: 1.39 ns per vector
// instruction as compiled, 1.11 ns with its twelve DPP instructions replaced by plain ones.  So fp32 units of up
// to four waves over at most fifteen letters take another way: every lane stores its D terms of an increment,
// padded to kDP, into a slab of its wave (one or more 16-byte LDS stores), and once kSubTile increments have
// gathered there the lanes read the slab back across the lanes, eight 16-byte reads each, and leave eight
// partial sums per increment and letter in `sg`.
template <typename T, int D, int N, int P, int MAXW = 0>
struct BackwardShape {
    using G = Geometry<D, N, P, sizeof(T), MAXW>;
    static constexpr int KS = N - P;
    static constexpr int kDP = D <= 4 ? 4 : D <= 8 ? 8 : 16;  // letters padded to whole 16-byte pieces
    // (blocks of eight waves, their 64 KB of slabs in dynamic LDS and sums tiled by sixteen increments, measured
    // slower than the DPP form: the depth-5 sweep over eight letters 359 us against 336 us)
    static constexpr bool kSlab = sizeof(T) == 4 && D <= 15 && !G::kSplit && G::kWaves <= 4;
    static constexpr int kGroups = kDP / 4;        // 16-byte pieces per lane and increment
    static constexpr int kSubTile = 32 / kDP;      // increments that wait in the slab: 8, 4 or 2 (8 KB per wave)
    static constexpr int kSlabElems = kSlab ? G::kWaves * kSubTile * kWave * kDP : 4;
    static constexpr int kParts = kSlab ? 8 : 4;
    static constexpr int kLetters = kSlab ? kDP : D;  // cells of one increment in a row of `sg`
    // LDS bytes of the parts of one increment
    static constexpr int kRowBytes = G::kWaves * kParts * kLetters * (int)sizeof(T);
    // (letter blocks: eight one-wave blocks and their 8 KB slabs share a CU, so the sums of a tile take 4 KB)
    static constexpr int kTileBytes = G::kLetterBlocks ? 4096 : 8192;
    static constexpr int kBwdTile =
        kSlab ? (kRowBytes * 32 <= kTileBytes ? 32 : kRowBytes * 16 <= kTileBytes ? 16 : 8)
              : (kRowBytes * 64 <= 49152 ? 64 : kRowBytes * 32 <= 49152 ? 32
                 : kRowBytes * 16 <= 131072 ? 16 : kRowBytes * 8 <= 131072 ? 8 : 4);
    // Increments are staged for several tiles at a time where that takes little LDS (at most 4 KB, plus the
    // increment of the ghost step; eight one-wave blocks with their slabs still share a CU): a round trip to
    // memory per stage instead of one per tile.
    static constexpr int kTileStage = kBwdTile * KS * D;
    static constexpr int kStageRoom = 4096 / (kTileStage * (int)sizeof(T));
    static constexpr int kStageTiles = !kSlab || kStageRoom < 1 ? 1 : kStageRoom > 8 ? 8 : kStageRoom;
    static constexpr int kStage = kStageTiles * kTileStage + (kStageTiles > 1 ? KS * D : 0);
    static constexpr int kSums = G::kWaves * kParts;
    static constexpr int kSumRow = kBwdTile * kLetters;
    // fp64: the chain's P terms reach their letters through LDS (a row of D cells per lane, letter-major so that
    // a wave's accesses never share a bank).  A lane's prefix never changes, so it only ever touches the same
    // P cells and the others stay zero: P LDS adds, D loads and P clearing stores replace 3 * P * D selects and
    // adds of a kernel that is bound by vector instruction issue.  fp32 multiplies by one-hot constants instead
    // where those fit the register file.
    static constexpr bool kChainCells = sizeof(T) == 8 && D <= 8 && D * G::kBlock * (int)sizeof(T) <= 32 * 1024;
    static constexpr int kCells = kChainCells ? D * G::kBlock : 1;
};

// BOUND: the upstream gradient is zero on every top-level word that has a letter below BOUND after the
// prefix's first letter, and the sweep leaves those words out; the LDS arrays belong to the calling kernel.
template <typename T, int D, int N, int P, bool ACCUMULATE, bool CHUNKED, int BOUND, int MAXW = 0>
__device__ __forceinline__ void dense_backward_body(
    const T *__restrict__ path, const T *__restrict__ sig, const T *__restrict__ grad_sig, const T *__restrict__ edgeA,
    const T *__restrict__ edgeZ, T *__restrict__ grad_inc, const SigShape &shape, int chunks, T *__restrict__ grad_path,
    const int pu_unit,  // index of the thread within its unit (its prefix, unless the first level is split)
    const int tid,      // index of the thread within its block
    T (&sdx_all)[BackwardShape<T, D, N, P, MAXW>::kStage],
    T (&sg)[BackwardShape<T, D, N, P, MAXW>::kSums][BackwardShape<T, D, N, P, MAXW>::kSumRow],
    T (&cells)[BackwardShape<T, D, N, P, MAXW>::kCells], T (&slab)[BackwardShape<T, D, N, P, MAXW>::kSlabElems], T (&carry)[D],
    const T *__restrict__ edgeL = nullptr, const T *__restrict__ edgeR = nullptr) {
    using G = Geometry<D, N, P, sizeof(T), MAXW>;
    using BS = BackwardShape<T, D, N, P, MAXW>;
    constexpr int KS = N - P;
    constexpr int kParts = BS::kParts;
    constexpr int kBwdTile = BS::kBwdTile;
    constexpr bool kToPath = CHUNKED && !ACCUMULATE;  // writes the path gradient itself (see the tile flush)
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;  // within the block
    // first level split between lanes: pu_unit counts (part of the children, prefix); pu is the prefix
    constexpr int KF = G::kK, FQ = G::kSplit ? KS : 1, FK = G::kSplit ? KF : 1;
    const int spart = G::kSplit ? pu_unit / G::kPartLanes : 0;
    const int pu = G::kSplit ? pu_unit - spart * G::kPartLanes : pu_unit;
    const int a0 = spart * KF;
    const bool active = G::kSplit ? (pu < G::kPrefixes && spart < G::kParts)
                                  : ((G::kLanes == G::kBlock) || pu < G::kLanes);
    int u[P];
    prefix_letters<D, P>(active ? pu : 0, u);
    // chain terms through LDS (see BackwardShape): the lane's cells start at zero
    constexpr bool kCellChain = BS::kChainCells && !(sizeof(T) == 4 && P * D <= 24);
    T *my_cells = cells + (BS::kChainCells ? tid : 0);  // cell of letter k: my_cells[k * G::kBlock]
    if constexpr (kCellChain) {
#pragma unroll
        for (int k = 0; k < D; ++k) my_cells[k * G::kBlock] = T(0);
    }

    int64_t unit = unit_of_block<G>();
    if constexpr (CHUNKED && G::kUnitBlocks == 1) {
        // Consecutive blocks go to the eight XCDs in turn, each with an L2 of its own.  The chunks of a row read the
        // same upstream gradient, so they are dealt to one XCD: block b = 8 q + x works on the q-th unit of the
        // rows x, x + 8, x + 16, ... (as long as whole groups of eight rows remain).
        // (grid dimensions are below 2^31: 32-bit arithmetic)
        const unsigned total = gridDim.x, per_group = 8u * (unsigned)chunks, at = (unsigned)unit;
        if (at < total / per_group * per_group) {
            const unsigned group = at / per_group, in_group = at - group * per_group;
            const unsigned x = in_group & 7u, q = in_group >> 3;
            unit = ((int64_t)group * 8 + x) * chunks + q;
        }
    }
    int64_t row, chunk_of_row, b, w;
    divide_index(unit, chunks, row, chunk_of_row);
    const int c = (int)chunk_of_row;
    divide_index(row, shape.W, b, w);
    const Span span = unit_span(shape, w);
    int64_t begin, end;
    chunk_range(span.steps, chunks, c, begin, end);
    const T *x = path + (b * shape.L + span.start) * D;
    T *ginc = grad_inc + (b * (shape.L - 1) + span.start) * D;
    const T *grow = grad_sig + row * G::kSigSize;

    // A chunk that writes the path gradient itself (kToPath) owns the points begin .. end - 1 of its row (the last
    // chunk also the final point): dL/dx[t] = g[t-1] - g[t] with g the per-increment sums.  The sum of the last
    // increment before the chunk, g[begin - 1], belongs to the chunk on the left; this chunk computes it again with
    // one more step of its sweep (tile -1, the ghost step: the state after increment `begin` is exactly what that
    // step needs), so every point has one writer, nothing is added in memory and the order of the sums is fixed.
    const int64_t len = end - begin;
    const int64_t ntiles = (len + kBwdTile - 1) / kBwdTile;
    const bool ghost = kToPath && len > 0 && begin > 0;
    // Increments reach LDS a stage at a time: the tiles ti - ti % kStageTiles .. ti share one (the leftmost stage
    // also holds the ghost step).  The first stage is requested last of the prologue's loads (below).
    constexpr int kStageTiles = BS::kStageTiles;
    int64_t staged_from = 0;  // first increment in `sdx_all`
    auto stage_for = [&](int64_t ti) {
        if (ti < 0) {
            if (kStageTiles > 1) return;  // part of the leftmost stage
            staged_from = begin - 1;
            stage_increments<T, D, KS, G::kBlock>(sdx_all, x + staged_from * D, 1, tid);
        } else if (ti == ntiles - 1 || (ti + 1) % kStageTiles == 0) {
            const int64_t first_tile = ti - ti % kStageTiles;
            const int64_t until = end < begin + (ti + 1) * kBwdTile ? end : begin + (ti + 1) * kBwdTile;
            staged_from = begin + first_tile * kBwdTile - (kStageTiles > 1 && first_tile == 0 && ghost ? 1 : 0);
            stage_increments<T, D, KS, G::kBlock>(sdx_all, x + staged_from * D, (int)(until - staged_from), tid);
        }
    };
    // A: signature at the right edge of the unit (levels < N).  H: adjoint at the right edge.
    // Everything the prologue reads from memory is requested before the first wait: the upstream gradient, the two
    // rows of chunk products, and last the path points of the first stage, whose wait is then the only one.
    constexpr int kAS = G::kASub > 0 ? G::kASub : 1;
    T a[P + 1], hc[P + 1];
    T asub[kAS];
    T hsub[G::kFwdSub];
    load_state<T, D, P, N, G::kFwdSub, G::kK>(grow, pu, active, hc, hsub, a0);
    if constexpr (CHUNKED) {
        auto load_edge_state = [&](const T *edge_row) { load_state<T, D, P, N - 1, kAS>(edge_row, pu, active, a, asub); };
        // adjoint at the right edge of the chunk: the upstream gradient contracted with the signature of
        // everything to the right of the chunk
        const SubWords<D, P> sw(u);
        // The lanes read the row of suffix products at addresses of their own, each entry several times over
        // the block: where the slab has room for it the row goes there first, in one coalesced copy
        // (in the skewed layout of rows in LDS, see RowPlace).
        constexpr bool kStageEdge = BS::kSlab && RowPlace<D, true>::size((int)G::kLowSize) <= BS::kSlabElems;
        if constexpr (kStageEdge && N >= 4 && N - 1 >= P && sizeof(T) == 4) {
            if (edgeL != nullptr) {
                // Grouped hand-over: edgeA / edgeZ hold the products of the chunk with the chunks to its left / to
                // its right inside its group of four, edgeL / edgeR those of the groups to the left / right of the
                // group (all below the top level).  A = L (x) A_in;  H = G contracted with Z_in (x) R.
                const int grp = c >> 2, in_grp = c & 3, groups = chunks >> 2;
                const bool have_right = grp < groups - 1, have_rest = in_grp < 3, have_left = grp > 0;
                const int64_t group_row = (row * groups + grp) * G::kLowSize;
                using Stager = RowStager<T, (int)G::kLowSize, G::kBlock>;
                // (rows that are not needed are read all the same, from places that exist: loads under a
                // condition would make the compiler wait for everything at their first use)
                Stager right_row, own_row;
                T z[P + 1], zsub[kAS];  // the product to the right inside the group, as a lane state
                right_row.fetch(edgeR + (have_right ? group_row : (int64_t)0));
                load_state<T, D, P, N - 1, kAS>(edgeZ + unit * G::kLowSize, pu, active, z, zsub);
                own_row.fetch(edgeA + unit * G::kLowSize);
                load_edge_state(have_left ? edgeL + group_row : edgeA + unit * G::kLowSize);
                if (ntiles > 0) stage_for(ntiles - 1);
                adjoint_chain_of_lane<T, D, P>(pu, a0, hc);
                // suffix of the rest of the row, Z = Z_in (x) R: a product below the top level on the lanes' states
                // (a second contraction of the full adjoint would cost three times as much), handed to the
                // contraction through the slab
                if (have_right) {
                    right_row.template commit_skewed<D>(&slab[0]);
                    lds_barrier();
                    if (have_rest) {
                        apply_right<T, D, P, N - 1, kAS, true>(z, zsub, &slab[0], sw);
                        lds_barrier();
                    }
                }
                if (have_rest) {
                    if (active) store_state<T, D, P, N - 1, kAS, D, true>(&slab[0], pu, z, zsub);
                    lds_barrier();
                }
                if (have_right || have_rest) {
                    contract_right<T, D, N, P, G::kFwdSub, true>(hc, hsub, &slab[0], sw);
                    lds_barrier();
                }
                if (have_left) {
                    own_row.template commit_skewed<D>(&slab[0]);
                    lds_barrier();
                    apply_right<T, D, P, N - 1, kAS, true>(a, asub, &slab[0], sw);
                }
            } else {
                load_edge_state(edgeA + unit * G::kLowSize);
                RowStager<T, (int)G::kLowSize, G::kBlock> suffix_row;
                suffix_row.fetch(edgeZ + unit * G::kLowSize);
                if (ntiles > 0) stage_for(ntiles - 1);
                suffix_row.template commit_skewed<D>(&slab[0]);
                adjoint_chain_of_lane<T, D, P>(pu, a0, hc);
                lds_barrier();
                contract_right<T, D, N, P, G::kFwdSub, true>(hc, hsub, &slab[0], sw);
            }
        } else if constexpr (kStageEdge) {
            load_edge_state(edgeA + unit * G::kLowSize);
            RowStager<T, (int)G::kLowSize, G::kBlock> suffix_row;
            suffix_row.fetch(edgeZ + unit * G::kLowSize);
            if (ntiles > 0) stage_for(ntiles - 1);
            suffix_row.template commit_skewed<D>(&slab[0]);
            adjoint_chain_of_lane<T, D, P>(pu, a0, hc);
            lds_barrier();
            contract_right<T, D, N, P, G::kFwdSub, true>(hc, hsub, &slab[0], sw);
        } else {
            load_edge_state(edgeA + unit * G::kLowSize);
            if (ntiles > 0) stage_for(ntiles - 1);
            adjoint_chain_of_lane<T, D, P>(pu, a0, hc);
            contract_right<T, D, N, P, G::kFwdSub>(hc, hsub, edgeZ + unit * G::kLowSize, sw);
        }
    } else {
        load_state<T, D, P, N - 1, kAS, KF>(sig + row * G::kSigSize, pu, active, a, asub, a0);
        if (ntiles > 0) stage_for(ntiles - 1);
        adjoint_chain_of_lane<T, D, P>(pu, a0, hc);
    }
    a[0] = T(1);
    // onehot[j][k] = 1 when the j-th letter of the lane's prefix is k (kept in registers only where
    // registers are plentiful; otherwise the letters are compared every time)
    constexpr bool kOneHot = sizeof(T) == 4 && P * D <= 24;
    T onehot[kOneHot ? P : 1][kOneHot ? D : 1];
    // Wide alphabets compare every letter with the prefix letters to route the chain's terms (P * D selects and
    // adds per increment).  The last prefix letter is different in every lane of a row of sixteen, so its term
    // is added to the row's cell of that letter in LDS instead, after the pass that writes the cells.
    constexpr bool kLastDirect = !kOneHot && !BS::kChainCells && D >= 16 && kParts == 4;
    // The earlier prefix letters take at most two values within such a row (sixteen consecutive prefixes cross at
    // most one multiple of D, D^2, ..): the letter of the row's first lane and that of its last.  Their terms are
    // summed over the row in those two groups and added to the two cells by the row's first lane.
    constexpr int kRowLetters = kLastDirect ? P - 1 : 0;
    int ua[kRowLetters > 0 ? kRowLetters : 1], ub[kRowLetters > 0 ? kRowLetters : 1];
    bool with_first[kRowLetters > 0 ? kRowLetters : 1];
    bool row_live = false;
    if constexpr (kRowLetters > 0) {
        const int first = pu - (lane & 15);
        row_live = first < G::kPrefixes;
        const int last = first + 15 < G::kPrefixes ? first + 15 : G::kPrefixes - 1;
        int uf[P], ul[P];
        prefix_letters<D, P>(row_live ? first : 0, uf);
        prefix_letters<D, P>(row_live ? last : 0, ul);
#pragma unroll
        for (int j = 0; j < kRowLetters; ++j) {
            ua[j] = uf[j];
            ub[j] = ul[j];
            with_first[j] = u[j] == uf[j];
        }
    }
    if constexpr (kOneHot) {
#pragma unroll
        for (int j = 0; j < P; ++j)
#pragma unroll
            for (int k = 0; k < D; ++k) onehot[j][k] = (u[j] == k) ? T(1) : T(0);
    }


    for (int64_t ti = ntiles - 1; ti >= (ghost ? -1 : 0); --ti) {
        const int64_t t0 = ti < 0 ? begin - 1 : begin + ti * kBwdTile;
        const int nt = ti < 0 ? 1 : (int)((end - t0) < kBwdTile ? (end - t0) : kBwdTile);
        lds_barrier();
        if (ti < ntiles - 1) stage_for(ti);
        const T *sdx = sdx_all + (t0 - staged_from) * (KS * D);
        lds_barrier();
        auto step = [&](int tt, const T (&dxs)[KS][D], const T (&dxp)[P], const T (&dxf)[FQ][FK]) {
            // A_t = A_{t+1} (x) exp(-dx_t), levels < N
            if constexpr (N > 1) {
                if constexpr (G::kSplit)
                    StepTargets<T, D, P, N - 1, true, 0, KF>::template run<kAS, KS>(a, asub, dxs, dxf, dxp);
                else
                    StepTargets<T, D, P, N - 1, true>::template run<kAS, KS>(a, asub, dxs, dxs, dxp);
            }
            T gdxk[KS][D], gpre[P];
            T gdxf[FQ][FK];
#pragma unroll
            for (int q = 0; q < FQ; ++q)
#pragma unroll
                for (int i = 0; i < FK; ++i) gdxf[q][i] = T(0);
#pragma unroll
            for (int q = 0; q < KS; ++q)
#pragma unroll
                for (int k = 0; k < D; ++k) gdxk[q][k] = T(0);
#pragma unroll
            for (int j = 0; j < P; ++j) gpre[j] = T(0);
            if constexpr (G::kSplit)
                AdjTargets<T, D, N, P, 1, BOUND, KF>::template run<kAS, G::kFwdSub, KS>(a, asub, hc, hsub, dxs, dxf, dxp,
                                                                                        gdxk, gdxf, gpre);
            else
                AdjTargets<T, D, N, P, 1, BOUND>::template run<kAS, G::kFwdSub, KS>(a, asub, hc, hsub, dxs, dxs, dxp,
                                                                                    gdxk, gdxk, gpre);
            // letter k collects the sub-trie sums (with the 1/(q+1) of their increments) and the chain
            // positions whose letter is k
            T tot[D];
#pragma unroll
            for (int k = 0; k < D; ++k) {
                T v = gdxk[0][k];
#pragma unroll
                for (int q = 1; q < KS; ++q) v = fmad<T>(gdxk[q][k], rcp<T>(q + 1), v);
#pragma unroll
                for (int j = 0; j < (kLastDirect ? 0 : P); ++j) {
                    if constexpr (kOneHot) v = fmad<T>(onehot[j][k], gpre[j], v);
                    else if constexpr (!BS::kChainCells) v += (u[j] == k) ? gpre[j] : T(0);
                }
                tot[k] = v;
            }
            if constexpr (BS::kChainCells && !kOneHot) {
                // LDS adds, because two positions of the prefix may carry the same letter; no other lane touches
                // these cells, and the ones just used are cleared again for the next increment
#pragma unroll
                for (int j = 0; j < P; ++j) atomicAdd(&my_cells[u[j] * G::kBlock], gpre[j]);
#pragma unroll
                for (int k = 0; k < D; ++k) tot[k] += my_cells[k * G::kBlock];
#pragma unroll
                for (int j = 0; j < P; ++j) my_cells[u[j] * G::kBlock] = T(0);
            }
            if constexpr (BS::kSlab) {
                // the lane's terms of this increment go to its row of the wave's slab; the increment that completes
                // a group of kSubTile sums the group over the lanes
                using V4 = typename VecOf<T, 4>::type;
                constexpr int kSub = BS::kSubTile, kGroups = BS::kGroups;
                V4 *mine = reinterpret_cast<V4 *>(slab) +
                           (size_t)(((wave * kSub + (tt & (kSub - 1))) * kWave + lane) * kGroups);
#pragma unroll
                for (int g = 0; g < kGroups; ++g) {
                    V4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = 4 * g + e < D ? tot[4 * g + e < D ? 4 * g + e : 0] : T(0);
                    mine[g] = v;
                }
                if ((tt & (kSub - 1)) == 0) {
                    // (the LDS operations of a wave complete in order; the fence keeps the compiler from moving
                    // the reads of other lanes' rows above the stores)
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    // lane -> (increment of the group, one eighth of the lanes, 16-byte piece of the letters)
                    constexpr int kPer = kWave / kSub;  // lanes that share an increment: 8 * kGroups
                    const int ttl = lane / kPer, part = (lane % kPer) / kGroups, piece = lane % kGroups;
                    const V4 *rows = reinterpret_cast<const V4 *>(slab) +
                                     (size_t)((wave * kSub + ttl) * kWave) * kGroups + piece;
                    // source lanes 8 s + (part + s) % 8: the eight lanes that read together hit different banks
                    V4 acc = rows[(size_t)(part & 7) * kGroups];
#pragma unroll
                    for (int s8 = 1; s8 < 8; ++s8) acc += rows[(size_t)(8 * s8 + ((part + s8) & 7)) * kGroups];
                    if (tt + ttl < nt)  // (rows beyond the last increment of the tile hold nothing of this tile)
                        reinterpret_cast<V4 *>(&sg[wave * 8 + part][0])[(tt + ttl) * kGroups + piece] = acc;
                }
            } else if constexpr (kParts == 4) {
                // up to sixteen letters in one pass of exchanges (padded to a power of two with zeros), wider
                // alphabets sixteen letters at a time; one store per row of 16 lanes and pass
                constexpr int DP = D <= 2 ? 2 : D <= 4 ? 4 : D <= 8 ? 8 : 16;
#pragma unroll
                for (int base = 0; base < D; base += DP) {
                    T padded[DP];
#pragma unroll
                    for (int k = 0; k < DP; ++k) padded[k] = base + k < D ? tot[base + k] : T(0);
                    const T r = row_totals<T, DP>(padded, lane);
                    const int letter = base + row_letter<DP>(lane);
                    if (row_writer<DP>(lane) && letter < D) sg[wave * 4 + (lane >> 4)][tt * D + letter] = r;
                }
                // The passes below add to cells that other lanes of the same wave have just stored.  A wave's LDS
                // operations complete in order; the fences keep the compiler from moving or merging them across
                // the passes (no instruction is emitted for them).
                auto order_wave_lds = [] {
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                };
                // (the cells of a row of sixteen lanes belong to one wave, sg[wave * 4 + row]: a bounded sweep, which
                // runs a copy of this body per wave, still has writer and adder in the same copy)
                if constexpr (kLastDirect) {
                    order_wave_lds();
                    // the term of the last prefix letter goes straight to its cell: the sixteen lanes of a row hold
                    // consecutive prefixes, so with sixteen letters or more their last letters differ
                    if (active) sg[wave * 4 + (lane >> 4)][tt * D + u[P - 1]] += gpre[P - 1];
#pragma unroll
                    for (int j = 0; j < kRowLetters; ++j) {
                        const T mine = with_first[j] ? gpre[j] : T(0);
                        const T sum_first = row_total(mine);
                        const T sum_last = row_total(gpre[j] - mine);
                        order_wave_lds();
                        if ((lane & 15) == 0 && row_live) {
                            T *cells_of_step = &sg[wave * 4 + (lane >> 4)][tt * D];
                            cells_of_step[ua[j]] += sum_first;
                            if (ub[j] != ua[j]) cells_of_step[ub[j]] += sum_last;
                        }
                    }
                }
                if constexpr (G::kSplit) {
                    // The lane's own children carry the letters a0 .. a0 + K - 1, the same for the whole wave.  Their
                    // row sums are added to the cells just written: the cell depends on the part, and a register
                    // array cannot be indexed at run time.  (The LDS operations of a wave complete in order.)
                    constexpr int KP = KF <= 2 ? 2 : KF <= 4 ? 4 : 8;
                    static_assert(KF <= 8, "one pass of exchanges holds eight letters");
                    T padded[KP];
#pragma unroll
                    for (int k = 0; k < KP; ++k) {
                        T v = T(0);
                        if (k < KF) {
                            v = gdxf[0][k < FK ? k : 0];
#pragma unroll
                            for (int q = 1; q < FQ; ++q) v = fmad<T>(gdxf[q][k < FK ? k : 0], rcp<T>(q + 1), v);
                        }
                        padded[k] = v;
                    }
                    const T r = row_totals<T, KP>(padded, lane);
                    const int li = row_letter<KP>(lane);
                    order_wave_lds();
                    if (row_writer<KP>(lane) && li < KF && a0 + li < D)
                        sg[wave * 4 + (lane >> 4)][tt * D + a0 + li] += r;
                }
            } else {
#pragma unroll
                for (int k = 0; k < D; ++k) {
                    T v = tot[k];
                    if constexpr (kParts == 4) {
                        v = row_total(v);
                        if ((lane & 15) == 0) sg[wave * 4 + (lane >> 4)][tt * D + k] = v;
                    } else {
                        v = wave_total(v);
                        if (lane == kWave - 1) sg[wave][tt * D + k] = v;
                    }
                }
            }
        };
        if constexpr (sizeof(T) == 4 && D <= 64) {
            // two register sets of increments, so the LDS reads of the next step hide behind the current one
            T dxs0[KS][D], dxp0[P], dxs1[KS][D], dxp1[P];
            T dxf0[FQ][FK], dxf1[FQ][FK];
            auto read = [&](int at, T (&dxs)[KS][D], T (&dxp)[P], T (&dxf)[FQ][FK]) {
                read_increments<T, D, P, KS>(sdx, at, u, dxs, dxp);
                if constexpr (G::kSplit) read_first_level<T, D, KF, KS>(sdx, at, a0, dxf);
            };
            int tt = nt - 1;
            read(tt, dxs0, dxp0, dxf0);
            for (; tt >= 1; tt -= 2) {
                read(tt - 1, dxs1, dxp1, dxf1);
                step(tt, dxs0, dxp0, dxf0);
                read(tt - 2 >= 0 ? tt - 2 : 0, dxs0, dxp0, dxf0);
                step(tt - 1, dxs1, dxp1, dxf1);
            }
            if (tt == 0) step(0, dxs0, dxp0, dxf0);
        } else {
            // fp64 state, or a hundred children and their adjoints, fill the register file: one set of increments
            for (int tt = nt - 1; tt >= 0; --tt) {
                T dxs[KS][D], dxp[P];
                T dxf[FQ][FK];
                read_increments<T, D, P, KS>(sdx, tt, u, dxs, dxp);
                if constexpr (G::kSplit) read_first_level<T, D, KF, KS>(sdx, tt, a0, dxf);
                step(tt, dxs, dxp, dxf);
            }
        }
        lds_barrier();
        // cell of (increment, letter) number idx in a row of `sg`
        auto cell = [](int idx) { return BS::kLetters == D ? idx : (idx / D) * BS::kLetters + idx % D; };
        if constexpr (kToPath) {
            // Time-chunked, no windows: the path gradient dL/dx[t] = g[t-1] - g[t] leaves the kernel directly.
            // Tiles are flushed from the right end of the chunk to its left end; `carry` holds g of the first
            // increment of the tile flushed before (the one to the right), whose point is written now.
            for (int idx = tid; idx < nt * D; idx += G::kBlock) {
                const int at = cell(idx);
                T v = sg[0][at];
#pragma unroll
                for (int q = 1; q < G::kWaves * kParts; ++q) v += sg[q][at];
                sg[0][at] = v;
            }
            lds_barrier();
            T *gp = grad_path + (b * shape.L + span.start + t0) * D;
            const bool rightmost = ti == ntiles - 1;
            if (ti < 0) {
                // ghost step: g[begin - 1] completes the first point of the chunk
                for (int k = tid; k < D; k += G::kBlock) gp[D + k] = sg[0][cell(k)] - carry[k];
            } else {
                for (int idx = tid; idx < nt * D; idx += G::kBlock) {
                    const T cur = sg[0][cell(idx)];
                    if (idx >= D) gp[idx] = sg[0][cell(idx - D)] - cur;
                    if (idx >= (nt - 1) * D) {
                        // the point to the right of the tile: the final point of the row, or the first point of
                        // the tile flushed before
                        const int k = idx - (nt - 1) * D;
                        if (!rightmost) gp[idx + D] = cur - carry[k];
                        else if (c == chunks - 1) gp[idx + D] = cur;
                    }
                }
                lds_barrier();
                for (int k = tid; k < D; k += G::kBlock) {
                    const T first = sg[0][cell(k)];
                    if (ti == 0 && !ghost) gp[k] = -first;  // the first point of the row: nothing on its left
                    carry[k] = first;
                }
            }
        } else {
            for (int idx = tid; idx < nt * D; idx += G::kBlock) {
                const int at = cell(idx);
                T v = sg[0][at];
#pragma unroll
                for (int q = 1; q < G::kWaves * kParts; ++q) v += sg[q][at];
                if constexpr (ACCUMULATE) {
                    atomicAdd(&ginc[t0 * D + idx], v);
                } else {
                    ginc[t0 * D + idx] = v;
                }
            }
        }
    }
}

// BOUNDED: the upstream gradient is zero on every top-level word outside the letter bounds in `bounds` (see
// LetterBounds).  Every wave runs the copy of the sweep compiled for its bound; all copies meet at the same
// barriers.
template <typename T, int D, int N, int P, bool ACCUMULATE, bool CHUNKED, bool BOUNDED = false, int MAXW = 0>
__global__ void __launch_bounds__((Geometry<D, N, P, sizeof(T), MAXW>::kBlock))
    dense_backward_kernel(const T *__restrict__ path, const T *__restrict__ sig, const T *__restrict__ grad_sig,
                          const T *__restrict__ edgeA, const T *__restrict__ edgeZ, T *__restrict__ grad_inc,
                          SigShape shape, int chunks, T *__restrict__ grad_path = nullptr,
                          const int *__restrict__ bounds = nullptr, const T *__restrict__ edgeL = nullptr,
                          const T *__restrict__ edgeR = nullptr) {
    using BS = BackwardShape<T, D, N, P, MAXW>;
    static_assert(!BOUNDED || LetterBounds<D, P>::kUsable, "letter bounds need one first letter per wave");
    __shared__ __align__(16) T sdx[BS::kStage];
    __shared__ __align__(16) T sg[BS::kSums][BS::kSumRow];
    __shared__ T cells[BS::kCells];
    __shared__ __align__(16) T slab[BS::kSlabElems];
    __shared__ T carry[D];  // kToPath: per-letter sums of the first increment of the tile flushed before
    using G = Geometry<D, N, P, sizeof(T), MAXW>;
    static_assert((G::kUnitBlocks == 1 || ACCUMULATE) &&
                      (!G::kOnePiece || (G::kLetterBlocks ? (CHUNKED && BOUNDED) : (!CHUNKED && !BOUNDED))),
                  "a unit of several blocks adds its per-increment sums in memory; it is swept in one piece, or, "
                  "with letter bounds, in time chunks by letter blocks");
    const int tid = (int)threadIdx.x;
    if constexpr (BOUNDED) {
        const int pu = G::kLetterBlocks ? tid + part_of_block<G>() * G::kBlock : LetterBounds<D, P>::prefix_of_thread(tid);
        const int lo = LetterBounds<D, P>::of_wave(bounds, pu);
        dispatch_value<0, D>(lo, [&](auto loc) {
            dense_backward_body<T, D, N, P, ACCUMULATE, CHUNKED, decltype(loc)::value, MAXW>(
                path, sig, grad_sig, edgeA, edgeZ, grad_inc, shape, chunks, grad_path, pu, tid, sdx, sg, cells, slab, carry,
                edgeL, edgeR);
        });
    } else {
        const int pu = G::kUnitBlocks > 1 ? tid + part_of_block<G>() * G::kBlock : tid;
        dense_backward_body<T, D, N, P, ACCUMULATE, CHUNKED, 0, MAXW>(path, sig, grad_sig, edgeA, edgeZ, grad_inc,
                                                                      shape, chunks, grad_path, pu, tid, sdx, sg, cells,
                                                                      slab, carry, edgeL, edgeR);
    }
}

// ---------------------------------------------------------------------------------------------
// host side: table of compiled shapes and launch sequences
// ---------------------------------------------------------------------------------------------
// X(index, D, N, P, PC, PS): signature over D letters to depth N; the sweep kernels put lanes on prefixes
// of length P, the per-row combine kernel on prefixes of length PC and the per-row scan kernel (which
// works on levels below N) on prefixes of length PS.  The backward also runs the forward kernel of
// depth N-1 (same P) to get chunk signatures below the top level.
// A (D, N) listed twice: the entry with the shorter prefix comes first and is taken when the call has enough
// rows to fill the GPU with it; otherwise the longer prefix (more lanes per row, a few more chain FMAs per
// lane) is taken.
#define PSIG_VARIANTS(X) \
    X(0, 4, 6, 3, 5, 4) X(1, 8, 4, 2, 3, 2) X(2, 6, 5, 3, 3, 3) X(3, 4, 4, 2, 3, 2) X(4, 3, 5, 3, 4, 3) \
    X(5, 2, 8, 5, 7, 6) X(6, 8, 5, 3, 4, 3) X(7, 8, 4, 3, 3, 2) X(8, 3, 6, 3, 5, 4) X(9, 4, 5, 3, 4, 3) \
    X(10, 5, 4, 2, 3, 2) X(11, 5, 5, 3, 4, 3) X(12, 5, 6, 4, 4, 4) X(13, 6, 4, 2, 3, 2) X(14, 7, 4, 2, 3, 2) \
    X(15, 7, 5, 3, 3, 3) X(16, 2, 2, 1, 1, 1) X(17, 3, 2, 1, 1, 1) X(18, 4, 2, 1, 1, 1) X(19, 5, 2, 1, 1, 1) \
    X(20, 6, 2, 1, 1, 1) X(21, 7, 2, 1, 1, 1) X(22, 8, 2, 1, 1, 1) X(23, 2, 3, 2, 2, 1) X(24, 3, 3, 2, 2, 1) \
    X(25, 4, 3, 2, 2, 1) X(26, 5, 3, 2, 2, 1) X(27, 6, 3, 2, 2, 1) X(28, 7, 3, 2, 2, 1) X(29, 8, 3, 2, 2, 1) \
    X(30, 2, 4, 3, 3, 2) X(31, 3, 4, 3, 3, 2) X(32, 2, 5, 4, 4, 3) X(33, 2, 6, 4, 5, 4) X(34, 6, 6, 4, 4, 3) \
    X(35, 7, 6, 4, 4, 3) X(36, 8, 6, 4, 4, 3) X(37, 9, 2, 1, 1, 1) X(38, 10, 2, 1, 1, 1) \
    X(39, 11, 2, 1, 1, 1) X(40, 12, 2, 1, 1, 1) X(41, 13, 2, 1, 1, 1) X(42, 14, 2, 1, 1, 1) \
    X(43, 15, 2, 1, 1, 1) X(44, 16, 2, 1, 1, 1) X(45, 9, 3, 2, 2, 1) X(46, 10, 3, 2, 2, 1) \
    X(47, 11, 3, 2, 2, 1) X(48, 12, 3, 2, 2, 1) X(49, 13, 3, 2, 2, 1) X(50, 14, 3, 2, 2, 1) \
    X(51, 15, 3, 2, 2, 1) X(52, 16, 3, 2, 2, 1) X(53, 9, 4, 2, 3, 2) X(54, 10, 4, 2, 3, 2) \
    X(55, 11, 4, 2, 3, 2) X(56, 12, 4, 2, 3, 2) X(57, 13, 4, 2, 3, 2) X(58, 14, 4, 2, 3, 2) \
    X(59, 15, 4, 2, 3, 2) X(60, 16, 4, 2, 3, 2) X(61, 9, 5, 3, 3, 3) X(62, 10, 5, 3, 3, 3) \
    X(63, 11, 5, 3, 3, 3) X(64, 12, 5, 3, 3, 3) X(65, 2, 7, 5, 6, 5) X(66, 3, 7, 4, 5, 4) \
    X(67, 4, 7, 4, 5, 4) X(68, 3, 8, 5, 6, 5) X(69, 2, 9, 6, 8, 7) X(70, 2, 10, 6, 8, 7) \
    X(71, 17, 2, 1, 1, 1) X(72, 18, 2, 1, 1, 1) X(73, 19, 2, 1, 1, 1) X(74, 20, 2, 1, 1, 1) \
    X(75, 21, 2, 1, 1, 1) X(76, 22, 2, 1, 1, 1) X(77, 23, 2, 1, 1, 1) X(78, 24, 2, 1, 1, 1) \
    X(79, 25, 2, 1, 1, 1) X(80, 26, 2, 1, 1, 1) X(81, 27, 2, 1, 1, 1) X(82, 28, 2, 1, 1, 1) \
    X(83, 29, 2, 1, 1, 1) X(84, 30, 2, 1, 1, 1) X(85, 31, 2, 1, 1, 1) X(86, 32, 2, 1, 1, 1) \
    X(87, 17, 3, 2, 2, 1) X(88, 18, 3, 2, 2, 1) X(89, 19, 3, 2, 2, 1) X(90, 20, 3, 2, 2, 1) \
    X(91, 21, 3, 2, 2, 1) X(92, 22, 3, 2, 2, 1) X(93, 23, 3, 2, 2, 1) X(94, 24, 3, 2, 2, 1) \
    X(95, 25, 3, 2, 2, 1) X(96, 26, 3, 2, 2, 1) X(97, 27, 3, 2, 2, 1) X(98, 28, 3, 1, 2, 1) \
    X(99, 29, 3, 1, 2, 1) X(100, 30, 3, 1, 2, 1) X(101, 31, 3, 1, 2, 1) X(102, 32, 3, 1, 2, 1) \
    X(103, 33, 2, 1, 1, 1) X(104, 34, 2, 1, 1, 1) X(105, 35, 2, 1, 1, 1) X(106, 36, 2, 1, 1, 1) \
    X(107, 37, 2, 1, 1, 1) X(108, 38, 2, 1, 1, 1) X(109, 39, 2, 1, 1, 1) X(110, 40, 2, 1, 1, 1) \
    X(111, 41, 2, 1, 1, 1) X(112, 42, 2, 1, 1, 1) X(113, 43, 2, 1, 1, 1) X(114, 44, 2, 1, 1, 1) \
    X(115, 45, 2, 1, 1, 1) X(116, 46, 2, 1, 1, 1) X(117, 47, 2, 1, 1, 1) X(118, 48, 2, 1, 1, 1) \
    X(119, 49, 2, 1, 1, 1) X(120, 50, 2, 1, 1, 1) X(121, 51, 2, 1, 1, 1) X(122, 52, 2, 1, 1, 1) \
    X(123, 53, 2, 1, 1, 1) X(124, 54, 2, 1, 1, 1) X(125, 55, 2, 1, 1, 1) X(126, 56, 2, 1, 1, 1) \
    X(127, 57, 2, 1, 1, 1) X(128, 58, 2, 1, 1, 1) X(129, 59, 2, 1, 1, 1) X(130, 60, 2, 1, 1, 1) \
    X(131, 61, 2, 1, 1, 1) X(132, 62, 2, 1, 1, 1) X(133, 63, 2, 1, 1, 1) X(134, 64, 2, 1, 1, 1) \
    X(135, 33, 3, 1, 2, 1) X(136, 34, 3, 1, 2, 1) X(137, 35, 3, 1, 2, 1) X(138, 36, 3, 1, 2, 1) \
    X(139, 37, 3, 1, 2, 1) X(140, 38, 3, 1, 2, 1) X(141, 39, 3, 1, 2, 1) X(142, 40, 3, 1, 2, 1) \
    X(143, 41, 3, 1, 2, 1) X(144, 42, 3, 1, 2, 1) X(145, 43, 3, 1, 2, 1) X(146, 44, 3, 1, 2, 1) \
    X(147, 45, 3, 1, 2, 1) X(148, 46, 3, 1, 2, 1) X(149, 47, 3, 1, 2, 1) X(150, 48, 3, 1, 2, 1) \
    X(151, 49, 3, 2, 2, 1) X(152, 50, 3, 2, 2, 1) X(153, 51, 3, 2, 2, 1) X(154, 52, 3, 2, 2, 1) \
    X(155, 53, 3, 2, 2, 1) X(156, 54, 3, 2, 2, 1) X(157, 55, 3, 2, 2, 1) X(158, 56, 3, 2, 2, 1) \
    X(159, 57, 3, 2, 2, 1) X(160, 58, 3, 2, 2, 1) X(161, 59, 3, 2, 2, 1) X(162, 60, 3, 2, 2, 1) \
    X(163, 61, 3, 2, 2, 1) X(164, 62, 3, 2, 2, 1) X(165, 63, 3, 2, 2, 1) X(166, 64, 3, 2, 2, 1) \
    X(167, 2, 11, 7, 9, 8) X(168, 3, 9, 6, 6, 6) X(169, 3, 10, 7, 6, 6) X(170, 4, 8, 5, 5, 5) \
    X(171, 5, 7, 5, 5, 4) X(172, 6, 7, 5, 5, 4) X(173, 2, 12, 7, 9, 8) X(174, 7, 7, 5, 5, 4) \
    X(175, 8, 7, 5, 5, 4) X(176, 4, 9, 6, 6, 6) X(177, 3, 11, 8, 6, 6) \
    X(178, 3, 12, 9, 6, 6) X(179, 4, 10, 7, 6, 6) X(180, 4, 11, 8, 6, 6) X(181, 5, 8, 6, 5, 5) \
    X(182, 5, 9, 7, 5, 5) X(183, 6, 8, 6, 5, 5) X(184, 7, 8, 6, 5, 5) X(185, 9, 6, 4, 4, 3) \
    X(186, 10, 6, 4, 4, 3) X(187, 11, 6, 4, 4, 3) X(188, 12, 6, 4, 4, 3) X(189, 13, 5, 3, 3, 3) \
    X(190, 14, 5, 3, 3, 3) X(191, 15, 5, 3, 3, 3) X(192, 16, 5, 3, 3, 3) X(193, 17, 4, 2, 3, 2) \
    X(194, 18, 4, 2, 3, 2) X(195, 19, 4, 2, 3, 2) X(196, 20, 4, 2, 3, 2) X(197, 21, 4, 2, 3, 2) \
    X(198, 22, 4, 2, 3, 2) X(199, 23, 4, 2, 3, 2) X(200, 24, 4, 2, 3, 2) X(201, 25, 4, 2, 3, 2) \
    X(202, 26, 4, 2, 3, 2) X(203, 27, 4, 2, 3, 2) X(204, 28, 4, 2, 3, 2) X(205, 29, 4, 2, 3, 2) \
    X(206, 30, 4, 2, 3, 2) X(207, 31, 4, 2, 3, 2) X(208, 32, 4, 2, 3, 2) \
    X(209, 9, 4, 3, 3, 2) X(210, 10, 4, 3, 3, 2) X(211, 11, 4, 3, 3, 2) X(212, 12, 4, 3, 3, 2) \
    X(213, 13, 4, 3, 3, 2) X(214, 14, 4, 3, 3, 2) X(215, 15, 4, 3, 3, 2) X(216, 9, 5, 4, 4, 3) \
    X(217, 10, 5, 4, 4, 3) X(218, 11, 5, 4, 4, 3) X(219, 12, 5, 4, 4, 3) X(220, 13, 5, 4, 4, 3) \
    X(221, 14, 5, 4, 4, 3) X(222, 15, 5, 4, 4, 3) X(223, 9, 6, 5, 5, 4) X(224, 10, 6, 5, 5, 4) \
    X(225, 11, 6, 5, 5, 4) X(226, 12, 6, 5, 5, 4) \
    X(227, 16, 4, 3, 3, 2) X(228, 16, 5, 4, 4, 3) X(229, 17, 4, 3, 3, 2) X(230, 18, 4, 3, 3, 2) \
    X(231, 19, 4, 3, 3, 2) X(232, 20, 4, 3, 3, 2) X(233, 21, 4, 3, 3, 2) X(234, 22, 4, 3, 3, 2) \
    X(235, 23, 4, 3, 3, 2) X(236, 24, 4, 3, 3, 2) X(237, 25, 4, 3, 3, 2) X(238, 26, 4, 3, 3, 2) \
    X(239, 27, 4, 3, 3, 2) X(240, 28, 4, 3, 3, 2) X(241, 29, 4, 3, 3, 2) X(242, 30, 4, 3, 3, 2) \
    X(243, 31, 4, 3, 3, 2) X(244, 32, 4, 3, 3, 2) \
    X(245, 28, 3, 2, 2, 1) X(246, 29, 3, 2, 2, 1) X(247, 30, 3, 2, 2, 1) X(248, 31, 3, 2, 2, 1) \
    X(249, 32, 3, 2, 2, 1) X(250, 33, 3, 2, 2, 1) X(251, 34, 3, 2, 2, 1) X(252, 35, 3, 2, 2, 1) \
    X(253, 36, 3, 2, 2, 1) X(254, 37, 3, 2, 2, 1) X(255, 38, 3, 2, 2, 1) X(256, 39, 3, 2, 2, 1) \
    X(257, 40, 3, 2, 2, 1) X(258, 41, 3, 2, 2, 1) X(259, 42, 3, 2, 2, 1) X(260, 43, 3, 2, 2, 1) \
    X(261, 44, 3, 2, 2, 1) X(262, 45, 3, 2, 2, 1) X(263, 46, 3, 2, 2, 1) X(264, 47, 3, 2, 2, 1) \
    X(265, 48, 3, 2, 2, 1) \
    X(266, 80, 3, 2, 2, 1) X(267, 96, 3, 2, 2, 1) X(268, 112, 3, 2, 2, 1) X(269, 72, 3, 2, 2, 1) \
    X(270, 88, 3, 2, 2, 1) X(271, 104, 3, 2, 2, 1)

// The scan kernel of the time-chunked backward streams rows of levels 1..N-1 through a double buffer and keeps
// two result rows, all in LDS; a shape whose rows are too long for that in type T is swept unchunked in T.
template <typename T, int D, int N, int PS>
constexpr bool scan_fits() {
    using GS = Geometry<D, N, PS>;
    if (N < 2 || GS::kOnePiece) return false;
    const int64_t padded = RowStager<T, (int)GS::kLowSize, GS::kBlock>::kPadded;
    return (2 * padded + 2 * GS::kLowSize) * (int64_t)sizeof(T) + 1024 <= 160 * 1024;
}

struct VariantInfo {
    int d, depth, block;  // block: threads of one unit
    int unit_blocks;      // blocks a unit is spread over (more than one: swept in one piece, dense only)
    int64_t sig_size, low_size;
    bool bounds_ok;       // the sweeps can leave out top-level words by letter bounds
    bool chunks_ok[2];    // fp32, fp64: rows can be cut into time chunks
    bool fp64_fits;       // a lane's state fits the register file in fp64 too (else a later entry of the shape serves fp64)
    bool grouped_ok;      // fp32: the hand-over of chunk products by groups of four chunks is compiled
};

// Grouped hand-over (fp32): the forward sweep, four chunks to a block, leaves the products of every chunk with its
// neighbours inside the block, a small launch the products of whole blocks, and the reverse sweep puts the two
// together (one more contraction and one more product per chunk in its prologue).  It replaces the scan over all
// chunks of a row, fifteen dependent products per direction and twice the chunk rows through memory.
template <int D, int N, int P, int PC, int PS>
constexpr bool grouped_handover_ok() {
    if constexpr (N < 4 || N - 1 < P) {
        return false;
    } else {
        using G = Geometry<D, N, P, 4>;
        using BS = BackwardShape<float, D, N, P>;
        constexpr bool staged = 2 * Geometry<D, N, PC>::kSigSize * sizeof(float) <= 48 * 1024;
        return ForwardShape<float, D, N, P, 4>::kGrouped && G::kBlock * 4 <= 1024 && staged &&
               EdgesShape<float, D, N, PS, PC>::kUsable && scan_fits<float, D, N, PS>() && BS::kSlab &&
               RowPlace<D, true>::size((int)G::kLowSize) <= BS::kSlabElems;
    }
}

template <int D, int N, int P, int PC, int PS>
constexpr VariantInfo variant_info() {
    using G = Geometry<D, N, P>;
    using G64 = Geometry<D, N, P, 8>;
    return VariantInfo{D, N, G::kUnitWaves * kWave, G::kUnitBlocks, G::kSigSize, G::kLowSize,
                       LetterBounds<D, P>::kUsable && !G::kOnePiece && D <= 16,
                       {!G::kOnePiece && scan_fits<float, D, N, PS>(),
                        !G64::kOnePiece && scan_fits<double, D, N, PS>()},
                       G::kSplit || trie_size(D, N - P) <= 132,
                       grouped_handover_ok<D, N, P, PC, PS>()};
}

constexpr size_t kBoundsBytes = 256;  // scratch for the letter bounds (16 ints, padded)

#if PSIG_GROUP < 0
// Computes the letter bounds of the top-level word list into the head of *workspace and moves *workspace
// past them; returns nullptr (and launches nothing) when the call does not use bounds.
const int *stage_letter_bounds(const DenseChoice &dc, const int64_t *top_codes, int64_t top_count, int d, int depth,
                               void **workspace, hipStream_t stream) {
    if (!dc.bounded) return nullptr;
    int *bounds = (int *)*workspace;
    *workspace = (unsigned char *)*workspace + kBoundsBytes;
    const bool narrow = (double)depth * std::log2((double)d) < 32.0;
    hipLaunchKernelGGL(letter_bounds_kernel, dim3(1), dim3(1024), 0, stream, top_codes, top_count, d, depth, narrow,
                       bounds);
    return bounds;
}

#endif

// A reduced library: -DPSIG_ONLY="{4,6},{8,4}" compiles the register-tiled kernels of the listed (d, depth) pairs
// only; every other shape then runs on the per-word kernels.  (The full table takes minutes to compile.)
#ifdef PSIG_ONLY
constexpr int kOnlyShapes[][2] = {PSIG_ONLY};
constexpr bool shape_enabled(int d, int depth) {
    for (const auto &s : kOnlyShapes)
        if (s[0] == d && s[1] == depth) return true;
    return false;
}
#else
constexpr bool shape_enabled(int, int) { return true; }
#endif

template <int D, int N, int P, int PC, int PS>
constexpr VariantInfo variant_info_if_enabled() {
    if constexpr (shape_enabled(D, N)) return variant_info<D, N, P, PC, PS>();
    else return VariantInfo{-1, -1, 0, 0, 0, 0, false, {false, false}, false, false};
}

#define PSIG_INFO(I, D, N, P, PC, PS) variant_info_if_enabled<D, N, P, PC, PS>(),
constexpr VariantInfo kVariants[] = {PSIG_VARIANTS(PSIG_INFO)};
#undef PSIG_INFO
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

size_t pad256(size_t n) { return (n + 255) / 256 * 256; }

#if PSIG_GROUP < 0
struct SweepProfile {
    bool enabled = false, valid = false;
    hipEvent_t start = nullptr, stop = nullptr;
} g_profile;

void profile_mark(bool begin, hipStream_t stream) {
    if (!g_profile.enabled) return;
    if (!g_profile.start) {
        if (hipEventCreate(&g_profile.start) != hipSuccess || hipEventCreate(&g_profile.stop) != hipSuccess) return;
    }
    (void)hipEventRecord(begin ? g_profile.start : g_profile.stop, stream);
    if (!begin) g_profile.valid = true;
}

// number of time chunks per row: enough waves to give every SIMD of the GPU about two (want_waves = 2048), but
// chunks of at least 16 increments
int pick_chunks(int64_t rows, int block, int64_t L, int64_t want_waves) {
    const int64_t waves_per_row = block / kWave;
    int64_t c = (want_waves + rows * waves_per_row - 1) / (rows * waves_per_row);
    const int64_t max_c = (L - 1) / 16;
    if (c > max_c) c = max_c;
    if (c > 64) c = 64;
    if (c >= 4) c = (c + 3) / 4 * 4 <= max_c ? (c + 3) / 4 * 4 : c / 4 * 4;  // whole blocks of four chunks
    if (c < 1) c = 1;
    return (int)c;
}

#endif

template <typename T, int D, int N, int P, int GW>
constexpr bool group_fits() {
    return Geometry<D, N, P, sizeof(T)>::kBlock * GW <= 1024 && forward_lds_bytes<D, N, P, GW, T>() <= 64 * 1024;
}

// Prefix products edgeA and suffix products edgeZ of the chunk signatures below the top level (dense_scan_kernel).
template <typename T, int D, int N, int PS>
hipError_t launch_scan(const T *chunk_low, T *edgeA, T *edgeZ, int64_t rows, int chunks, hipStream_t stream) {
    using GC = Geometry<D, N, PS>;

    // all chunk rows of a row go to LDS at once when they fit (a little under the 160 KB of a CU)
    const size_t resident_bytes = (size_t)chunks * GC::kLowSize * sizeof(T);
    const size_t fixed_bytes = 2 * GC::kLowSize * sizeof(T) + 1024;
    if (resident_bytes + fixed_bytes <= 150 * 1024) {
        auto kernel = dense_scan_kernel<T, D, N, PS, true>;
        if (resident_bytes > 48 * 1024) {
            hipError_t e = allow_dynamic_lds<dense_scan_kernel<T, D, N, PS, true>>(resident_bytes);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kernel, dim3((unsigned)rows, 2), dim3(GC::kBlock + kCopyThreads), resident_bytes, stream,
                           chunk_low, edgeA, edgeZ, chunks, (T *)nullptr, (int64_t)0);
    } else {
        hipLaunchKernelGGL((dense_scan_kernel<T, D, N, PS, false>), dim3((unsigned)rows, 2),
                           dim3(GC::kBlock + kCopyThreads), 0, stream, chunk_low, edgeA, edgeZ, chunks, (T *)nullptr,
                           (int64_t)0);
    }
    return hipGetLastError();
}

// keep (optional): receives the prefix and suffix products of the chunk signatures below the top level, which the
// time-chunked backward of the same call starts its chunks from: [rows, chunks, low] twice, the second array
// pad256 bytes after the start of the first.
template <typename T, int D, int N, int P, int PC, int PS>
hipError_t run_forward(const T *path, T *sig, const SigShape &shape, int chunks, const int *bounds, T *keep,
                       void *workspace, hipStream_t stream, bool grouped) {
    using G = Geometry<D, N, P, sizeof(T)>;
    using GC = Geometry<D, N, PC>;
    constexpr bool kStaged = 2 * GC::kSigSize * sizeof(T) <= 48 * 1024;
    constexpr bool kBoundsOk = LetterBounds<D, P>::kUsable && !G::kOnePiece;
    const int64_t rows = shape.B * shape.W;
    if (bounds && !kBoundsOk) return hipErrorInvalidValue;
    if (chunks <= 1) {
        if constexpr (kBoundsOk) {
            if (bounds) {
                hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P, 1, true>), dim3((unsigned)rows), dim3(G::kBlock),
                                   0, stream, path, sig, shape, 1, (T *)nullptr, bounds);
                return hipGetLastError();
            }
        }
        hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P, 1>), dim3((unsigned)(rows * G::kUnitBlocks)),
                           dim3(G::kBlock), 0, stream, path, sig, shape, 1);
        return hipGetLastError();
    }
    if constexpr (G::kOnePiece) {
        return hipErrorNotSupported;  // such shapes are never cut into time chunks (dense_choice)
    } else {
    // chunks are swept GW to a block when that divides the chunk count and fits the block and LDS limits;
    // a row that fits one block goes straight to the output, without the combine launch
    T *chunk_sig = (T *)workspace;
    // the chunks' own signatures below the top level, from which the products for the backward are made
    T *chunk_low = keep ? (T *)((unsigned char *)workspace + pad256((size_t)rows * chunks * G::kSigSize * sizeof(T)))
                        : (T *)nullptr;
    if constexpr (sizeof(T) == 4 && grouped_handover_ok<D, N, P, PC, PS>()) {
        if (keep && grouped && !bounds && chunks % 4 == 0 && chunks >= 8) {
            // grouped hand-over: keep = [in-group prefix products][in-group suffix products], both
            // [rows, chunks, low], then [products of the groups to the left][.. to the right], both
            // [rows, chunks / 4, low]
            using ES = EdgesShape<T, D, N, PS, PC>;
            const int groups4 = chunks / 4;
            const size_t unit_bytes = pad256((size_t)rows * chunks * G::kLowSize * sizeof(T));
            const size_t group_bytes = pad256((size_t)rows * groups4 * G::kLowSize * sizeof(T));
            T *in_suffix = (T *)((unsigned char *)keep + unit_bytes);
            T *edgeL = (T *)((unsigned char *)keep + 2 * unit_bytes);
            T *edgeR = (T *)((unsigned char *)keep + 2 * unit_bytes + group_bytes);
            hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P, 4>), dim3((unsigned)(rows * groups4)),
                               dim3(G::kBlock * 4), 0, stream, path, chunk_sig, shape, chunks, (T *)nullptr,
                               (const int *)nullptr, keep, in_suffix);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
            auto kernel = dense_group_edges_kernel<T, D, N, PS, PC>;
            if (ES::kCombineBytes > 48 * 1024) {
                e = allow_dynamic_lds<dense_group_edges_kernel<T, D, N, PS, PC>>(ES::kCombineBytes);
                if (e != hipSuccess) return e;
            }
            hipLaunchKernelGGL(kernel, dim3((unsigned)rows, 1 + ES::kCombineParts), dim3(ES::kThreads),
                               ES::kCombineBytes, stream, (const T *)chunk_sig, edgeL, edgeR, sig, groups4);
            return hipGetLastError();
        }
    }
    int groups = chunks;
    if constexpr (kBoundsOk) {
        if (bounds) {
            // bounded sweeps exist one chunk to a block only; in fp32 they run in letter blocks, one wave to a
            // block (in fp64 a wave alone takes more registers than two of them have together on a SIMD)
            if constexpr (sizeof(T) == 4) {
                using GL = Geometry<D, N, P, sizeof(T), 1>;
                hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P, 1, true, 1>),
                                   dim3((unsigned)(rows * chunks * GL::kUnitBlocks)), dim3(GL::kBlock), 0, stream, path,
                                   chunk_sig, shape, chunks, (T *)nullptr, bounds, chunk_low);
            } else {
                hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P, 1, true>), dim3((unsigned)(rows * chunks)),
                                   dim3(G::kBlock), 0, stream, path, chunk_sig, shape, chunks, (T *)nullptr, bounds,
                                   chunk_low);
            }
            groups = -1;
        }
    }
    if constexpr (group_fits<T, D, N, P, 4>()) {
        if (groups == chunks && chunks % 4 == 0) {
            groups = chunks / 4;
            hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P, 4>), dim3((unsigned)(rows * groups)),
                               dim3(G::kBlock * 4), 0, stream, path, groups == 1 ? sig : chunk_sig, shape, chunks,
                               (T *)nullptr, (const int *)nullptr, chunk_low);
        }
    }
    if constexpr (group_fits<T, D, N, P, 2>()) {
        if (groups == chunks && chunks % 2 == 0) {
            groups = chunks / 2;
            hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P, 2>), dim3((unsigned)(rows * groups)),
                               dim3(G::kBlock * 2), 0, stream, path, groups == 1 ? sig : chunk_sig, shape, chunks,
                               (T *)nullptr, (const int *)nullptr, chunk_low);
        }
    }
    if (groups == chunks)
        hipLaunchKernelGGL((dense_forward_kernel<T, D, N, P, 1>), dim3((unsigned)(rows * chunks)), dim3(G::kBlock), 0,
                           stream, path, chunk_sig, shape, chunks, (T *)nullptr, (const int *)nullptr, chunk_low);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (groups < 0) groups = chunks;
    if (keep) {
        if constexpr (scan_fits<T, D, N, PS>()) {
            T *edgeZ = (T *)((unsigned char *)keep + pad256((size_t)rows * chunks * G::kLowSize * sizeof(T)));
            if constexpr (kStaged && EdgesShape<T, D, N, PS, PC>::kUsable) {
                // the products for the backward and the product of the partial signatures in one launch, when
                // all but kEdgeExtra of the chunk rows of a scan fit the LDS share of a block
                using ES = EdgesShape<T, D, N, PS, PC>;
                const size_t room = ES::kBudget - ES::kStaticBytes;
                const int used = chunks - 1;
                const int resident = (int)std::min<size_t>((size_t)used, room / ES::kRowBytes);
                if (groups > 1 && resident >= 2 && used - resident <= kEdgeExtra) {
                    const size_t dynamic = std::max((size_t)resident * ES::kRowBytes, ES::kCombineBytes);
                    auto kernel = dense_edges_kernel<T, D, N, PS, PC>;
                    if (dynamic > 48 * 1024) {
                        e = allow_dynamic_lds<dense_edges_kernel<T, D, N, PS, PC>>(dynamic);
                        if (e != hipSuccess) return e;
                    }
                    hipLaunchKernelGGL(kernel, dim3((unsigned)rows, 2 + ES::kCombineParts), dim3(ES::kThreads),
                                       dynamic, stream, (const T *)chunk_low, keep, edgeZ, chunks, resident,
                                       (const T *)chunk_sig, sig, groups);
                    return hipGetLastError();
                }
            }
            e = launch_scan<T, D, N, PS>((const T *)chunk_low, keep, edgeZ, rows, chunks, stream);
            if (e != hipSuccess) return e;
        } else {
            return hipErrorNotSupported;  // such shapes are never cut into time chunks (dense_choice)
        }
    }
    if (groups == 1) return hipSuccess;
    if constexpr (kStaged)
        hipLaunchKernelGGL((dense_combine_kernel<T, D, N, PC, true>), dim3((unsigned)rows), dim3(GC::kBlock), 0, stream,
                           (const T *)chunk_sig, sig, groups);
    else
        hipLaunchKernelGGL((dense_combine_kernel<T, D, N, PC, false>), dim3((unsigned)rows, (unsigned)GC::kUnitWaves),
                           dim3(kWave), 0, stream, (const T *)chunk_sig, sig, groups, bounds);
    return hipGetLastError();
    }
}

template <typename T, int D, int N, int P, int PC, int PS>
hipError_t run_backward(const T *path, const T *sig, const T *grad_sig, T *grad_inc, T *grad_path, bool *wrote_path,
                        const SigShape &shape, int chunks, const int *bounds, const T *kept, void *workspace,
                        hipStream_t stream, bool grouped, bool inc_cleared) {
    using G = Geometry<D, N, P, sizeof(T)>;
    using GC = Geometry<D, N, PS>;
    constexpr bool kBoundsOk = LetterBounds<D, P>::kUsable && !G::kOnePiece;
    const int64_t rows = shape.B * shape.W;
    // per-increment sums are added in memory for overlapping windows and for units spread over several blocks
    // (among them the letter blocks of a sweep with letter bounds)
    const bool accumulate =
        shape.windows != nullptr || G::kUnitBlocks > 1 || (bounds != nullptr && kBoundsOk && sizeof(T) == 4);
    *wrote_path = false;
    hipError_t e;
    // bounded sweeps exist for time-chunked calls only (every call that embeds a projection is chunked)
    if (bounds && (!kBoundsOk || chunks <= 1)) return hipErrorInvalidValue;
    if (accumulate && !inc_cleared) {
        e = launch_fill_zero<T>(grad_inc, shape.B * (shape.L - 1) * shape.d, stream);
        if (e != hipSuccess) return e;
    }
    if (rows == 0) return hipSuccess;
    if (chunks <= 1) {
        profile_bracket(true, stream);
        if (accumulate) {
            hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, true, false>),
                               dim3((unsigned)(rows * G::kUnitBlocks)), dim3(G::kBlock), 0, stream, path, sig, grad_sig,
                               (const T *)nullptr, (const T *)nullptr, grad_inc, shape, 1);
        } else {
            if constexpr (G::kUnitBlocks == 1)
                hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, false, false>), dim3((unsigned)rows),
                                   dim3(G::kBlock), 0, stream, path, sig, grad_sig, (const T *)nullptr,
                                   (const T *)nullptr, grad_inc, shape, 1);
        }
        profile_bracket(false, stream);
        return hipGetLastError();
    }
    if constexpr (G::kOnePiece || !scan_fits<T, D, N, PS>()) {
        // never cut into time chunks (dense_choice): shapes whose units take several blocks, rows too long for
        // the scan kernel's LDS in this type
        return hipErrorNotSupported;
    } else {
        const int64_t units = rows * chunks;
        const size_t edge_bytes = pad256((size_t)units * G::kLowSize * sizeof(T));
        const T *dumpA, *dumpH;
        const T *edgeL = nullptr, *edgeR = nullptr;  // grouped hand-over: products of whole groups of chunks
        if (kept) {
            // the forward of this call left the prefix and suffix products of its chunk signatures
            dumpA = kept;
            dumpH = (const T *)((const unsigned char *)kept + edge_bytes);
            if constexpr (sizeof(T) == 4 && grouped_handover_ok<D, N, P, PC, PS>()) {
                if (grouped && !bounds && chunks % 4 == 0 && chunks >= 8) {
                    const size_t group_bytes = pad256((size_t)rows * (chunks / 4) * G::kLowSize * sizeof(T));
                    edgeL = (const T *)((const unsigned char *)kept + 2 * edge_bytes);
                    edgeR = (const T *)((const unsigned char *)kept + 2 * edge_bytes + group_bytes);
                }
            }
        } else {
            unsigned char *ws = (unsigned char *)workspace;
            T *chunk_low = (T *)ws;
            T *edgeA = (T *)(ws + edge_bytes), *edgeZ = (T *)(ws + 2 * edge_bytes);
            // chunk signatures below the top level: the depth N-1 forward kernel on the same units
            // (the forward kernel needs a prefix shorter than its depth; the layout it writes does not depend on it)
            if constexpr (N == 2) {
                hipLaunchKernelGGL(chunk_level1_kernel<T>, dim3((unsigned)units), dim3(kWave), 0, stream, path, chunk_low,
                                   shape, chunks, (T *)nullptr);
            } else {
                constexpr int PK = P <= N - 2 ? P : N - 2;
                hipLaunchKernelGGL((dense_forward_kernel<T, D, N - 1, PK, 1>), dim3((unsigned)units),
                                   dim3(Geometry<D, N - 1, PK, sizeof(T)>::kBlock), 0, stream, path, chunk_low, shape, chunks,
                                   (T *)nullptr);
            }
            e = hipGetLastError();
            if (e != hipSuccess) return e;
            e = launch_scan<T, D, N, PS>((const T *)chunk_low, edgeA, edgeZ, rows, chunks, stream);
            if (e != hipSuccess) return e;
            dumpA = edgeA;
            dumpH = edgeZ;
        }
        profile_bracket(true, stream);
        bool launched = false;
        if constexpr (kBoundsOk) {
            if (bounds) {
                if constexpr (sizeof(T) == 4) {
                    // letter blocks (see Geometry::kLetterBlocks): the per-increment sums meet in memory
                    using GL = Geometry<D, N, P, sizeof(T), 1>;
                    hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, true, true, true, 1>),
                                       dim3((unsigned)(units * GL::kUnitBlocks)), dim3(GL::kBlock), 0, stream, path, sig,
                                       grad_sig, dumpA, dumpH, grad_inc, shape, chunks, (T *)nullptr, bounds);
                } else if (accumulate) {
                    hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, true, true, true>), dim3((unsigned)units),
                                       dim3(G::kBlock), 0, stream, path, sig, grad_sig, dumpA,
                                       dumpH, grad_inc, shape, chunks, (T *)nullptr, bounds);
                } else {
                    hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, false, true, true>), dim3((unsigned)units),
                                       dim3(G::kBlock), 0, stream, path, sig, grad_sig, dumpA,
                                       dumpH, grad_inc, shape, chunks, grad_path, bounds);
                }
                launched = true;
            }
        }
        if (!launched) {
            if (accumulate)
                hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, true, true>), dim3((unsigned)units),
                                   dim3(G::kBlock), 0, stream, path, sig, grad_sig, dumpA, dumpH,
                                   grad_inc, shape, chunks, (T *)nullptr, (const int *)nullptr, edgeL, edgeR);
            else
                hipLaunchKernelGGL((dense_backward_kernel<T, D, N, P, false, true>), dim3((unsigned)units),
                                   dim3(G::kBlock), 0, stream, path, sig, grad_sig, dumpA, dumpH,
                                   grad_inc, shape, chunks, grad_path, (const int *)nullptr, edgeL, edgeR);
        }
        if (!accumulate) *wrote_path = true;
        profile_bracket(false, stream);
        return hipGetLastError();
    }
}

}  // namespace

#if PSIG_GROUP < 0
void profile_bracket(bool begin, hipStream_t stream) { profile_mark(begin, stream); }

void profile_enable(bool on) {
    g_profile.enabled = on;
    g_profile.valid = false;
}

float profile_sweep_ms() {
    if (!g_profile.valid) return -1.0f;
    float ms = -1.0f;
    if (hipEventSynchronize(g_profile.stop) != hipSuccess) return -1.0f;
    if (hipEventElapsedTime(&ms, g_profile.start, g_profile.stop) != hipSuccess) return -1.0f;
    return ms;
}

DenseChoice dense_choice(size_t elem, int64_t d, int depth, bool all_dense, const int64_t *level_sizes, int64_t B,
                         int64_t L, int64_t W, bool) {
    DenseChoice dc{};
    dc.variant = -1;
    dc.fwd_chunks = dc.bwd_chunks = 1;
    if (B <= 0 || W <= 0 || options().tiled == 0) return dc;
    for (int i = 0; i < kNumVariants; ++i) {
        const VariantInfo &v = kVariants[i];
        if (v.d != d || v.depth != depth) continue;
        const int64_t rows = B * W;
        {
            // a later entry for the same (d, depth) has more lanes per row: take it when this one cannot
            // put about a wave on every SIMD even with the most time chunks the path allows
            bool later = false;
            for (int j = i + 1; j < kNumVariants; ++j) later = later || (kVariants[j].d == d && kVariants[j].depth == depth);
            const int64_t max_chunks = (L - 1) / 16 < 1 ? 1 : ((L - 1) / 16 > 64 ? 64 : (L - 1) / 16);
            // (a shape that is not cut into chunks has its rows only; half a wave per SIMD is then enough to take it,
            // the later entry being two to three times slower per coefficient)
            const bool cut = v.chunks_ok[elem == 8 ? 1 : 0];
            if (later && rows * (v.block / kWave) * (cut ? max_chunks : 1) < (cut ? 1024 : 512)) continue;
            // the short prefixes of the wide alphabets hold 68 to 240 values per lane: fp64 up to 132 (d = 11) and
            // wherever the children are split
            if (later && elem == 8 && !v.fp64_fits) continue;
        }
        const bool chunks_ok = v.chunks_ok[elem == 8 ? 1 : 0];
        if (!all_dense) {
            // A word projection is computed densely and gathered when that is the cheaper way: when its top level
            // keeps a fair share of the dense one (the top level dominates the cost), or when the dense sweep is
            // small against what the per-word kernels cost.  Those sweep the path one increment after the other
            // whatever the number of words (about 1.7 us per increment), or about 4 ns per thousand (word, path,
            // increment) when there are many; the dense kernels run at 40 TFLOP/s or more (25 for alphabets of more
            // than eight letters; fp64: half) on 10 flops per signature coefficient, path and increment, and a
            // step costs 80 us at least.
            // The time-chunked backward rebuilds what it reads; for a shape that is not cut into chunks the
            // backward needs the dense signature itself, kept by the forward or swept again (a second buffer).
            if (!level_sizes) return dc;
            const int64_t top_dense = v.sig_size - v.low_size;
            const int64_t share = options().embed_share;
            if (share == 0) return dc;
            if (share > 0) {
                if ((double)level_sizes[depth] * (double)share < (double)top_dense) return dc;
            } else if (level_sizes[depth] * 8 < top_dense) {
                double words = 0;
                for (int k = 1; k <= depth; ++k) words += (double)level_sizes[k];
                const double steps = (double)(L - 1);
                const double per_word_us = std::max(1.7 * steps, 3.9e-6 * words * (double)rows * steps);
                const double dense_us =
                    std::max(80.0, 10.0 * (double)v.sig_size * (double)rows * steps / (v.d <= 8 ? 40e6 : 25e6) *
                                       (elem == 8 ? 2.0 : 1.0));
                if (dense_us > 0.8 * per_word_us) return dc;
            }
            if ((double)rows * (double)v.sig_size * (double)elem * (chunks_ok ? 1.0 : 2.0) > 4e9) return dc;
            dc.embed = true;
            dc.resweep = !chunks_ok;
            dc.dense_bytes = pad256((size_t)rows * v.sig_size * elem);
            dc.bounded = chunks_ok && v.bounds_ok && level_sizes[depth] > 0 && level_sizes[depth] < top_dense &&
                         options().letter_bounds != 0;
        }
        // (letter blocks: twice the waves that fit the GPU at once, so that the short ones fill in behind the long)
        int chunks = pick_chunks(rows, v.block, L, dc.bounded && elem == 4 ? 4096 : 2048);
        // deep fp32 shapes: the reverse sweep rebuilds A_t = A_{t+1} (x) exp(-dx_t) step by step, and over a span of
        // large increments that roll-back loses digits at depth 9 and more (d = 2, depth 12, five increments of
        // size 0.8: gradient off by 1.5e-5 in one piece, 1e-6 in two or more); four chunks at least
        if (elem == 4 && depth >= 9 && chunks < 4) chunks = (int)std::max<int64_t>(1, std::min<int64_t>(4, L - 1));
        if (const int64_t forced = options().chunks; forced >= 1 && forced <= 1024) chunks = (int)forced;
        // not chunked: units of several blocks (a row is dozens of waves already), rows too long for the scan
        // kernel's LDS
        if (!chunks_ok) chunks = 1;
        if (rows * (chunks + 1) >= (int64_t(1) << 31)) return dc;
        dc.usable = true;
        dc.variant = i;
        dc.fwd_chunks = chunks;
        dc.bwd_chunks = (dc.embed && !dc.resweep && chunks < 2) ? 2 : chunks;
        dc.forward_workspace = dc.dense_bytes + (dc.bounded ? kBoundsBytes : 0);
        dc.backward_workspace = (dc.resweep ? 2 : 1) * dc.dense_bytes + (dc.bounded ? kBoundsBytes : 0);
        // forward: the chunk signatures, and those below the top level from which a keeping forward makes the
        // products its backward starts from; backward: the latter and the two arrays of products
        if (dc.fwd_chunks > 1)
            dc.forward_workspace += pad256((size_t)rows * dc.fwd_chunks * v.sig_size * elem) +
                                    pad256((size_t)rows * dc.fwd_chunks * v.low_size * elem);
        if (dc.bwd_chunks > 1) dc.backward_workspace += 3 * pad256((size_t)rows * dc.bwd_chunks * v.low_size * elem);
        // the forward can hand those products to the backward when both cut the rows the same way
        if (dc.bwd_chunks > 1 && dc.fwd_chunks == dc.bwd_chunks) {
            dc.keep_bytes = 2 * pad256((size_t)rows * dc.bwd_chunks * v.low_size * elem);
            // grouped hand-over (see grouped_handover_ok): whole groups of four chunks, two groups at least
            dc.grouped = elem == 4 && v.grouped_ok && !dc.embed && chunks % 4 == 0 && chunks >= 8 &&
                         options().grouped != 0;
            if (dc.grouped) dc.keep_bytes += 2 * pad256((size_t)rows * (chunks / 4) * v.low_size * elem);
        }
        if (dc.resweep) dc.keep_bytes = (size_t)rows * v.sig_size * elem;
        return dc;
    }
    return dc;
}

// f(std::integral_constant<int, g>) for the group g of a shape
template <int GI = 0, typename F>
void dispatch_group(int group, F &&f) {
    if constexpr (GI + 1 >= kDenseGroups) {
        f(std::integral_constant<int, GI>{});
    } else {
        if (group == GI) f(std::integral_constant<int, GI>{});
        else dispatch_group<GI + 1>(group, f);
    }
}

template <typename T>
hipError_t launch_dense_forward(const T *path, T *sig, const SigShape &shape, const DenseChoice &dc,
                                const int64_t *top_codes, int64_t top_count, T *keep, void *workspace,
                                hipStream_t stream) {
    if (dc.variant < 0 || dc.variant >= kNumVariants) return hipErrorNotSupported;
    if (keep && dc.keep_bytes == 0) return hipErrorInvalidValue;
    const int *bounds = stage_letter_bounds(dc, top_codes, top_count, kVariants[dc.variant].d,
                                            kVariants[dc.variant].depth, &workspace, stream);
    hipError_t e = hipErrorNotSupported;
    dispatch_group(dc.variant % kDenseGroups, [&](auto g) {
        e = launch_dense_forward_group<decltype(g)::value, T>(path, sig, shape, dc, bounds, keep, workspace, stream);
    });
    return e;
}

template <typename T>
hipError_t launch_dense_backward(const T *path, const T *sig, const T *grad_sig, T *grad_inc, T *grad_path,
                                 bool *wrote_path, const SigShape &shape, const DenseChoice &dc,
                                 const int64_t *top_codes, int64_t top_count, const T *kept, void *workspace,
                                 bool prepared, hipStream_t stream) {
    if (dc.variant < 0 || dc.variant >= kNumVariants) return hipErrorNotSupported;
    if (kept && dc.keep_bytes == 0) return hipErrorInvalidValue;
    const int *bounds = nullptr;
    if (prepared && dc.bounded) {
        bounds = (const int *)workspace;
        workspace = (unsigned char *)workspace + kBoundsBytes;
    } else {
        bounds = stage_letter_bounds(dc, top_codes, top_count, kVariants[dc.variant].d, kVariants[dc.variant].depth,
                                     &workspace, stream);
    }
    hipError_t e = hipErrorNotSupported;
    dispatch_group(dc.variant % kDenseGroups, [&](auto g) {
        e = launch_dense_backward_group<decltype(g)::value, T>(path, sig, grad_sig, grad_inc, grad_path, wrote_path,
                                                               shape, dc, bounds, kept, workspace, prepared, stream);
    });
    return e;
}

template <typename T>
hipError_t prepare_dense_backward(const DenseChoice &dc, T *zero, int64_t count, const int64_t *top_codes,
                                  int64_t top_count, void *bounds_at, hipStream_t stream) {
    if (dc.variant < 0 || dc.variant >= kNumVariants) return hipErrorNotSupported;
    const int d = kVariants[dc.variant].d, depth = kVariants[dc.variant].depth;
    const bool narrow = (double)depth * std::log2((double)d) < 32.0;
    int64_t blocks = (count / (16 / (int64_t)sizeof(T)) + 1023) / 1024 + 1;  // one thread per 16-byte piece
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(zero_and_bounds_kernel<T>, dim3((unsigned)blocks + 1), dim3(1024), 0, stream, zero, count,
                       top_codes, top_count, d, depth, narrow, dc.bounded ? (int *)bounds_at : (int *)nullptr);
    return hipGetLastError();
}

#define PSIG_INSTANTIATE(T)                                                                                      \
    template hipError_t launch_dense_forward<T>(const T *, T *, const SigShape &, const DenseChoice &,            \
                                                const int64_t *, int64_t, T *, void *, hipStream_t);             \
    template hipError_t launch_dense_backward<T>(const T *, const T *, const T *, T *, T *, bool *, const SigShape &, \
                                                 const DenseChoice &, const int64_t *, int64_t, const T *, void *,  \
                                                 bool, hipStream_t);                                                \
    template hipError_t prepare_dense_backward<T>(const DenseChoice &, T *, int64_t, const int64_t *, int64_t,      \
                                                  void *, hipStream_t);
PSIG_INSTANTIATE(float)
PSIG_INSTANTIATE(double)
#undef PSIG_INSTANTIATE

#else  // the kernels and launch sequences of one group of shapes

static_assert(PSIG_GROUP < kDenseGroups, "group index out of range");

#define PSIG_CASE_FWD(I, D, N, P, PC, PS)                                                                         \
    case I:                                                                                                       \
        if constexpr (I % kDenseGroups == PSIG_GROUP && shape_enabled(D, N))                                      \
            return run_forward<T, D, N, P, PC, PS>(path, sig, shape, dc.fwd_chunks, bounds, keep, workspace,    \
                                                   stream, dc.grouped);                                           \
        break;
#define PSIG_CASE_BWD(I, D, N, P, PC, PS)                                                                          \
    case I:                                                                                                        \
        if constexpr (I % kDenseGroups == PSIG_GROUP && shape_enabled(D, N))                                       \
            return run_backward<T, D, N, P, PC, PS>(path, sig, grad_sig, grad_inc, grad_path, wrote_path, shape,   \
                                                    dc.bwd_chunks, bounds, kept, workspace, stream, dc.grouped,    \
                                                    inc_cleared);                                                  \
        break;

template <int GROUP, typename T>
hipError_t launch_dense_forward_group(const T *path, T *sig, const SigShape &shape, const DenseChoice &dc,
                                      const int *bounds, T *keep, void *workspace, hipStream_t stream) {
    switch (dc.variant) {
        PSIG_VARIANTS(PSIG_CASE_FWD)
        default: break;
    }
    return hipErrorNotSupported;
}

template <int GROUP, typename T>
hipError_t launch_dense_backward_group(const T *path, const T *sig, const T *grad_sig, T *grad_inc, T *grad_path,
                                       bool *wrote_path, const SigShape &shape, const DenseChoice &dc,
                                       const int *bounds, const T *kept, void *workspace, bool inc_cleared,
                                       hipStream_t stream) {
    switch (dc.variant) {
        PSIG_VARIANTS(PSIG_CASE_BWD)
        default: break;
    }
    return hipErrorNotSupported;
}

#define PSIG_INSTANTIATE(T)                                                                                          \
    template hipError_t launch_dense_forward_group<PSIG_GROUP, T>(const T *, T *, const SigShape &, const DenseChoice &, \
                                                                  const int *, T *, void *, hipStream_t);            \
    template hipError_t launch_dense_backward_group<PSIG_GROUP, T>(const T *, const T *, const T *, T *, T *, bool *,  \
                                                                   const SigShape &, const DenseChoice &, const int *, \
                                                                   const T *, void *, bool, hipStream_t);
PSIG_INSTANTIATE(float)
PSIG_INSTANTIATE(double)
#undef PSIG_INSTANTIATE

#endif  // PSIG_GROUP

}  // namespace psig

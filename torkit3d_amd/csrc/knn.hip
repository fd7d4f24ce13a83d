// K nearest neighbours for gfx950, returning the reference's MinK slot order.
//
// A lane owns one query and keeps its k best (distance, index) pairs in registers
// (KMAX slots, fully unrolled, no dynamic register indexing); key points are
// staged through LDS as (x,y,z,pad) quads that all lanes read as a broadcast.
// The result is not just "the k smallest": the reference returns them in the
// order its MinK structure leaves them (mink.cuh:61-89) - the first k keys fill
// slots 0..k-1, later a key that beats the current maximum (strict '<') replaces
// that maximum's slot, and the new maximum is the first slot (ascending, strict
// '>') above the inserted key. The insertion below follows that rule slot for
// slot, with selects instead of indexed writes.
//
// k above the largest register variant falls back to a kernel that keeps the
// structure in the output arrays in global memory, as the reference's generic
// variant does (knn_distance_kernel.cu:102-177).
#include <type_traits>

#include "tk3d_common.h"
#include "tk3d_debug.h"

namespace {

constexpr int KNN_BLOCK = 256;
constexpr int KNN_STAGE = 1024;

// Coordinate `a` of point `j` of an n-point cloud: [n,3] rows, or with SOA three planes
// [3,n] (the layout the reference's models keep their clouds in).
template <bool SOA, typename T>
__device__ __forceinline__ T knn_coord(const T *__restrict__ cloud, int n, int j, int a)
{
    return SOA ? cloud[(int64_t)a * n + j] : cloud[(int64_t)j * 3 + a];
}

// Inverse-squared-distance weights of the three neighbours, as FeatureInterpolator
// forms them with torch ops (torkit3d/layers/pointnet2.py:128-130):
// inv = 1 / clamp(d, min=eps); w = inv / (inv0 + inv1 + inv2).
template <typename T>
__device__ __forceinline__ void knn_three_weights(const T (&d)[3], T eps, T *__restrict__ w)
{
    T inv[3];
#pragma unroll
    for (int i = 0; i < 3; ++i)
        inv[i] = (T)1 / (d[i] < eps ? eps : d[i]);  // a NaN stays a NaN, as in clamp
    const T norm = (inv[0] + inv[1]) + inv[2];
#pragma unroll
    for (int i = 0; i < 3; ++i)
        w[i] = inv[i] / norm;
}

template <typename T, int KMAX, bool SOA, bool WEIGHTS>
__global__ __launch_bounds__(KNN_BLOCK) void knn_register_kernel(
    const T *__restrict__ query, const T *__restrict__ key, T *__restrict__ distance,
    int64_t *__restrict__ index, T *__restrict__ weight, T eps, int blocks_per_batch, int n1,
    int n2, int k)
{
    __shared__ T skey[KNN_STAGE * 4];
    const int tid = threadIdx.x;
    const int b = blockIdx.x / blocks_per_batch;
    const int qi = (blockIdx.x - b * blocks_per_batch) * KNN_BLOCK + tid;
    const bool active = qi < n1;
    const T *__restrict__ K = key + (int64_t)b * n2 * 3;
    T qx = 0, qy = 0, qz = 0;
    if (active) {
        const T *__restrict__ Q = query + (int64_t)b * n1 * 3;
        qx = knn_coord<SOA>(Q, n1, qi, 0);
        qy = knn_coord<SOA>(Q, n1, qi, 1);
        qz = knn_coord<SOA>(Q, n1, qi, 2);
    }

    T kd[KMAX];
    int ki[KMAX];
    T max_key = (T)0;
    int max_idx = 0;
    // Fill phase: keys 0..k-1 go to slots 0..k-1; the maximum is the first slot
    // holding the largest value (mink.cuh:63-72). Slots >= k stay at -inf so the
    // rescan below never selects them.
#pragma unroll
    for (int s = 0; s < KMAX; ++s) {
        kd[s] = -tk_inf<T>();
        ki[s] = 0;
        if (s < k) {  // uniform
            const T d = tk_dist2<T>(knn_coord<SOA>(K, n2, s, 0), knn_coord<SOA>(K, n2, s, 1),
                                       knn_coord<SOA>(K, n2, s, 2), qx, qy, qz);
            kd[s] = d;
            ki[s] = s;
            if (s == 0 || d > max_key) {
                max_key = d;
                max_idx = s;
            }
        }
    }

    for (int stage0 = 0; stage0 < n2; stage0 += KNN_STAGE) {
        __syncthreads();
        for (int j = tid; j < KNN_STAGE; j += KNN_BLOCK) {
            const int kj = stage0 + j;
            T x = 0, y = 0, z = 0;
            if (kj < n2) {
                x = knn_coord<SOA>(K, n2, kj, 0);
                y = knn_coord<SOA>(K, n2, kj, 1);
                z = knn_coord<SOA>(K, n2, kj, 2);
            }
            skey[j * 4 + 0] = x;
            skey[j * 4 + 1] = y;
            skey[j * 4 + 2] = z;
            skey[j * 4 + 3] = (T)0;
        }
        __syncthreads();
        const int left = n2 - stage0;
        const int cnt = left < KNN_STAGE ? left : KNN_STAGE;
        int j = (stage0 < k) ? (k - stage0 < cnt ? k - stage0 : cnt) : 0;
        for (; j < cnt; ++j) {
            const T d = tk_dist2<T>(skey[j * 4 + 0], skey[j * 4 + 1], skey[j * 4 + 2], qx, qy,
                                    qz);
            if (d < max_key) {
                const int kj = stage0 + j;
#pragma unroll
                for (int s = 0; s < KMAX; ++s) {
                    const bool here = (s == max_idx);
                    kd[s] = here ? d : kd[s];
                    ki[s] = here ? kj : ki[s];
                }
                max_key = d;
#pragma unroll
                for (int s = 0; s < KMAX; ++s) {
                    const bool up = kd[s] > max_key;
                    max_key = up ? kd[s] : max_key;
                    max_idx = up ? s : max_idx;
                }
            }
        }
    }

    if (active) {
        T *od = distance + ((int64_t)b * n1 + qi) * k;
        int64_t *oi = index + ((int64_t)b * n1 + qi) * k;
#pragma unroll
        for (int s = 0; s < KMAX; ++s) {
            if (s < k) {
                od[s] = kd[s];
                oi[s] = (int64_t)ki[s];
            }
        }
        if constexpr (WEIGHTS && KMAX >= 3) {  // k == 3
            const T d3[3] = {kd[0], kd[1], kd[2]};
            knn_three_weights<T>(d3, eps, weight + ((int64_t)b * n1 + qi) * 3);
        }
    }
}

// fp32 variant with batched insertion. Inserting into the k-slot structure costs a
// few dozen instructions and, done at the moment a candidate appears, is paid by the
// whole wave for every candidate of every lane. Here a lane first sweeps a chunk of
// 32 keys and only records which of them beat its current maximum (the sign of the
// integer difference of the bit patterns - non-negative floats order as integers -
// shifted into a mask: two instructions per key on top of the distance). The wave
// then inserts in rounds: every lane with a recorded candidate takes its next one
// (ascending key order), recomputes the distance, tests it against its maximum as
// it stands now (strict '<', as MinK does) and inserts. Rounds per chunk = the
// largest number of candidates any lane has, instead of the number of distinct
// candidate keys across all lanes. The sequence of insertions seen by one lane is
// exactly MinK's, so the slot order is unchanged.

// `skey` is KNN_STAGE * 4 floats of LDS, 16-byte aligned; the whole workgroup calls this
// with query `qi` of batch `b` per lane (qi >= n1: the lane only helps staging).
template <int KMAX, bool SOA, bool WEIGHTS>
__device__ __forceinline__ void knn_batched_body(
    const float *__restrict__ query, const float *__restrict__ key,
    float *__restrict__ distance, int64_t *__restrict__ index, float *__restrict__ weight,
    float eps, int b, int qi, int n1, int n2, int k, float *skey)
{
    constexpr int CHUNK = 32;
    static_assert(KNN_STAGE % CHUNK == 0, "a chunk must not straddle stages");
    const int tid = threadIdx.x;
    const bool active = qi < n1;
    const float *__restrict__ K = key + (int64_t)b * n2 * 3;
    float qx = 0, qy = 0, qz = 0;
    if (active) {
        const float *__restrict__ Q = query + (int64_t)b * n1 * 3;
        qx = knn_coord<SOA>(Q, n1, qi, 0);
        qy = knn_coord<SOA>(Q, n1, qi, 1);
        qz = knn_coord<SOA>(Q, n1, qi, 2);
    }

    float kd[KMAX];
    int ki[KMAX];
    float max_key = 0.0f;
    int max_idx = 0;
    bool fill_nan = false;
    // Fill phase: keys 0..k-1 go to slots 0..k-1 (mink.cuh:63-72); unused slots stay at
    // -inf so the rescan never selects them.
#pragma unroll
    for (int s = 0; s < KMAX; ++s) {
        kd[s] = -__builtin_huge_valf();
        ki[s] = 0;
        if (s < k) {  // uniform
            const float d = tk_dist2<float>(knn_coord<SOA>(K, n2, s, 0), knn_coord<SOA>(K, n2, s, 1),
                                       knn_coord<SOA>(K, n2, s, 2), qx, qy, qz);
            kd[s] = d;
            ki[s] = s;
            fill_nan |= d != d;
            if (s == 0 || d > max_key) {
                max_key = d;
                max_idx = s;
            }
        }
    }
    // The rescan below orders the slots by their bit patterns, which is the float order
    // for everything a squared distance can be except NaN. A NaN can only enter during
    // the fill (later keys must compare below the maximum); a wave that has one rescans
    // with float compares instead.
    const bool float_rescan = __builtin_amdgcn_ballot_w64(fill_nan) != 0;

    for (int stage0 = 0; stage0 < n2; stage0 += KNN_STAGE) {
        __syncthreads();
        for (int j = tid; j < KNN_STAGE; j += KNN_BLOCK) {
            const int kj = stage0 + j;
            float4 e = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (kj < n2) {
                e.x = knn_coord<SOA>(K, n2, kj, 0);
                e.y = knn_coord<SOA>(K, n2, kj, 1);
                e.z = knn_coord<SOA>(K, n2, kj, 2);
            }
            reinterpret_cast<float4 *>(skey)[j] = e;
        }
        __syncthreads();
        const int left = n2 - stage0;
        const int cnt = left < KNN_STAGE ? left : KNN_STAGE;
        for (int c0 = 0; c0 < cnt; c0 += CHUNK) {
            // ---- sweep: bit (31 - i) of `mask` <=> key c0+i is below the maximum ----
            const int maxbits = __builtin_bit_cast(int, max_key);
            const float4 *ck = reinterpret_cast<const float4 *>(skey) + c0;
            const int first = stage0 + c0;  // global index of bit 31
            unsigned mask = 0u;
            if (c0 + CHUNK <= cnt) {
                // A full chunk comes straight from global memory: the addresses are the
                // same for the whole wave, so the loads are scalar and the coordinates are
                // scalar operands of the vector arithmetic - no LDS traffic in the sweep.
#pragma unroll
                for (int i = 0; i < CHUNK; ++i) {
                    const float d = tk_dist2<float>(knn_coord<SOA>(K, n2, first + i, 0),
                                                    knn_coord<SOA>(K, n2, first + i, 1),
                                                    knn_coord<SOA>(K, n2, first + i, 2), qx, qy,
                                                    qz);
                    const unsigned diff = (unsigned)(__builtin_bit_cast(int, d) - maxbits);
                    mask = __builtin_amdgcn_alignbit(mask, diff, 31);  // (mask << 1) | sign
                }
            } else {
#pragma unroll 4
                for (int i = 0; i < CHUNK; ++i) {
                    const float4 e = ck[i];  // zero padding beyond the last key
                    const float d = tk_dist2<float>(e.x, e.y, e.z, qx, qy, qz);
                    const unsigned diff = (unsigned)(__builtin_bit_cast(int, d) - maxbits);
                    mask = __builtin_amdgcn_alignbit(mask, diff, 31);
                }
            }
            // Keys that do not exist, or that the fill phase took, are no candidates.
            int lo = k - first;                          // keys below k filled the slots
            lo = lo < 0 ? 0 : (lo > CHUNK ? CHUNK : lo);
            int hi = cnt - c0;                           // keys at or beyond hi are padding
            hi = hi > CHUNK ? CHUNK : hi;
            unsigned valid = (lo >= CHUNK) ? 0u : (0xffffffffu >> lo);
            valid &= (hi >= CHUNK) ? 0xffffffffu : ~(0xffffffffu >> hi);
            mask &= valid;

            // ---- insertion rounds; the next candidate's key is fetched from LDS while the
            // current one is inserted ----
            bool has = mask != 0u;
            int i = has ? __builtin_clz(mask) : 0;
            float4 e = ck[i];
            while (__builtin_amdgcn_ballot_w64(has)) {  // wave-uniform
                mask &= ~(0x80000000u >> i);  // no-op for a lane without a candidate
                const bool has_next = mask != 0u;
                const int i_next = has_next ? __builtin_clz(mask) : 0;
                const float4 e_next = ck[i_next];
                const float d = tk_dist2<float>(e.x, e.y, e.z, qx, qy, qz);
                if (has && d < max_key) {
                    const int kj = first + i;
#pragma unroll
                    for (int s = 0; s < KMAX; ++s) {
                        const bool here = (s == max_idx);
                        kd[s] = here ? d : kd[s];
                        ki[s] = here ? kj : ki[s];
                    }
                    if (float_rescan) {
                        max_key = d;
#pragma unroll
                        for (int s = 0; s < KMAX; ++s) {
                            const bool up = kd[s] > max_key;
                            max_key = up ? kd[s] : max_key;
                            max_idx = up ? s : max_idx;
                        }
                    } else {
                        // New maximum = largest bit pattern. MinK starts its rescan from the
                        // inserted key, so the maximum stays in the inserted slot when nothing
                        // is strictly above it; otherwise it is the first slot that holds the
                        // largest pattern: (top - 1 - bits) is negative exactly there, and
                        // the sign bits shifted together put slot 0 in the highest position.
                        // Both steps are written as short independent chains: with few waves
                        // per SIMD the round is bound by its dependent latency.
                        int t[KMAX];
#pragma unroll
                        for (int s = 0; s < KMAX; ++s)
                            t[s] = __builtin_bit_cast(int, kd[s]);
#pragma unroll
                        for (int n = KMAX; n > 1; n = (n + 2) / 3) {
#pragma unroll
                            for (int j = 0; 3 * j < n; ++j) {
                                int v = t[3 * j];
                                if (3 * j + 1 < n)
                                    v = t[3 * j + 1] > v ? t[3 * j + 1] : v;
                                if (3 * j + 2 < n)
                                    v = t[3 * j + 2] > v ? t[3 * j + 2] : v;
                                t[j] = v;
                            }
                        }
                        const int top = t[0];
                        const unsigned below = (unsigned)top - 1u;
                        constexpr int GS = KMAX <= 16 ? 4 : 8;  // slots per independent chain
                        unsigned eq[(KMAX + 31) / 32] = {};
#pragma unroll
                        for (int g0 = 0; g0 < KMAX; g0 += GS) {
                            unsigned part = 0u;
#pragma unroll
                            for (int s = g0; s < g0 + GS; ++s)
                                part = __builtin_amdgcn_alignbit(
                                    part, below - __builtin_bit_cast(unsigned, kd[s]), 31);
                            eq[g0 / 32] = (eq[g0 / 32] << GS) | part;
                        }
                        max_key = __builtin_bit_cast(float, top);
                        int first_top;
                        if constexpr (KMAX <= 32)
                            first_top = __builtin_clz(eq[0]) - (32 - KMAX);
                        else
                            first_top = eq[0] ? __builtin_clz(eq[0]) : 32 + __builtin_clz(eq[1]);
                        max_idx = top != __builtin_bit_cast(int, d) ? first_top : max_idx;
                    }
                }
                has = has_next;
                i = i_next;
                e = e_next;
            }
        }
    }

    if (active) {
        float *od = distance + ((int64_t)b * n1 + qi) * k;
        int64_t *oi = index + ((int64_t)b * n1 + qi) * k;
#pragma unroll
        for (int s = 0; s < KMAX; ++s) {
            if (s < k) {
                od[s] = kd[s];
                oi[s] = (int64_t)ki[s];
            }
        }
        if constexpr (WEIGHTS && KMAX >= 3) {  // k == 3
            const float d3[3] = {kd[0], kd[1], kd[2]};
            knn_three_weights<float>(d3, eps, weight + ((int64_t)b * n1 + qi) * 3);
        }
    }
}

template <int KMAX, bool SOA, bool WEIGHTS>
__global__ __launch_bounds__(KNN_BLOCK) void knn_batched_kernel_f32(
    const float *__restrict__ query, const float *__restrict__ key,
    float *__restrict__ distance, int64_t *__restrict__ index, float *__restrict__ weight,
    float eps, int blocks_per_batch, int n1, int n2, int k)
{
    __shared__ __align__(16) float skey[KNN_STAGE * 4];
    const int b = blockIdx.x / blocks_per_batch;
    const int qi = (blockIdx.x - b * blocks_per_batch) * KNN_BLOCK + threadIdx.x;
    knn_batched_body<KMAX, SOA, WEIGHTS>(query, key, distance, index, weight, eps, b, qi, n1, n2,
                                         k, skey);
}

// The slot number of every position of a sorted list of KMAX distances (see SORTED below).
// Up to 16 positions: a nibble each in one 64-bit word. 32 positions: the low nibbles in two
// 64-bit words and the fifth bits in a 32-bit word.
template <int KMAX> struct KnnSlotNumbers;

template <> struct KnnSlotNumbers<16> {
    unsigned long long w;
    __device__ __forceinline__ void identity() { w = 0xfedcba9876543210ull; }
    __device__ __forceinline__ unsigned head() const { return (unsigned)w & 15u; }
    __device__ __forceinline__ unsigned at(int p) const
    {
        return (unsigned)(w >> ((4 * p) & 63)) & 15u;
    }
    // positions 0..m turn by one towards the head; `slot` (the old head's) goes to position m
    __device__ __forceinline__ void turn(int m, unsigned slot)
    {
        const unsigned long long turning = ~0ull >> (60 - 4 * m);
        w = (w & ~turning) | ((w & turning) >> 4) | ((unsigned long long)slot << (4 * m));
    }
    // positions m..s move one position down (s is a compile-time constant, s > 0), `slot`
    // enters at position m
    __device__ __forceinline__ void make_room(int m, int s, unsigned slot)
    {
        const unsigned long long field = (~0ull >> (60 - 4 * s)) & (~0ull << (4 * m));
        w = (w & ~field) | (((w & field) << 4) & field) | ((unsigned long long)slot << (4 * m));
    }
    __device__ __forceinline__ void keep() { asm volatile("" : "+v"(w)); }
};

template <> struct KnnSlotNumbers<32> {
    unsigned long long w0, w1;  // low nibbles of positions 0..15 and 16..31
    unsigned fifth;             // bit p: the fifth bit of position p's slot
    __device__ __forceinline__ void identity()
    {
        w0 = w1 = 0xfedcba9876543210ull;
        fifth = 0xffff0000u;
    }
    __device__ __forceinline__ unsigned head() const
    {
        return ((unsigned)w0 & 15u) | ((fifth & 1u) << 4);
    }
    __device__ __forceinline__ unsigned at(int p) const
    {
        const unsigned long long w = p < 16 ? w0 : w1;
        return ((unsigned)(w >> ((4 * p) & 63)) & 15u) | (((fifth >> (p & 31)) & 1u) << 4);
    }
    __device__ __forceinline__ void turn(int m, unsigned slot)
    {
        const unsigned turning5 = ~0u >> (31 - m);
        fifth = (fifth & ~turning5) | ((fifth & turning5) >> 1) | ((slot >> 4) << m);
        const bool far = m >= 16;
        const unsigned long long low = slot & 15u;
        // the first word turns as far as m reaches in it and takes the second word's first
        // nibble, or the slot, at the end of that range
        const int m0 = far ? 15 : m;
        const unsigned long long t0 = ~0ull >> (60 - 4 * m0);
        const unsigned long long in0 = far ? (w1 & 15ull) : low;
        w0 = (w0 & ~t0) | ((w0 & t0) >> 4) | (in0 << (4 * m0));
        const int m1 = far ? m - 16 : 0;
        const unsigned long long t1 = far ? ~0ull >> (60 - 4 * m1) : 0ull;
        w1 = (w1 & ~t1) | ((w1 & t1) >> 4) | (far ? low << (4 * m1) : 0ull);
    }
    __device__ __forceinline__ void make_room(int m, int s, unsigned slot)
    {
        const unsigned field5 = (~0u >> (31 - s)) & (~0u << m);
        fifth = (fifth & ~field5) | (((fifth & field5) << 1) & field5) | ((slot >> 4) << m);
        const unsigned long long low = slot & 15u;
        if (s < 16) {  // (compile-time) only the first word
            const unsigned long long field = (~0ull >> (60 - 4 * s)) & (~0ull << (4 * m));
            w0 = (w0 & ~field) | (((w0 & field) << 4) & field) | (low << (4 * m));
        } else {
            const bool far = m >= 16;  // the first word stays as it is
            // second word: positions max(m, 16)..s move down; what enters at its start is
            // the first word's last nibble, or the slot itself
            const int m1 = far ? m - 16 : 0;
            const unsigned long long f1 = (~0ull >> (60 - 4 * (s - 16))) & (~0ull << (4 * m1));
            const unsigned long long in1 = far ? low : (w0 >> 60);
            w1 = (w1 & ~f1) | (((w1 & f1) << 4) & f1) | (in1 << (4 * m1));
            const unsigned long long f0 = far ? 0ull : ~0ull << (4 * m);
            w0 = (w0 & ~f0) | ((w0 & f0) << 4) | (far ? 0ull : low << (4 * m));
        }
    }
    __device__ __forceinline__ void keep()
    {
        asm volatile("" : "+v"(w0), "+v"(w1), "+v"(fifth));
    }
};

// How many of positions 1..KMAX-1 of a descending list satisfy `above` (true for a prefix of
// them), by bisection through the registers: the pivot of a level is chosen among its 2^level
// possible places by selects on the outcomes so far (KMAX - 1 - log2 KMAX selects in all).
// `last` returns the last position's value that satisfied it (`none` without one).
template <int KMAX, typename Above>
__device__ __forceinline__ int knn_sorted_position(const int (&v)[KMAX], Above above, int none,
                                                   int &last)
{
    constexpr int LEVELS = KMAX == 32 ? 5 : KMAX == 16 ? 4 : KMAX == 8 ? 3 : 2;
    static_assert((1 << LEVELS) == KMAX, "KMAX is a power of two from 4 to 32");
    bool taken[LEVELS];
    int m = 0;
    last = none;
#pragma unroll
    for (int level = 0; level < LEVELS; ++level) {
        const int step = KMAX >> (level + 1);
        int c[1 << (LEVELS - 1)];
#pragma unroll
        for (int j = 0; j < (1 << level); ++j)
            c[j] = v[(2 * j + 1) * step];
        // the outcome of the previous level is the lowest bit of the place, and so on
#pragma unroll
        for (int d = level - 1; d >= 0; --d) {
#pragma unroll
            for (int j = 0; j < (1 << d); ++j)
                c[j] = taken[d] ? c[2 * j + 1] : c[2 * j];
        }
        taken[level] = above(c[0]);
        last = taken[level] ? c[0] : last;
        m = 2 * m + (taken[level] ? 1 : 0);
    }
    return m;
}

// fp32, k <= 16, launches with many queries: pre-filtered sweep with deferred insertions.
//
// Two costs dominate the batched kernel above: its sweep spends 8 vector instructions per
// pair (six for the canonical distance), and its insertion rounds run after every chunk
// for as long as the slowest lane of the wave has candidates, most lanes idling.
//
// Sweep. As in the chamfer kernel, most pairs only need to be ruled out, which the score
//     s(q,k) = |k'|^2 - 2 q'.k'      (k' = k - c, q' = q - c, c the centre of the key
//                                      cloud's bounding box)
// does with three fused multiply-adds: d2(q,k) = s + |q'|^2 up to rounding. A key can
// only be inserted if its canonical distance is below the query's current maximum M, so
// the sweep evaluates t = s - thr, thr = (M - |q'|^2) + slack, by starting the three fmas
// from |k'|^2 - thr, and collects the sign bits of t: 5 instructions per pair. With
// u = 2^-24, rho = |k'| + |q'|, R = (max|k'| + |q'|)^2:
//     canonical d2 against the exact distance of the centred points   7.02 u rho^2
//         (three rounded differences, a product and two fmas of non-negative terms,
//          plus the rounding of k' and q' themselves)
//     |k'|^2 as staged                                                 3 u |k'|^2
//     |k'|^2 - thr and the three fmas: four roundings of partial sums
//         bounded by R + |thr|                                         4.04 u (R + |thr|)
//     thr itself: M - |q'|^2 and the added slack                      3 u (M + R)
// With |thr| <= M + R the total is below 21.2 u R + 7.1 u M; the kernel uses
// slack = 32 u R + 16 u M (+1e-37 against underflow), R from max|k'| and |q'| inflated by
// 1e-6 for their own rounding. Every key with canonical d2 < M therefore has t < 0: the
// sign bits are a superset of MinK's insertions. Queries or key clouds that are
// non-finite or huge (where the bound means nothing) take every key as a candidate, or
// the workgroup runs the exact batched sweep.
//
// Insertions. A candidate is re-evaluated with the canonical arithmetic and inserted
// under MinK's strict test against the maximum as it stands then, in ascending key
// order per query, so the slots go through exactly MinK's states. But insertion does not
// follow every chunk: a lane keeps up to CAP non-empty chunk masks per query in a small
// register queue and the wave runs a service step (every lane with a pending candidate
// takes its first one) only while some lane holds T candidates or a full queue; the
// rest waits for company. Deferring only makes M - and with it thr - a little stale,
// i.e. admits more candidates, each rejected by the strict test when it is served.
// Per 2048 keys a wave runs 68 steps at k = 3 and 145 at k = 16 instead of 142 and 253
// rounds. Keys are centred and staged in LDS as (x', y', z', |k'|^2); a lane serves QPL
// queries, so one LDS read feeds QPL pairs and the steps of its queries interleave.
//
// MATRIX. The scores of a chunk of 32 keys come from the matrix cores instead: one
// v_mfma_f32_32x32x16_f16 gives t = s - thr for 32 keys x 32 queries as a 16-term dot
// product of fp16 pieces, and a lane only has to collect the 16 sign bits it is handed
// (1.1 vector instructions per pair instead of 5). Coordinates are centred and multiplied
// by a power of two that brings the largest centred key norm into [1, 2) (exact; outside
// 2^-40 .. 2^40 the workgroup takes the exact sweep), then split into two fp16 pieces
// each, x = xh + xl + e with |e| <= 2^-23 |x| + 2^-25, |k'|^2 into two and -thr into two:
//     key   : xh xh xl  yh yh yl  1  1  | zh zh zl  n0 n1 0  1  1
//     query : Xh Xl Xh  Yh Yl Yh  T0 T1 | Zh Zl Zh  1  1  0  T0 T1        (X = -2 q'x)
// In the 32 x 32 result lane l holds rows (keys) 16 h .. 16 h + 15, h = l / 32, of column
// (query) l % 32; the keys of a tile are stored in that row order, so the sign bits of a
// lane are 16 consecutive bits of the chunk mask. The wave's 64 QPL queries are 2 QPL
// blocks of 32; lane l owns the queries of column l % 32 in blocks h, 2 + h, ..., computes
// their thr and writes -thr into the T terms of its own half only (the other half holds
// zeros there), so no thr crosses lanes; the two halves of a mask meet through one exchange
// between lanes l and l ^ 32 per chunk. The library runs it with one query per lane in
// workgroups of 512 lanes (LANES): 120 registers, four waves per SIMD, where two queries
// per lane need 238 and leave two. Error budget in the rescaled units, on top of the
// one above (products of the second pieces are left out, thr is rounded to two pieces):
//     pieces dropped from 2 q'.k', subnormal pieces                       5 u R
//     |k'|^2 and thr in two pieces                           4 u R + 4 u (M + R)
//     the matrix core's 16 additions: 32 u times the sum of the products' magnitudes
//         as the matrix core sees them (a subnormal fp16 factor counts as 2^-14; see
//         the chamfer kernel and tests/test_gpu_mfma_bound.py), which is below
//         1.02 (M + R) here because the scale makes max|k'| >= 1     33 u (M + R)
//     canonical d2, |k'|^2 as staged, thr itself             10 u R + 3 u (M + R)
// below 59 u R + 40 u M; the kernel uses slack = 64 u R + 48 u M. Queries further than 200
// from the centre (rescaled; thr would leave fp16's range) take every key as a candidate.
// KI_LDS: the key indices of the slots live in LDS (16-bit, so clouds of up to 65536 keys),
// one column per lane: they are only written during the sweep, and a write into a column of
// one's own is one instruction where the slot in registers takes a select per slot.
//
// SORTED (8 to 32 slots, key indices in LDS; described for 16): the registers hold the
// distances in descending order instead of slot order, and a 64-bit word holds the slot
// number of every position, a nibble each. MinK's maximum is then position 0, and an
// insertion is one v_med3_i32 per position (remove the head, let the new key x sink to its place: position p becomes the
// median of its old value, its lower neighbour's and x) plus a rotation of the nibbles of
// positions 0..m, m being x's new position, found by a binary search through the registers
// (4 compares, 11 selects): 86 instructions per step where the slot-ordered registers take
// 116 (a select per slot to write, a max3 tree and a sign-bit scan for the first slot that
// holds the new maximum). MinK's order among equal distances (mink.cuh:74-87: the rescan
// starts from the inserted key and moves on only to a strictly larger one, so the maximum
// is the inserted slot if nothing is strictly above it, else the lowest slot holding the
// largest distance) becomes: equal distances are kept in ascending slot order, except
// that a key with nothing strictly above it goes to the head. With R the list without its
// head, x goes to position 0 if no element of R is above it, else behind the elements of R
// that are above it or equal to it with a lower slot number. Equal distances are rare
// outside quantised clouds: the binary search counts the elements >= x and hands back the
// last of them; only when that equals x in some lane does the wave search again, for the
// elements strictly above x, and walk the run of equals between the two results comparing
// slot numbers.
template <int KMAX, int QPL, bool SOA, bool WEIGHTS, bool MATRIX, int LANES = KNN_BLOCK,
          bool KI_LDS = false, bool SORTED = false>
__global__ __launch_bounds__(LANES) void knn_filter_kernel_f32(
    const float *__restrict__ query, const float *__restrict__ key,
    float *__restrict__ distance, int64_t *__restrict__ index, float *__restrict__ weight,
    float eps, int blocks_per_batch, int n1, int n2, int k)
{
    constexpr int BLOCK = LANES;
    constexpr int NW = BLOCK / TK_WAVE;
    constexpr int STAGE = 512;
    constexpr int CHUNK = 32;
    constexpr int CAP = 4;
    constexpr int T = 6;
    constexpr int PER = STAGE / BLOCK;
    static_assert(STAGE % BLOCK == 0 && STAGE % CHUNK == 0, "stage shape");
    static_assert(!SORTED || (KI_LDS && QPL == 1 && KMAX >= 4 && KMAX <= 32 && !WEIGHTS),
                  "the sorted list is for one query of 4 to 32 slots per lane, no weights");
    static_assert(2 * STAGE * 4 * (int)sizeof(float) >= KNN_STAGE * 4 * (int)sizeof(float),
                  "the staging buffers double as the exact sweep's stage");
    // Two stage buffers of centred keys (x', y', z', |k'|^2) (+ 8 keys the read-ahead of
    // the sweep runs into), then two of raw keys (x, y, z, 0) for the service steps.
    // (MATRIX: two stage buffers of key terms, [tile][half][row] x 16 bytes, instead.)
    static_assert(!MATRIX || QPL == 1 || QPL == 2, "two or four blocks of 32 queries per wave");
    constexpr int SCORE_FLOATS = MATRIX ? 2 * STAGE * 8 : 2 * STAGE * 4 + 32;
    constexpr int STAGING_FLOATS = SCORE_FLOATS + 2 * STAGE * 4;
    // waves that transpose their results together (32 slots: two, 34 KB of LDS)
    constexpr int TWAVES = NW < 4 ? NW : KMAX > 16 ? 2 : 4;
    constexpr int TRANSPOSE_FLOATS = TWAVES * 2 * TK_WAVE * (KMAX + 1);  // see the end of the kernel
    __shared__ __align__(16) float
        skey[STAGING_FLOATS > TRANSPOSE_FLOATS ? STAGING_FLOATS : TRANSPOSE_FLOATS];
    float4 *const sraw = reinterpret_cast<float4 *>(skey + SCORE_FLOATS);
    uint4 *const sterm = reinterpret_cast<uint4 *>(skey);
    extern __shared__ __align__(16) unsigned short knn_filter_ski[];  // KI_LDS: [QPL][KMAX][LANES]
    const int half = (threadIdx.x >> 5) & 1;
    __shared__ float sred[NW][8];
    const int tid = threadIdx.x;
    const int lane = tid & (TK_WAVE - 1);
    const int wave = tid / TK_WAVE;
    const int b = blockIdx.x / blocks_per_batch;
    const int qblock = blockIdx.x - b * blocks_per_batch;
    const float *__restrict__ K = key + (int64_t)b * n2 * 3;
    const float *__restrict__ Q = query + (int64_t)b * n1 * 3;
    const float INF = __builtin_huge_valf();

    // ---- bounding box of the key cloud -> centre; largest centred norm ----
    float lo[3] = {INF, INF, INF}, hi[3] = {-INF, -INF, -INF};
    for (int j = tid; j < n2; j += BLOCK) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            const float v = knn_coord<SOA>(K, n2, j, a);
            lo[a] = __builtin_fminf(lo[a], v);
            hi[a] = __builtin_fmaxf(hi[a], v);
        }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            lo[a] = __builtin_fminf(lo[a], __shfl_xor(lo[a], o));
            hi[a] = __builtin_fmaxf(hi[a], __shfl_xor(hi[a], o));
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            sred[wave][a] = lo[a];
            sred[wave][3 + a] = hi[a];
        }
    }
    __syncthreads();
    float cc[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        float l = INF, h = -INF;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            l = __builtin_fminf(l, sred[w][a]);
            h = __builtin_fmaxf(h, sred[w][3 + a]);
        }
        cc[a] = 0.5f * l + 0.5f * h;
    }
    const float c0 = cc[0], c1 = cc[1], c2 = cc[2];
    float kmax2 = 0.0f;
    for (int j = tid; j < n2; j += BLOCK) {
        const float x = knn_coord<SOA>(K, n2, j, 0) - c0;
        const float y = knn_coord<SOA>(K, n2, j, 1) - c1;
        const float z = knn_coord<SOA>(K, n2, j, 2) - c2;
        kmax2 = __builtin_fmaxf(kmax2, __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x)));
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        kmax2 = __builtin_fmaxf(kmax2, __shfl_xor(kmax2, o));
    if (lane == 0)
        sred[wave][6] = kmax2;
    __syncthreads();
    kmax2 = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w)
        kmax2 = __builtin_fmaxf(kmax2, sred[w][6]);
    bool safe = (c0 - c0 == 0.0f) && (c1 - c1 == 0.0f) && (c2 - c2 == 0.0f) && (kmax2 < 1e30f);
    float scale = 1.0f;  // MATRIX: 2^-(exponent of the largest centred key norm)
    if constexpr (MATRIX) {
        const float ext = __builtin_sqrtf(kmax2);
        const int ebits = (int)((__builtin_bit_cast(unsigned, ext) >> 23) & 0xffu) - 127;
        safe = safe && (ext == 0.0f || (ebits >= -40 && ebits <= 40));
        scale = (!safe || ext == 0.0f) ? 1.0f
                                       : __builtin_bit_cast(float, (unsigned)(127 - ebits) << 23);
    }
    if (!safe) {  // uniform over the workgroup
#pragma unroll 1
        for (int i = 0; i < QPL; ++i)
            knn_batched_body<KMAX, SOA, WEIGHTS>(query, key, distance, index, weight, eps, b,
                                                 (qblock * QPL + i) * BLOCK + tid, n1, n2, k,
                                                 skey);
        return;
    }
    const float kmax = __builtin_sqrtf(kmax2) * scale * 1.000001f;
    const float scale2 = scale * scale;  // <= 2^80

    // ---- queries ----
    float qx[QPL], qy[QPL], qz[QPL], ax[QPL], ay[QPL], az[QPL], qn[QPL], slack_r[QPL];
    bool active[QPL], usable[QPL];
    // Slots hold the bit patterns of the distances: squared distances are non-negative, so
    // their patterns order as signed integers. A NaN can only enter during the fill (a later
    // key must compare below the maximum) and MinK never selects such a slot as maximum
    // unless it is slot 0, in which case it never inserts again: here a NaN slot holds the
    // pattern of -inf (below everything) and is recomputed when the results are written, and
    // a NaN in slot 0 freezes the query (maximum -inf: no key compares below it).
    int kd[QPL][KMAX];
    int ki[QPL][KI_LDS ? 1 : KMAX];
    auto ski = [&](int i, int slot) -> unsigned short & {
        return knn_filter_ski[(i * KMAX + slot) * LANES + threadIdx.x];
    };
    float max_key[QPL];
    int max_idx[QPL];
    unsigned nan_slots[QPL];
    KnnSlotNumbers<(KMAX > 16 ? 32 : 16)> ids[QPL];  // SORTED: the slot of every position of kd
    constexpr int NEG_INF_BITS = (int)0xff800000u;
    constexpr int INT_LOWEST = (int)0x80000000u, INT_HIGHEST = 0x7fffffff;
    // the median of three (v_med3_i32)
    auto med3 = [](int a, int b, int c) {
        const int lo = a < b ? a : b, hi = a < b ? b : a;
        const int t = hi < c ? hi : c;
        return lo > t ? lo : t;
    };
    // Pending chunk masks per query, oldest first (bit 31 = first key of the chunk), and
    // the key index of bit 31 of each. Named members and no loops over the queue, so it
    // stays in registers (an array indexed through a loop ends up in scratch memory).
    static_assert(CAP == 4, "the queue is written out for four entries");
    struct Pending {
        unsigned m0, m1, m2, m3;
        int b0, b1, b2, b3;
    } pq[QPL];
    int qlen[QPL], pending[QPL];
#pragma unroll
    for (int i = 0; i < QPL; ++i) {
        const int qi = (qblock * QPL + i) * BLOCK + tid;
        active[i] = qi < n1;
        qx[i] = active[i] ? knn_coord<SOA>(Q, n1, qi, 0) : c0;
        qy[i] = active[i] ? knn_coord<SOA>(Q, n1, qi, 1) : c1;
        qz[i] = active[i] ? knn_coord<SOA>(Q, n1, qi, 2) : c2;
        const float px = (qx[i] - c0) * scale, py = (qy[i] - c1) * scale, pz = (qz[i] - c2) * scale;
        ax[i] = -2.0f * px;
        ay[i] = -2.0f * py;
        az[i] = -2.0f * pz;
        qn[i] = __builtin_fmaf(pz, pz, __builtin_fmaf(py, py, px * px));
        const float qnorm = __builtin_sqrtf(qn[i]) * 1.000001f;
        const float r = kmax + qnorm;
        if constexpr (MATRIX) {
            slack_r[i] = r * r * 3.8146973e-06f + 1e-37f * scale2;  // 64 u R
            usable[i] = qnorm <= 200.0f;                            // false for NaN
            ax[i] = usable[i] ? ax[i] : 0.0f;
            ay[i] = usable[i] ? ay[i] : 0.0f;
            az[i] = usable[i] ? az[i] : 0.0f;
        } else {
            slack_r[i] = r * r * 1.9073486e-06f + 1e-37f;  // 32 u R
            usable[i] = slack_r[i] < 1e30f;                  // false for NaN / inf / huge
        }
        // fill: keys 0..k-1 go to slots 0..k-1 (mink.cuh:63-72); unused slots stay at -inf
        max_key[i] = 0.0f;
        max_idx[i] = 0;
        nan_slots[i] = 0u;
        bool frozen = false;
        ids[i].identity();
#pragma unroll
        for (int s = 0; s < KMAX; ++s)
            kd[i][s] = NEG_INF_BITS;
#pragma unroll
        for (int s = 0; s < KMAX; ++s) {
            if constexpr (KI_LDS)
                ski(i, s) = (unsigned short)(s < k ? s : 0);
            else
                ki[i][s] = 0;
            if constexpr (SORTED) {
                if (s < k) {  // uniform
                    const float d = tk_dist2<float>(knn_coord<SOA>(K, n2, s, 0),
                                                    knn_coord<SOA>(K, n2, s, 1),
                                                    knn_coord<SOA>(K, n2, s, 2), qx[i], qy[i], qz[i]);
                    const bool isnan = d != d;
                    const int x = isnan ? NEG_INF_BITS : __builtin_bit_cast(int, d);
                    nan_slots[i] |= isnan ? (1u << s) : 0u;
                    frozen |= isnan && s == 0;
                    // Positions 0..s-1 hold the keys so far, all of lower slot numbers: key s
                    // goes behind those that are >= it, the rest move down one position
                    // (position s held the placeholder of slot s).
                    int m = 0;
#pragma unroll
                    for (int p = 0; p < s; ++p)
                        m += kd[i][p] >= x ? 1 : 0;
#pragma unroll
                    for (int p = s; p >= 1; --p)
                        kd[i][p] = med3(kd[i][p - 1], kd[i][p], x);
                    kd[i][0] = kd[i][0] > x ? kd[i][0] : x;
                    if (s > 0)
                        ids[i].make_room(m, s, (unsigned)s);
                }
                continue;
            }
            if (s < k) {  // uniform
                const float d = tk_dist2<float>(knn_coord<SOA>(K, n2, s, 0),
                                                knn_coord<SOA>(K, n2, s, 1),
                                                knn_coord<SOA>(K, n2, s, 2), qx[i], qy[i], qz[i]);
                const bool isnan = d != d;
                kd[i][s] = isnan ? NEG_INF_BITS : __builtin_bit_cast(int, d);
                if constexpr (!KI_LDS)
                    ki[i][s] = s;
                nan_slots[i] |= isnan ? (1u << s) : 0u;
                frozen |= isnan && s == 0;
                if (s == 0 || d > max_key[i]) {
                    max_key[i] = d;
                    max_idx[i] = s;
                }
            }
        }
        if constexpr (SORTED)
            max_key[i] = __builtin_bit_cast(float, kd[i][0]);  // (-inf if every key is a NaN)
        max_key[i] = frozen ? -INF : max_key[i];
        pq[i] = Pending{0u, 0u, 0u, 0u, 0, 0, 0, 0};
        qlen[i] = 0;
        pending[i] = 0;
    }

    // MATRIX: the query side of the 16 terms for the wave's 2 QPL blocks of 32 queries.
    // Block 2 i + h' holds query i of the lanes of half h'; this lane supplies terms
    // 8 h .. 8 h + 7 of column lane % 32 in every block, from its own coordinates or, for
    // the other half's blocks, its partner's. The T terms (.w) are written per chunk.
    uint4 qterm[MATRIX ? 2 * QPL : 1];
    if constexpr (MATRIX) {
#pragma unroll
        for (int i = 0; i < QPL; ++i) {
            const float ox = __shfl_xor(ax[i], 32), oy = __shfl_xor(ay[i], 32),
                        oz = __shfl_xor(az[i], 32);
#pragma unroll
            for (int hb = 0; hb < 2; ++hb) {  // the block owned by half hb
                const bool own = half == hb;
                const float X = own ? ax[i] : ox, Y = own ? ay[i] : oy, Z = own ? az[i] : oz;
                const unsigned sx = tk_f16_split2(X), sy = tk_f16_split2(Y), sz = tk_f16_split2(Z);
                const unsigned xh = sx & 0xffffu, yh = sy & 0xffffu, zh = sz & 0xffffu;
                qterm[2 * i + hb] =
                    half == 0 ? make_uint4(sx, xh | (yh << 16), (sy >> 16) | (yh << 16), 0u)
                              : make_uint4(sz, zh | 0x3c000000u, 0x00003c00u, 0u);
            }
        }
    }

    // One service step: every query with a pending candidate takes its first one. Written
    // without branches so that the chains of a lane's queries interleave.
    auto service = [&]() {
        float4 raw[QPL];
        int kj[QPL];
        bool has[QPL];
#pragma unroll
        for (int i = 0; i < QPL; ++i) {
            Pending &p = pq[i];
            has[i] = qlen[i] > 0;
            // (an empty queue has m0 == 0: the bit number is then meaningless, the address
            // below stays inside the buffer and nothing is inserted)
            const int bit = __builtin_clz(p.m0 | 1u);
            kj[i] = p.b0 + bit;
            // resident: candidates are never older than the previous stage (see below)
            raw[i] = sraw[kj[i] & (2 * STAGE - 1)];
            const unsigned rest = p.m0 & ~(0x80000000u >> bit);
            const bool shift = has[i] && rest == 0u;
            p.m0 = shift ? p.m1 : rest;
            p.b0 = shift ? p.b1 : p.b0;
            p.m1 = shift ? p.m2 : p.m1;
            p.b1 = shift ? p.b2 : p.b1;
            p.m2 = shift ? p.m3 : p.m2;
            p.b2 = shift ? p.b3 : p.b2;
            p.m3 = shift ? 0u : p.m3;
            qlen[i] -= shift ? 1 : 0;
            pending[i] -= has[i] ? 1 : 0;
        }
#pragma unroll
        for (int i = 0; i < QPL; ++i) {
            const float d = tk_dist2<float>(raw[i].x, raw[i].y, raw[i].z, qx[i], qy[i], qz[i]);
            const bool ins = has[i] && d < max_key[i];  // MinK's strict test (mink.cuh:74)
            const int dbits = __builtin_bit_cast(int, d);
            if constexpr (SORTED) {
                int(&v)[KMAX] = kd[i];
                // a key that is not inserted sinks nowhere: above every pattern
                const int x = ins ? dbits : INT_HIGHEST;
                // m: how many of positions 1..KMAX-1 are >= x; last: the last of them
                int last;
                int m = knn_sorted_position<KMAX>(v, [&](int pivot) { return pivot >= x; },
                                                  INT_LOWEST, last);
                const unsigned slot = ids[i].head();  // of the maximum: x takes it
                if (__builtin_amdgcn_ballot_w64(last == x) != 0) {  // uniform: equal distances
                    // the same search for the positions strictly above x ...
                    int unused;
                    const int above = knn_sorted_position<KMAX>(
                        v, [&](int pivot) { return pivot > x; }, INT_LOWEST, unused);
                    // ... and positions above + 1 .. m hold x, in ascending slot order: x goes
                    // behind those of lower slots
                    const int equal = m - above;
                    int before = 0;
                    for (int q = 0; __builtin_amdgcn_ballot_w64(q < equal) != 0; ++q) {
                        const unsigned other = ids[i].at((above + 1 + q) & (KMAX - 1));
                        before += (q < equal && other < slot) ? 1 : 0;
                    }
                    m = above == 0 ? 0 : above + before;
                }
#pragma unroll
                for (int p = 0; p < KMAX; ++p)
                    v[p] = med3(v[p], p + 1 < KMAX ? v[p + 1] : INT_LOWEST, x);
                ids[i].turn(m, slot);  // the head's slot goes with x to position m
                if (ins)
                    ski(i, slot) = (unsigned short)kj[i];
                max_key[i] = ins ? __builtin_bit_cast(float, v[0]) : max_key[i];
                continue;
            }
            // the key takes the slot of the maximum ...
#pragma unroll
            for (int s = 0; s < KMAX; ++s) {
                const bool here = ins && s == max_idx[i];
                kd[i][s] = here ? dbits : kd[i][s];
                if constexpr (!KI_LDS)
                    ki[i][s] = here ? kj[i] : ki[i][s];
            }
            if constexpr (KI_LDS) {
                if (ins)
                    ski(i, max_idx[i]) = (unsigned short)kj[i];
            }
            // ... and the new maximum is the largest pattern: it stays in the written slot
            // when nothing is strictly above the new key, otherwise it is the first slot
            // holding the largest pattern ((top - 1 - bits) is negative exactly there; the
            // sign bits shifted together put slot 0 in the highest position).
            int t[KMAX];
#pragma unroll
            for (int s = 0; s < KMAX; ++s)
                t[s] = kd[i][s];
#pragma unroll
            for (int n = KMAX; n > 1; n = (n + 2) / 3) {
#pragma unroll
                for (int j = 0; 3 * j < n; ++j) {
                    int v = t[3 * j];
                    if (3 * j + 1 < n)
                        v = t[3 * j + 1] > v ? t[3 * j + 1] : v;
                    if (3 * j + 2 < n)
                        v = t[3 * j + 2] > v ? t[3 * j + 2] : v;
                    t[j] = v;
                }
            }
            const int top = t[0];
            const unsigned below = (unsigned)top - 1u;
            constexpr int GS = 4;
            unsigned eq = 0u;
#pragma unroll
            for (int g0 = 0; g0 < KMAX; g0 += GS) {
                unsigned part = 0u;
#pragma unroll
                for (int s = g0; s < g0 + GS; ++s)
                    part = __builtin_amdgcn_alignbit(part, below - (unsigned)kd[i][s], 31);
                eq = (eq << GS) | part;
            }
            // (eq | 1 keeps the count defined; eq is never 0 when it matters)
            const int first_top = __builtin_clz(eq | 1u) - (32 - KMAX);
            const int new_idx = top != dbits ? first_top : max_idx[i];
            max_key[i] = ins ? __builtin_bit_cast(float, top) : max_key[i];
            max_idx[i] = ins ? new_idx : max_idx[i];
        }
        // Keep the loop-carried state where it is: without this the register allocator
        // rotates some forty values through copies on every step.
#pragma unroll
        for (int i = 0; i < QPL; ++i) {
            asm volatile("" : "+v"(pq[i].m0), "+v"(pq[i].m1), "+v"(pq[i].m2), "+v"(pq[i].m3));
            asm volatile("" : "+v"(pq[i].b0), "+v"(pq[i].b1), "+v"(pq[i].b2), "+v"(pq[i].b3));
            asm volatile("" : "+v"(qlen[i]), "+v"(pending[i]), "+v"(max_key[i]), "+v"(max_idx[i]));
            if constexpr (SORTED)
                ids[i].keep();
#pragma unroll
            for (int s = 0; s < KMAX; ++s) {
                asm volatile("" : "+v"(kd[i][s]));
                if constexpr (!KI_LDS)
                    asm volatile("" : "+v"(ki[i][s]));
            }
        }
    };
    auto must_serve = [&]() {
        bool need = false;
#pragma unroll
        for (int i = 0; i < QPL; ++i)
            need |= pending[i] >= T || qlen[i] >= CAP;
        return __builtin_amdgcn_ballot_w64(need) != 0;
    };

    // ---- sweep: keys centred and staged in two LDS buffers, one barrier per stage ----
    const int nstages = (n2 + STAGE - 1) / STAGE;
    float4 pre[PER], pre_raw[PER];
    auto fetch = [&](int st) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int kj = st * STAGE + r * BLOCK + tid;
            float4 e = make_float4(0.0f, 0.0f, 0.0f, INF);  // past the end: never a candidate
            float4 w = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (kj < n2) {
                w.x = knn_coord<SOA>(K, n2, kj, 0);
                w.y = knn_coord<SOA>(K, n2, kj, 1);
                w.z = knn_coord<SOA>(K, n2, kj, 2);
                e.x = w.x - c0;
                e.y = w.y - c1;
                e.z = w.z - c2;
                e.w = __builtin_fmaf(e.z, e.z, __builtin_fmaf(e.y, e.y, e.x * e.x));
            }
            pre[r] = e;
            pre_raw[r] = w;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int j = r * BLOCK + tid;  // key within the stage
            if constexpr (MATRIX) {
                const float4 e = pre[r];
                const float x = e.x * scale, y = e.y * scale, z = e.z * scale;
                const float n = e.w * scale2;  // (+inf past the end)
                const unsigned sx = tk_f16_split2(x), sy = tk_f16_split2(y), sz = tk_f16_split2(z);
                const unsigned xh = sx & 0xffffu, yh = sy & 0xffffu, zh = sz & 0xffffu;
                const unsigned sn = tk_f16_split2(n);
                const bool exists = e.w < INF || e.w != e.w;
                const unsigned n0 = exists ? (sn & 0xffffu) : 0x7c00u, n1 = exists ? (sn >> 16) : 0u;
                // row of the tile: lane half h of the result holds rows 8 a + 4 h + c
                const int row = ((j & 12) << 1) | ((j & 16) >> 2) | (j & 3);
                uint4 *t = sterm + buf * (STAGE * 2) + (j >> 5) * 64 + row;
                t[0] = make_uint4(xh * 0x10001u, (sx >> 16) | (yh << 16), yh | (sy & 0xffff0000u),
                                  0x3c003c00u);
                t[32] = make_uint4(zh * 0x10001u, (sz >> 16) | (n0 << 16), n1, 0x3c003c00u);
            } else {
                reinterpret_cast<float4 *>(skey)[buf * STAGE + j] = pre[r];
            }
            sraw[buf * STAGE + j] = pre_raw[r];
        }
    };
    __syncthreads();
    fetch(0);
    stash(0);
    __syncthreads();
    for (int st = 0; st < nstages; ++st) {
        const int stage0 = st * STAGE;
        if (st + 1 < nstages)
            fetch(st + 1);
        const float4 *sbuf = reinterpret_cast<const float4 *>(skey) + (st & 1) * STAGE;
        const int left = n2 - stage0;
        const int cnt = left < STAGE ? left : STAGE;
        for (int c0k = 0; c0k < cnt; c0k += CHUNK) {
            const int first = stage0 + c0k;  // key index of bit 31
            float thr[QPL];
            unsigned mask[QPL];
#pragma unroll
            for (int i = 0; i < QPL; ++i) {
                if constexpr (MATRIX) {  // rescaled units; slack 64 u R + 48 u M
                    const float m = max_key[i] * scale2;
                    thr[i] = (m - qn[i]) + __builtin_fmaf(m, 2.8610229e-06f, slack_r[i]);
                } else {
                    thr[i] = (max_key[i] - qn[i]) +
                             __builtin_fmaf(max_key[i], 9.5367432e-07f, slack_r[i]);
                }
                mask[i] = 0u;
            }
            if constexpr (MATRIX) {
                const tk_f16x8 ka = __builtin_bit_cast(
                    tk_f16x8, sterm[(st & 1) * (STAGE * 2) + (c0k >> 5) * 64 + lane]);
#pragma unroll
                for (int i = 0; i < QPL; ++i) {
                    const unsigned tp = tk_f16_split2(-thr[i]);
                    qterm[2 * i].w = half == 0 ? tp : 0u;
                    qterm[2 * i + 1].w = half == 1 ? tp : 0u;
                }
                const tk_f32x16 zero = {};
                unsigned m16[2 * QPL];
#pragma unroll
                for (int g = 0; g < 2 * QPL; ++g) {
                    const tk_f32x16 acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        ka, __builtin_bit_cast(tk_f16x8, qterm[g]), zero, 0, 0, 0);
                    unsigned m = 0u;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float t = acc[r];  // (a bit_cast applied to acc[r] itself reads element 0)
                        m = __builtin_amdgcn_alignbit(m, __builtin_bit_cast(unsigned, t), 31);
                    }
                    m16[g] = m;
                }
                // rows of this half: keys 16 h .. 16 h + 15 of the chunk, first key in the
                // highest bit; the other half's rows of this lane's blocks come from lane ^ 32
                if constexpr (QPL == 2) {
                    const unsigned send =
                        half == 0 ? (m16[1] | (m16[3] << 16)) : (m16[0] | (m16[2] << 16));
                    const unsigned recv = __shfl_xor(send, 32);
                    const unsigned own0 = half == 0 ? m16[0] : m16[1],
                                   own1 = half == 0 ? m16[2] : m16[3];
                    const unsigned oth0 = recv & 0xffffu, oth1 = recv >> 16;
                    mask[0] = half == 0 ? ((own0 << 16) | oth0) : ((oth0 << 16) | own0);
                    mask[1] = half == 0 ? ((own1 << 16) | oth1) : ((oth1 << 16) | own1);
                } else {
                    const unsigned recv = __shfl_xor(half == 0 ? m16[1] : m16[0], 32);
                    const unsigned own = half == 0 ? m16[0] : m16[1];
                    mask[0] = half == 0 ? ((own << 16) | recv) : ((recv << 16) | own);
                }
            } else {
            const float4 *ck = sbuf + c0k;
            // Groups of G keys: the next group is read from LDS before the current one is
            // used, and the G scores of a query are independent chains.
            constexpr int G = 4;
            float4 cur[G];
#pragma unroll
            for (int g = 0; g < G; ++g)
                cur[g] = ck[g];
#pragma unroll
            for (int j = 0; j < CHUNK; j += G) {
                float4 nxt[G];
#pragma unroll
                for (int g = 0; g < G; ++g)
                    nxt[g] = ck[j + G + g];  // runs into the next chunk / the pad at the end
#pragma unroll
                for (int i = 0; i < QPL; ++i) {
                    float t[G];
#pragma unroll
                    for (int g = 0; g < G; ++g)
                        t[g] = cur[g].w - thr[i];
#pragma unroll
                    for (int g = 0; g < G; ++g)
                        t[g] = __builtin_fmaf(cur[g].z, az[i], t[g]);
#pragma unroll
                    for (int g = 0; g < G; ++g)
                        t[g] = __builtin_fmaf(cur[g].y, ay[i], t[g]);
#pragma unroll
                    for (int g = 0; g < G; ++g)
                        t[g] = __builtin_fmaf(cur[g].x, ax[i], t[g]);
#pragma unroll
                    for (int g = 0; g < G; ++g)
                        mask[i] = __builtin_amdgcn_alignbit(mask[i],
                                                            __builtin_bit_cast(unsigned, t[g]), 31);
                }
#pragma unroll
                for (int g = 0; g < G; ++g)
                    cur[g] = nxt[g];
            }
            }
            // Keys that do not exist, or that the fill phase took, are no candidates.
            int vlo = k - first;
            vlo = vlo < 0 ? 0 : (vlo > CHUNK ? CHUNK : vlo);
            int vhi = cnt - c0k;
            vhi = vhi > CHUNK ? CHUNK : vhi;
            unsigned valid = (vlo >= CHUNK) ? 0u : (0xffffffffu >> vlo);
            valid &= (vhi >= CHUNK) ? 0xffffffffu : ~(0xffffffffu >> vhi);
#pragma unroll
            for (int i = 0; i < QPL; ++i) {
                unsigned m = usable[i] ? mask[i] : 0xffffffffu;
                m = active[i] ? (m & valid) : 0u;
                const bool nz = m != 0u;
                Pending &p = pq[i];
                const int at = nz ? qlen[i] : -1;
                p.m0 = at == 0 ? m : p.m0;
                p.b0 = at == 0 ? first : p.b0;
                p.m1 = at == 1 ? m : p.m1;
                p.b1 = at == 1 ? first : p.b1;
                p.m2 = at == 2 ? m : p.m2;
                p.b2 = at == 2 ? first : p.b2;
                p.m3 = at == 3 ? m : p.m3;
                p.b3 = at == 3 ? first : p.b3;
                qlen[i] += nz ? 1 : 0;
                pending[i] += __builtin_popcount(m);
            }
            // (two steps per trip: the loop-carried state is copied between registers once
            // per trip, some forty moves)
            while (must_serve()) {
                service();
                if (!must_serve())
                    break;
                service();
            }
        }
        if (st + 1 < nstages) {
            // The next stage replaces the previous one in LDS: whatever is still pending
            // from it is served first (the queue is in key order, so its head tells).
            for (;;) {
                bool old = false;
#pragma unroll
                for (int i = 0; i < QPL; ++i)
                    old |= qlen[i] > 0 && pq[i].b0 < stage0;
                if (!__builtin_amdgcn_ballot_w64(old))
                    break;
                service();
            }
            __syncthreads();  // every wave is done with the previous stage
            stash((st + 1) & 1);
        }
        __syncthreads();
    }
    for (;;) {
        bool any = false;
#pragma unroll
        for (int i = 0; i < QPL; ++i)
            any |= qlen[i] > 0;
        if (!__builtin_amdgcn_ballot_w64(any))
            break;
        service();
    }

    // ---- results: a wave's 64 queries own 64 * k consecutive output elements; the slots
    // are transposed through LDS (row stride KMAX + 1: no bank conflicts) so that the
    // stores are runs of consecutive elements instead of one element per k ----
    __syncthreads();
    constexpr int ROW = KMAX + 1;
    float *const tbuf = skey + (wave % TWAVES) * (2 * TK_WAVE * ROW);  // values, then indices
    int *const ibuf = reinterpret_cast<int *>(tbuf + TK_WAVE * ROW);
    static_assert(TWAVES * 2 * TK_WAVE * ROW == TRANSPOSE_FLOATS, "LDS for the transpose");
    auto emit = [&]() {
#pragma unroll
    for (int i = 0; i < QPL; ++i) {
        const int q0 = (qblock * QPL + i) * BLOCK + wave * TK_WAVE;  // first query of the wave
        if constexpr (SORTED) {
#pragma unroll
            for (int p = 0; p < KMAX; ++p) {
                const int slot = (int)ids[i].at(p);
                tbuf[lane * ROW + slot] = __builtin_bit_cast(float, kd[i][p]);
                ibuf[lane * ROW + p] = (int)ski(i, p);
            }
            if (nan_slots[i] != 0u) {  // NaNs of the fill, still in their slots
#pragma unroll
                for (int s = 0; s < KMAX; ++s) {
                    if (s < k && ((nan_slots[i] >> s) & 1u))
                        tbuf[lane * ROW + s] = tk_dist2<float>(
                            knn_coord<SOA>(K, n2, s, 0), knn_coord<SOA>(K, n2, s, 1),
                            knn_coord<SOA>(K, n2, s, 2), qx[i], qy[i], qz[i]);
                }
            }
        }
#pragma unroll
        for (int s = 0; s < (SORTED ? 0 : KMAX); ++s) {
            float d = __builtin_bit_cast(float, kd[i][s]);
            if (s < k && ((nan_slots[i] >> s) & 1u))  // a NaN of the fill, still in its slot
                d = tk_dist2<float>(knn_coord<SOA>(K, n2, s, 0), knn_coord<SOA>(K, n2, s, 1),
                                    knn_coord<SOA>(K, n2, s, 2), qx[i], qy[i], qz[i]);
            kd[i][s] = __builtin_bit_cast(int, d);
            tbuf[lane * ROW + s] = d;
            if constexpr (KI_LDS)
                ibuf[lane * ROW + s] = (int)ski(i, s);
            else
                ibuf[lane * ROW + s] = ki[i][s];
        }
        const int nvalid = n1 - q0 < TK_WAVE ? n1 - q0 : TK_WAVE;  // may be <= 0
        const int total = nvalid * k;
        float *od = distance + ((int64_t)b * n1 + q0) * k;
        int64_t *oi = index + ((int64_t)b * n1 + q0) * k;
#pragma unroll
        for (int r = 0; r < KMAX; ++r) {
            const int e = r * TK_WAVE + lane;
            if (e < total) {
                const int row = e / k;
                const int col = e - row * k;
                od[e] = tbuf[row * ROW + col];
                oi[e] = (int64_t)ibuf[row * ROW + col];
            }
        }
        if constexpr (WEIGHTS && KMAX >= 3) {  // k == 3
            if (active[i]) {
                const float d3[3] = {__builtin_bit_cast(float, kd[i][0]),
                                     __builtin_bit_cast(float, kd[i][1]),
                                     __builtin_bit_cast(float, kd[i][2])};
                knn_three_weights<float>(d3, eps, weight + ((int64_t)b * n1 + q0 + lane) * 3);
            }
        }
    }
    };
    if constexpr (NW == TWAVES) {
        emit();
    } else {
#pragma unroll 1
        for (int pass = 0; pass < NW / TWAVES; ++pass) {
            if (pass > 0)
                __syncthreads();  // the waves of the previous pass are done with the buffers
            if (wave / TWAVES == pass)
                emit();
        }
    }
}

// fp32 variant with the slots in LDS as a per-lane tournament tree.
//
// With the slots in registers every insertion pays O(k) selects and compares, because
// registers cannot be indexed per lane. LDS can: a lane keeps, in columns of its own
// (row r of an array at [r * 64 + lane], conflict-free whatever r each lane uses),
//   leaf[s]  distance in slot s           kidx[s]  key index in slot s
//   ival[n]  largest distance below node n of a binary tree over the slots (heap
//            numbering, node 1 the root, the leaf of slot s at KMAX + s)
//   iarg[n]  the first slot that holds ival[n]
// ival / iarg exist for nodes 1 .. KMAX/2-1 only: a parent of two leaves is worked out
// from its leaves when needed, which saves a quarter of the LDS (the LDS footprint
// decides how many waves a CU holds). An insertion overwrites the leaf of the current
// maximum and replays the log2(KMAX) matches on the way to the root. The other side of
// each of those matches is known up front, so all of them are fetched at once and the
// path costs one LDS round trip plus three vector instructions per level. A right child
// wins a match only when strictly greater, so a node reports the first slot holding its
// maximum - MinK's rescan order (mink.cuh:74-87); MinK starts that rescan from the
// inserted key, hence the maximum stays in the inserted slot when the root is not
// strictly above it.
//
// The sweep takes its keys through scalar loads (the address is the same for every
// lane) and the rounds fetch their candidates straight from global memory, one round
// ahead; a block is one wave and never synchronises. IDX16 stores key indices in 16
// bits (clouds up to 65536 keys).
//
// NaN distances can only enter during the fill (a later key must compare below the
// maximum). MinK never selects such a slot as maximum unless it is slot 0, in which
// case it never inserts again. Here a NaN in slot 0 freezes the lane; a NaN elsewhere
// plays the tournament as -inf and is recomputed when the results are written.
template <int KMAX, bool IDX16, typename T = float> struct KnnTreeLayout {
    static constexpr int NT = 64;
    using Idx = typename std::conditional<IDX16, unsigned short, int>::type;
    static constexpr int LEAF_BYTES = (int)sizeof(T) * KMAX * NT;
    static constexpr int KIDX_BYTES = (int)sizeof(Idx) * KMAX * NT;
    static constexpr int IVAL_BYTES = (int)sizeof(T) * (KMAX / 2) * NT;
    static constexpr int IARG_BYTES = (KMAX / 2) * NT;
    static constexpr int BYTES = LEAF_BYTES + KIDX_BYTES + IVAL_BYTES + IARG_BYTES;
};

template <typename T, int KMAX, bool IDX16, bool SOA = false>
__global__ __launch_bounds__(64) void knn_tree_kernel(
    const T *__restrict__ query, const T *__restrict__ key,
    T *__restrict__ distance, int64_t *__restrict__ index, int blocks_per_batch, int n1,
    int n2, int k)
{
    using Lay = KnnTreeLayout<KMAX, IDX16, T>;
    using Idx = typename Lay::Idx;
    constexpr int CHUNK = 32;
    constexpr int NT = 64;
    constexpr int HALF = KMAX / 2;  // nodes HALF .. KMAX-1 are the parents of the leaves
    constexpr int LEVELS = KMAX == 8 ? 3 : KMAX == 16 ? 4 : KMAX == 32 ? 5 : KMAX == 64 ? 6
                           : KMAX == 128 ? 7 : 8;
    static_assert((1 << LEVELS) == KMAX, "KMAX must be a power of two from 8 to 256");
    static_assert(KMAX <= 256, "slot numbers are kept in one byte");
    extern __shared__ __align__(16) unsigned char knn_tree_lds[];
    const int lane = threadIdx.x;
    T *const leaf = reinterpret_cast<T *>(knn_tree_lds) + lane;
    Idx *const kidx = reinterpret_cast<Idx *>(knn_tree_lds + Lay::LEAF_BYTES) + lane;
    T *const ival =
        reinterpret_cast<T *>(knn_tree_lds + Lay::LEAF_BYTES + Lay::KIDX_BYTES) + lane;
    unsigned char *const iarg =
        knn_tree_lds + Lay::LEAF_BYTES + Lay::KIDX_BYTES + Lay::IVAL_BYTES + lane;

    const int b = blockIdx.x / blocks_per_batch;
    const int qi = (blockIdx.x - b * blocks_per_batch) * NT + lane;
    const bool active = qi < n1;
    const T *__restrict__ K = key + (int64_t)b * n2 * 3;
    T qx = 0, qy = 0, qz = 0;
    if (active) {
        const T *__restrict__ Q = query + (int64_t)b * n1 * 3;
        qx = knn_coord<SOA>(Q, n1, qi, 0);
        qy = knn_coord<SOA>(Q, n1, qi, 1);
        qz = knn_coord<SOA>(Q, n1, qi, 2);
    }

    // Value and first slot of a node whose children are leaves.
    auto leaf_parent = [&](int n, T &v, int &a) {
        const int s = 2 * n - KMAX;
        const T lv = leaf[s * NT], rv = leaf[(s + 1) * NT];
        const bool right = rv > lv;
        v = right ? rv : lv;
        a = right ? s + 1 : s;
    };

    // Fill phase: keys 0..k-1 go to slots 0..k-1 (mink.cuh:63-72); unused slots hold -inf.
    bool frozen = false;
    for (int s = 0; s < KMAX; ++s) {
        T d = -tk_inf<T>();
        if (s < k) {
            d = tk_dist2<T>(knn_coord<SOA>(K, n2, s, 0), knn_coord<SOA>(K, n2, s, 1),
                                knn_coord<SOA>(K, n2, s, 2), qx, qy, qz);
            if (d != d) {
                frozen |= s == 0;
                d = -tk_inf<T>();  // marks the slot: no real distance is -inf
            }
        }
        leaf[s * NT] = d;
        kidx[s * NT] = (Idx)s;
    }
    for (int n = HALF - 1; n >= 1; --n) {
        T lv, rv;
        int la, ra;
        if (2 * n >= HALF) {
            leaf_parent(2 * n, lv, la);
            leaf_parent(2 * n + 1, rv, ra);
        } else {
            lv = ival[2 * n * NT];
            rv = ival[(2 * n + 1) * NT];
            la = iarg[2 * n * NT];
            ra = iarg[(2 * n + 1) * NT];
        }
        const bool right = rv > lv;
        ival[n * NT] = right ? rv : lv;
        iarg[n * NT] = (unsigned char)(right ? ra : la);
    }
    T max_key = frozen ? -tk_inf<T>() : ival[NT];
    int max_idx = iarg[NT];

    for (int first = 0; first < n2; first += CHUNK) {  // `first` = key index of bit 31
        // ---- sweep: bit (31 - i) of `mask` <=> key first+i is below the maximum ----
        // (fp32: squared distances are non-negative, their bit patterns order as integers
        // and the sign of the difference is shifted in with one instruction)
        auto below_max = [&](unsigned m, T d) {
            if constexpr (sizeof(T) == 4) {
                const unsigned diff = (unsigned)(__builtin_bit_cast(int, d) -
                                                 __builtin_bit_cast(int, max_key));
                return __builtin_amdgcn_alignbit(m, diff, 31);  // (m << 1) | sign
            } else {
                return (m << 1) | (d < max_key ? 1u : 0u);
            }
        };
        unsigned mask = 0u;
        if (first + CHUNK <= n2) {
#pragma unroll
            for (int i = 0; i < CHUNK; ++i) {  // (wave-uniform addresses: scalar loads)
                const T d = tk_dist2<T>(knn_coord<SOA>(K, n2, first + i, 0),
                                        knn_coord<SOA>(K, n2, first + i, 1),
                                        knn_coord<SOA>(K, n2, first + i, 2), qx, qy, qz);
                mask = below_max(mask, d);
            }
        } else {
            for (int i = 0; i < CHUNK; ++i) {
                const int j = first + i < n2 ? first + i : n2 - 1;  // clamped, masked below
                const T d = tk_dist2<T>(knn_coord<SOA>(K, n2, j, 0), knn_coord<SOA>(K, n2, j, 1),
                                        knn_coord<SOA>(K, n2, j, 2), qx, qy, qz);
                mask = below_max(mask, d);
            }
        }
        // Keys that do not exist, or that the fill phase took, are no candidates.
        int lo = k - first;                          // keys below k filled the slots
        lo = lo < 0 ? 0 : (lo > CHUNK ? CHUNK : lo);
        int hi = n2 - first;                         // keys at or beyond hi do not exist
        hi = hi > CHUNK ? CHUNK : hi;
        unsigned valid = (lo >= CHUNK) ? 0u : (0xffffffffu >> lo);
        valid &= (hi >= CHUNK) ? 0xffffffffu : ~(0xffffffffu >> hi);
        mask &= valid;

        // ---- insertion rounds, the next candidate's key in flight during the current ----
        bool has = mask != 0u;
        int i = has ? __builtin_clz(mask) : 0;
        T ex = knn_coord<SOA>(K, n2, first + i, 0), ey = knn_coord<SOA>(K, n2, first + i, 1),
          ez = knn_coord<SOA>(K, n2, first + i, 2);
        while (__builtin_amdgcn_ballot_w64(has)) {  // wave-uniform
            mask &= ~(0x80000000u >> i);  // no-op for a lane without a candidate
            const bool has_next = mask != 0u;
            const int i_next = has_next ? __builtin_clz(mask) : 0;
            const T nx = knn_coord<SOA>(K, n2, first + i_next, 0),
                    ny = knn_coord<SOA>(K, n2, first + i_next, 1),
                    nz = knn_coord<SOA>(K, n2, first + i_next, 2);
            const T d = tk_dist2<T>(ex, ey, ez, qx, qy, qz);
            if (has && d < max_key) {
                const int p = max_idx;
                leaf[p * NT] = d;
                kidx[p * NT] = (Idx)(first + i);
                // the other side of every match on the path, fetched together
                T sv[LEVELS];
                int sa[LEVELS];
                sv[0] = leaf[(p ^ 1) * NT];
                sa[0] = p ^ 1;
                leaf_parent(((KMAX + p) >> 1) ^ 1, sv[1], sa[1]);
#pragma unroll
                for (int l = 2; l < LEVELS; ++l) {
                    const int sib = ((KMAX + p) >> l) ^ 1;
                    sv[l] = ival[sib * NT];
                    sa[l] = iarg[sib * NT];
                }
                T v = d;
                int a = p;
#pragma unroll
                for (int l = 0; l < LEVELS; ++l) {
                    const int node = (KMAX + p) >> l;
                    // the other side wins from the right only when strictly greater
                    const bool take = (node & 1) ? !(v > sv[l]) : (sv[l] > v);
                    v = take ? sv[l] : v;
                    a = take ? sa[l] : a;
                    // parents of leaves are not stored; the root lives in max_key / max_idx
                    if (l >= 1 && l + 1 < LEVELS) {
                        ival[(node >> 1) * NT] = v;
                        iarg[(node >> 1) * NT] = (unsigned char)a;
                    }
                }
                max_key = v;
                max_idx = v != d ? a : p;
            }
            has = has_next;
            i = i_next;
            ex = nx;
            ey = ny;
            ez = nz;
        }
    }

    if (active) {
        T *od = distance + ((int64_t)b * n1 + qi) * k;
        int64_t *oi = index + ((int64_t)b * n1 + qi) * k;
        for (int s = 0; s < k; ++s) {
            T d = leaf[s * NT];
            if (d == -tk_inf<T>())  // a NaN of the fill phase, still in its slot
                d = tk_dist2<T>(knn_coord<SOA>(K, n2, s, 0), knn_coord<SOA>(K, n2, s, 1),
                                knn_coord<SOA>(K, n2, s, 2), qx, qy, qz);
            od[s] = d;
            oi[s] = (int64_t)kidx[s * NT];
        }
    }
}

// fp32, 17 <= k <= 32 on launches of a chip's worth of queries: the sweep of the pre-filtered kernel
// on the matrix cores (see knn_filter_kernel_f32, MATRIX) feeding the LDS tournament tree
// of knn_tree_kernel. A lane owns one query; a wave's 64 queries are two blocks of 32
// (block h = the lanes of half h), so a chunk of 32 keys is two matrix instructions, the
// lane collects the 16 sign bits of its rows in both blocks, keeps those of its own block
// and hands the other 16 to lane ^ 32. The mask is a superset of the keys below the
// query's maximum (slack 64 u R + 48 u M as above); every candidate is re-evaluated with
// the canonical arithmetic and inserted under MinK's strict test in ascending key order
// by the rounds of the tree kernel, so the slots go through exactly MinK's states. A key
// cloud outside the range of the fp16 pieces (or non-finite) makes the workgroup compute
// its masks with the exact distances instead, as the tree kernel does; a query outside it
// takes every key as a candidate.
template <int KMAX, bool IDX16, int NW>
__global__ __launch_bounds__(64 * NW) void knn_tree_matrix_kernel_f32(
    const float *__restrict__ query, const float *__restrict__ key,
    float *__restrict__ distance, int64_t *__restrict__ index, int blocks_per_batch, int n1,
    int n2, int k)
{
    using Lay = KnnTreeLayout<KMAX, IDX16>;
    using Idx = typename Lay::Idx;
    constexpr int CHUNK = 32;
    constexpr int NT = 64;
    constexpr int BLOCK = 64 * NW;
    constexpr int STAGE = 256;
    constexpr int PER = (STAGE + BLOCK - 1) / BLOCK;
    constexpr int HALF = KMAX / 2;
    constexpr int LEVELS = KMAX == 8 ? 3 : KMAX == 16 ? 4 : KMAX == 32 ? 5 : 6;
    static_assert((1 << LEVELS) == KMAX, "KMAX must be a power of two from 8 to 64");
    constexpr int TERM_BYTES = 2 * STAGE * 32;  // two stage buffers of key terms
    extern __shared__ __align__(16) unsigned char knn_tm_lds[];
    __shared__ float sred[NW][8];
    uint4 *const sterm = reinterpret_cast<uint4 *>(knn_tm_lds);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;
    unsigned char *const mine = knn_tm_lds + TERM_BYTES + wave * Lay::BYTES;
    float *const leaf = reinterpret_cast<float *>(mine) + lane;
    Idx *const kidx = reinterpret_cast<Idx *>(mine + Lay::LEAF_BYTES) + lane;
    float *const ival = reinterpret_cast<float *>(mine + Lay::LEAF_BYTES + Lay::KIDX_BYTES) + lane;
    unsigned char *const iarg =
        mine + Lay::LEAF_BYTES + Lay::KIDX_BYTES + Lay::IVAL_BYTES + lane;

    const int b = blockIdx.x / blocks_per_batch;
    const int qi = (blockIdx.x - b * blocks_per_batch) * BLOCK + tid;
    const bool active = qi < n1;
    const float *__restrict__ K = key + (int64_t)b * n2 * 3;
    const float INF = __builtin_huge_valf();
    float qx = 0, qy = 0, qz = 0;
    if (active) {
        const float *q = query + ((int64_t)b * n1 + qi) * 3;
        qx = q[0];
        qy = q[1];
        qz = q[2];
    }

    // ---- bounding box of the key cloud -> centre; largest centred norm -> scale ----
    float lo[3] = {INF, INF, INF}, hi[3] = {-INF, -INF, -INF};
    for (int j = tid; j < n2; j += BLOCK) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            const float v = K[(int64_t)j * 3 + a];
            lo[a] = __builtin_fminf(lo[a], v);
            hi[a] = __builtin_fmaxf(hi[a], v);
        }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            lo[a] = __builtin_fminf(lo[a], __shfl_xor(lo[a], o));
            hi[a] = __builtin_fmaxf(hi[a], __shfl_xor(hi[a], o));
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            sred[wave][a] = lo[a];
            sred[wave][3 + a] = hi[a];
        }
    }
    __syncthreads();
    float cc[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        float l = INF, h = -INF;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            l = __builtin_fminf(l, sred[w][a]);
            h = __builtin_fmaxf(h, sred[w][3 + a]);
        }
        cc[a] = 0.5f * l + 0.5f * h;
    }
    const float c0 = cc[0], c1 = cc[1], c2 = cc[2];
    float kmax2 = 0.0f;
    for (int j = tid; j < n2; j += BLOCK) {
        const float x = K[(int64_t)j * 3 + 0] - c0, y = K[(int64_t)j * 3 + 1] - c1,
                    z = K[(int64_t)j * 3 + 2] - c2;
        kmax2 = __builtin_fmaxf(kmax2, __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x)));
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        kmax2 = __builtin_fmaxf(kmax2, __shfl_xor(kmax2, o));
    if (lane == 0)
        sred[wave][6] = kmax2;
    __syncthreads();
    kmax2 = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w)
        kmax2 = __builtin_fmaxf(kmax2, sred[w][6]);
    // (a NaN or infinite key coordinate is skipped by the reductions above or makes the
    // centre non-finite; either way such keys never compare below a maximum and the exact
    // masks below handle the cloud)
    const float ext = __builtin_sqrtf(kmax2);
    const int ebits = (int)((__builtin_bit_cast(unsigned, ext) >> 23) & 0xffu) - 127;
    const bool matrix = (c0 - c0 == 0.0f) && (c1 - c1 == 0.0f) && (c2 - c2 == 0.0f) &&
                        (kmax2 < 1e30f) && (ext == 0.0f || (ebits >= -40 && ebits <= 40));  // uniform
    const float scale =
        (!matrix || ext == 0.0f) ? 1.0f : __builtin_bit_cast(float, (unsigned)(127 - ebits) << 23);
    const float scale2 = scale * scale;
    const float kmax = ext * scale * 1.000001f;

    // ---- the query in rescaled units; its terms for both blocks of the wave ----
    const float px = (qx - c0) * scale, py = (qy - c1) * scale, pz = (qz - c2) * scale;
    const float qn = __builtin_fmaf(pz, pz, __builtin_fmaf(py, py, px * px));
    const float qnorm = __builtin_sqrtf(qn) * 1.000001f;
    const bool usable = matrix && qnorm <= 200.0f;  // false for NaN
    const float rr = kmax + qnorm;
    const float slack_r = rr * rr * 3.8146973e-06f + 1e-37f * scale2;  // 64 u R
    uint4 qterm[2];
    {
        const float ax = usable ? -2.0f * px : 0.0f, ay = usable ? -2.0f * py : 0.0f,
                    az = usable ? -2.0f * pz : 0.0f;
        const float ox = __shfl_xor(ax, 32), oy = __shfl_xor(ay, 32), oz = __shfl_xor(az, 32);
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {  // block hb: the queries of the lanes of half hb
            const bool own = half == hb;
            const float X = own ? ax : ox, Y = own ? ay : oy, Z = own ? az : oz;
            const unsigned sx = tk_f16_split2(X), sy = tk_f16_split2(Y), sz = tk_f16_split2(Z);
            const unsigned xh = sx & 0xffffu, yh = sy & 0xffffu, zh = sz & 0xffffu;
            qterm[hb] = half == 0 ? make_uint4(sx, xh | (yh << 16), (sy >> 16) | (yh << 16), 0u)
                                  : make_uint4(sz, zh | 0x3c000000u, 0x00003c00u, 0u);
        }
    }

    auto leaf_parent = [&](int n, float &v, int &a) {
        const int s = 2 * n - KMAX;
        const float lv = leaf[s * NT], rv = leaf[(s + 1) * NT];
        const bool right = rv > lv;
        v = right ? rv : lv;
        a = right ? s + 1 : s;
    };

    // Fill phase: keys 0..k-1 go to slots 0..k-1 (mink.cuh:63-72); unused slots hold -inf.
    bool frozen = false;
    for (int s = 0; s < KMAX; ++s) {
        float d = -INF;
        if (s < k) {
            d = tk_dist2<float>(K[s * 3 + 0], K[s * 3 + 1], K[s * 3 + 2], qx, qy, qz);
            if (d != d) {
                frozen |= s == 0;
                d = -INF;  // marks the slot: no real distance is -inf
            }
        }
        leaf[s * NT] = d;
        kidx[s * NT] = (Idx)s;
    }
    for (int n = HALF - 1; n >= 1; --n) {
        float lv, rv;
        int la, ra;
        if (2 * n >= HALF) {
            leaf_parent(2 * n, lv, la);
            leaf_parent(2 * n + 1, rv, ra);
        } else {
            lv = ival[2 * n * NT];
            rv = ival[(2 * n + 1) * NT];
            la = iarg[2 * n * NT];
            ra = iarg[(2 * n + 1) * NT];
        }
        const bool right = rv > lv;
        ival[n * NT] = right ? rv : lv;
        iarg[n * NT] = (unsigned char)(right ? ra : la);
    }
    float max_key = frozen ? -INF : ival[NT];
    int max_idx = iarg[NT];

    // ---- key terms, staged STAGE keys at a time in two buffers ----
    const int nstages = (n2 + STAGE - 1) / STAGE;
    float pre[PER][3];
    auto fetch = [&](int st) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int j = r * BLOCK + tid;
            const int kj = st * STAGE + j;
            pre[r][0] = pre[r][1] = pre[r][2] = INF;  // past the end
            if (j < STAGE && kj < n2) {
                pre[r][0] = K[(int64_t)kj * 3 + 0];
                pre[r][1] = K[(int64_t)kj * 3 + 1];
                pre[r][2] = K[(int64_t)kj * 3 + 2];
            }
        }
    };
    auto stash = [&](int st, int buf) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int j = r * BLOCK + tid;  // key within the stage
            if (j >= STAGE)
                continue;
            const bool exists = st * STAGE + j < n2;
            const float x = exists ? (pre[r][0] - c0) * scale : 0.0f;
            const float y = exists ? (pre[r][1] - c1) * scale : 0.0f;
            const float z = exists ? (pre[r][2] - c2) * scale : 0.0f;
            const float n = __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x));
            const unsigned sx = tk_f16_split2(x), sy = tk_f16_split2(y), sz = tk_f16_split2(z);
            const unsigned xh = sx & 0xffffu, yh = sy & 0xffffu, zh = sz & 0xffffu;
            const unsigned sn = tk_f16_split2(n);
            const unsigned n0 = exists ? (sn & 0xffffu) : 0x7c00u, n1p = exists ? (sn >> 16) : 0u;
            // row of the tile: lane half h of the result holds rows 8 a + 4 h + c
            const int row = ((j & 12) << 1) | ((j & 16) >> 2) | (j & 3);
            uint4 *t = sterm + buf * (STAGE * 2) + (j >> 5) * 64 + row;
            t[0] = make_uint4(xh * 0x10001u, (sx >> 16) | (yh << 16), yh | (sy & 0xffff0000u),
                              0x3c003c00u);
            t[32] = make_uint4(zh * 0x10001u, (sz >> 16) | (n0 << 16), n1p, 0x3c003c00u);
        }
    };
    if (matrix) {  // uniform
        __syncthreads();
        fetch(0);
        stash(0, 0);
        __syncthreads();
    }
    for (int st = 0; st < nstages; ++st) {
        const int stage0 = st * STAGE;
        if (matrix && st + 1 < nstages)
            fetch(st + 1);
        const int left = n2 - stage0;
        const int cnt = left < STAGE ? left : STAGE;
        for (int c0k = 0; c0k < cnt; c0k += CHUNK) {
            const int first = stage0 + c0k;  // key index of bit 31
            unsigned mask = 0u;
            if (matrix) {
                const float m = max_key * scale2;
                const float thr = (m - qn) + __builtin_fmaf(m, 2.8610229e-06f, slack_r);
                const unsigned tp = tk_f16_split2(-thr);
                qterm[0].w = half == 0 ? tp : 0u;
                qterm[1].w = half == 1 ? tp : 0u;
                const tk_f16x8 ka = __builtin_bit_cast(
                    tk_f16x8, sterm[(st & 1) * (STAGE * 2) + (c0k >> 5) * 64 + lane]);
                const tk_f32x16 zero = {};
                unsigned m16[2];
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    const tk_f32x16 acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        ka, __builtin_bit_cast(tk_f16x8, qterm[g]), zero, 0, 0, 0);
                    unsigned mm = 0u;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float t = acc[r];
                        mm = __builtin_amdgcn_alignbit(mm, __builtin_bit_cast(unsigned, t), 31);
                    }
                    m16[g] = mm;
                }
                const unsigned own = half == 0 ? m16[0] : m16[1];
                const unsigned recv = __shfl_xor(half == 0 ? m16[1] : m16[0], 32);
                mask = half == 0 ? ((own << 16) | recv) : ((recv << 16) | own);
                mask = usable ? mask : 0xffffffffu;
            } else {
                const int maxbits = __builtin_bit_cast(int, max_key);
                for (int i = 0; i < CHUNK; ++i) {
                    const int j = first + i < n2 ? first + i : n2 - 1;  // clamped, masked below
                    const float d = tk_dist2<float>(K[(int64_t)j * 3 + 0], K[(int64_t)j * 3 + 1],
                                                    K[(int64_t)j * 3 + 2], qx, qy, qz);
                    const unsigned diff = (unsigned)(__builtin_bit_cast(int, d) - maxbits);
                    mask = __builtin_amdgcn_alignbit(mask, diff, 31);
                }
            }
            // Keys that do not exist, or that the fill phase took, are no candidates.
            int vlo = k - first;
            vlo = vlo < 0 ? 0 : (vlo > CHUNK ? CHUNK : vlo);
            int vhi = n2 - first;
            vhi = vhi > CHUNK ? CHUNK : vhi;
            unsigned valid = (vlo >= CHUNK) ? 0u : (0xffffffffu >> vlo);
            valid &= (vhi >= CHUNK) ? 0xffffffffu : ~(0xffffffffu >> vhi);
            mask = active ? (mask & valid) : 0u;

            // ---- insertion rounds, the next candidate's key in flight during the current ----
            const float *__restrict__ ck = K + (int64_t)first * 3;
            bool has = mask != 0u;
            int i = has ? __builtin_clz(mask) : 0;
            float ex = ck[3 * i + 0], ey = ck[3 * i + 1], ez = ck[3 * i + 2];
            while (__builtin_amdgcn_ballot_w64(has)) {  // wave-uniform
                mask &= ~(0x80000000u >> i);  // no-op for a lane without a candidate
                const bool has_next = mask != 0u;
                const int i_next = has_next ? __builtin_clz(mask) : 0;
                const float nx = ck[3 * i_next + 0], ny = ck[3 * i_next + 1],
                            nz = ck[3 * i_next + 2];
                const float d = tk_dist2<float>(ex, ey, ez, qx, qy, qz);
                if (has && d < max_key) {
                    const int p = max_idx;
                    leaf[p * NT] = d;
                    kidx[p * NT] = (Idx)(first + i);
                    // the other side of every match on the path, fetched together
                    float sv[LEVELS];
                    int sa[LEVELS];
                    sv[0] = leaf[(p ^ 1) * NT];
                    sa[0] = p ^ 1;
                    leaf_parent(((KMAX + p) >> 1) ^ 1, sv[1], sa[1]);
#pragma unroll
                    for (int l = 2; l < LEVELS; ++l) {
                        const int sib = ((KMAX + p) >> l) ^ 1;
                        sv[l] = ival[sib * NT];
                        sa[l] = iarg[sib * NT];
                    }
                    float v = d;
                    int a = p;
#pragma unroll
                    for (int l = 0; l < LEVELS; ++l) {
                        const int node = (KMAX + p) >> l;
                        // the other side wins from the right only when strictly greater
                        const bool take = (node & 1) ? !(v > sv[l]) : (sv[l] > v);
                        v = take ? sv[l] : v;
                        a = take ? sa[l] : a;
                        // parents of leaves are not stored; the root lives in max_key / max_idx
                        if (l >= 1 && l + 1 < LEVELS) {
                            ival[(node >> 1) * NT] = v;
                            iarg[(node >> 1) * NT] = (unsigned char)a;
                        }
                    }
                    max_key = v;
                    max_idx = v != d ? a : p;
                }
                has = has_next;
                i = i_next;
                ex = nx;
                ey = ny;
                ez = nz;
            }
        }
        if (matrix) {
            if (st + 1 < nstages) {
                __syncthreads();  // every wave is done with the buffer of the previous stage
                stash(st + 1, (st + 1) & 1);
            }
            __syncthreads();
        }
    }

    if (active) {
        float *od = distance + ((int64_t)b * n1 + qi) * k;
        int64_t *oi = index + ((int64_t)b * n1 + qi) * k;
        for (int s = 0; s < k; ++s) {
            float d = leaf[s * NT];
            if (d == -INF)  // a NaN of the fill phase, still in its slot
                d = tk_dist2<float>(K[s * 3 + 0], K[s * 3 + 1], K[s * 3 + 2], qx, qy, qz);
            od[s] = d;
            oi[s] = (int64_t)kidx[s * NT];
        }
    }
}

// The tree kernel for launches with few queries. One wave per 64 queries leaves most of
// the chip idle when B * N1 is small, and the keys cannot simply be divided among waves:
// the slot order MinK leaves behind depends on every insertion in key order. But a key
// that the k best of a *slice* of the keys would not take is not taken by the whole
// sequence either (the slice's k-th best so far is no better than the whole sequence's).
// So S waves serve the same 64 queries: wave 0 runs MinK on the first slice as usual;
// every other wave runs a MinK of its own on its slice, starting from k empty slots, and
// logs the keys it inserts (a superset of what the whole sequence would insert from that
// slice); then wave 0 replays the logs slice by slice, in key order, against its own
// structure with the usual strict test. A log that overflows makes wave 0 sweep that
// slice in full instead. The result is MinK's, slot for slot. A log entry is the key's
// position within its slice in 16 bits, so a slice has at most 65536 keys; longer clouds
// are taken in groups of S slices, wave 0 replaying each group before the next is swept.
template <int KMAX, bool IDX16, int S, int CAP> struct KnnSplitLayout {
    using Tree = KnnTreeLayout<KMAX, IDX16>;
    using Idx = typename Tree::Idx;
    using LogIdx = unsigned short;  // a logged key, counted from the start of its slice
    static constexpr int LOG_BYTES = (int)sizeof(LogIdx) * CAP * 64;
    static constexpr int LOGS_AT = S * Tree::BYTES;          // S trees, then S - 1 logs
    static constexpr int BYTES = LOGS_AT + (S - 1) * LOG_BYTES;  // (wave 0 keeps none)
};

template <int KMAX, bool IDX16, int S, int CAP>
__global__ __launch_bounds__(64 * S) void knn_tree_split_kernel_f32(
    const float *__restrict__ query, const float *__restrict__ key,
    float *__restrict__ distance, int64_t *__restrict__ index, int blocks_per_batch, int n1,
    int n2, int k, int slice_len)
{
    using Lay = KnnTreeLayout<KMAX, IDX16>;
    using Split = KnnSplitLayout<KMAX, IDX16, S, CAP>;
    using Idx = typename Lay::Idx;
    using LogIdx = typename Split::LogIdx;
    constexpr int CHUNK = 32;
    constexpr int NT = 64;
    constexpr int HALF = KMAX / 2;
    constexpr int LEVELS = KMAX == 8 ? 3 : KMAX == 16 ? 4 : KMAX == 32 ? 5 : KMAX == 64 ? 6
                           : KMAX == 128 ? 7 : 8;
    static_assert((1 << LEVELS) == KMAX, "KMAX must be a power of two from 8 to 256");
    extern __shared__ __align__(16) unsigned char knn_split_lds[];
    __shared__ int s_count[S][NT];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    unsigned char *const mine = knn_split_lds + wave * Lay::BYTES;
    float *const leaf = reinterpret_cast<float *>(mine) + lane;
    Idx *const kidx = reinterpret_cast<Idx *>(mine + Lay::LEAF_BYTES) + lane;
    float *const ival = reinterpret_cast<float *>(mine + Lay::LEAF_BYTES + Lay::KIDX_BYTES) + lane;
    unsigned char *const iarg =
        mine + Lay::LEAF_BYTES + Lay::KIDX_BYTES + Lay::IVAL_BYTES + lane;
    auto log_of = [&](int w) {  // w >= 1
        return reinterpret_cast<LogIdx *>(knn_split_lds + Split::LOGS_AT +
                                          (w - 1) * Split::LOG_BYTES) + lane;
    };
    LogIdx *const log = log_of(wave > 0 ? wave : 1);  // wave 0 never writes one

    const int b = blockIdx.x / blocks_per_batch;
    const int qi = (blockIdx.x - b * blocks_per_batch) * NT + lane;
    const bool active = qi < n1;
    const float *__restrict__ K = key + (int64_t)b * n2 * 3;
    float qx = 0, qy = 0, qz = 0;
    if (active) {
        const float *q = query + ((int64_t)b * n1 + qi) * 3;
        qx = q[0];
        qy = q[1];
        qz = q[2];
    }

    auto leaf_parent = [&](int n, float &v, int &a) {
        const int s = 2 * n - KMAX;
        const float lv = leaf[s * NT], rv = leaf[(s + 1) * NT];
        const bool right = rv > lv;
        v = right ? rv : lv;
        a = right ? s + 1 : s;
    };

    // Slots: wave 0 fills them with keys 0..k-1 (mink.cuh:63-72; unused slots hold -inf);
    // the other waves start from k empty slots (+inf), which any real distance displaces.
    bool frozen = false;
    float max_key = 0.0f;
    int max_idx = 0;
    auto start_slots = [&]() {
    for (int s = 0; s < KMAX; ++s) {
        float d = -__builtin_huge_valf();
        if (s < k) {
            if (wave == 0) {
                d = tk_dist2<float>(K[s * 3 + 0], K[s * 3 + 1], K[s * 3 + 2], qx, qy, qz);
                if (d != d) {
                    frozen |= s == 0;
                    d = -__builtin_huge_valf();
                }
            } else {
                d = __builtin_huge_valf();
            }
        }
        leaf[s * NT] = d;
        kidx[s * NT] = (Idx)s;
    }
    for (int n = HALF - 1; n >= 1; --n) {
        float lv, rv;
        int la, ra;
        if (2 * n >= HALF) {
            leaf_parent(2 * n, lv, la);
            leaf_parent(2 * n + 1, rv, ra);
        } else {
            lv = ival[2 * n * NT];
            rv = ival[(2 * n + 1) * NT];
            la = iarg[2 * n * NT];
            ra = iarg[(2 * n + 1) * NT];
        }
        const bool right = rv > lv;
        ival[n * NT] = right ? rv : lv;
        iarg[n * NT] = (unsigned char)(right ? ra : la);
    }
    max_key = frozen ? -__builtin_huge_valf() : ival[NT];
    max_idx = iarg[NT];
    };
    start_slots();
    int logged = 0;  // entries this lane wrote to its log (may exceed CAP: overflow)

    // MinK's insertion of key j at distance d < max_key (see knn_tree_kernel).
    auto insert = [&](float d, int j) {
        const int p = max_idx;
        leaf[p * NT] = d;
        kidx[p * NT] = (Idx)j;
        float sv[LEVELS];
        int sa[LEVELS];
        sv[0] = leaf[(p ^ 1) * NT];
        sa[0] = p ^ 1;
        leaf_parent(((KMAX + p) >> 1) ^ 1, sv[1], sa[1]);
#pragma unroll
        for (int l = 2; l < LEVELS; ++l) {
            const int sib = ((KMAX + p) >> l) ^ 1;
            sv[l] = ival[sib * NT];
            sa[l] = iarg[sib * NT];
        }
        float v = d;
        int a = p;
#pragma unroll
        for (int l = 0; l < LEVELS; ++l) {
            const int node = (KMAX + p) >> l;
            const bool take = (node & 1) ? !(v > sv[l]) : (sv[l] > v);
            v = take ? sv[l] : v;
            a = take ? sa[l] : a;
            if (l >= 1 && l + 1 < LEVELS) {
                ival[(node >> 1) * NT] = v;
                iarg[(node >> 1) * NT] = (unsigned char)a;
            }
        }
        max_key = v;
        max_idx = v != d ? a : p;
    };

    // Sweep of the keys [k_begin, k_end) in chunks of 32, inserting (and, for the waves
    // other than 0, logging) as the tree kernel does. `skip_below`: keys the fill took.
    int log_base = 0;  // first key of the slice this wave is sweeping
    auto sweep = [&](int k_begin, int k_end, int skip_below, bool write_log) {
        // With one wave per SIMD nothing hides the latency of the key loads, so they run
        // ahead: lane l holds key `held + l` (two chunks per load, the next 64 keys
        // requested before the current ones are used) and a chunk takes its keys out of
        // those registers lane by lane.
        float hx = 0, hy = 0, hz = 0, nx2 = 0, ny2 = 0, nz2 = 0;
        auto request = [&](int base) {
            int j = base + lane;
            j = j < k_end ? j : k_end - 1;
            j = j < 0 ? 0 : j;
            nx2 = K[(int64_t)j * 3 + 0];
            ny2 = K[(int64_t)j * 3 + 1];
            nz2 = K[(int64_t)j * 3 + 2];
        };
        if (k_begin < k_end)
            request(k_begin);
        for (int first = k_begin; first < k_end; first += CHUNK) {
            const int within = (first - k_begin) & 63;  // 0 or 32: uniform
            if (within == 0) {
                hx = nx2;
                hy = ny2;
                hz = nz2;
                if (first + 64 < k_end)
                    request(first + 64);
            }
            const int maxbits = __builtin_bit_cast(int, max_key);
            unsigned mask = 0u;
            if (first + CHUNK <= k_end) {
#pragma unroll
                for (int i = 0; i < CHUNK; ++i) {
                    const float kx = __builtin_bit_cast(
                        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, hx), within + i));
                    const float ky = __builtin_bit_cast(
                        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, hy), within + i));
                    const float kz = __builtin_bit_cast(
                        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, hz), within + i));
                    const float d = tk_dist2<float>(kx, ky, kz, qx, qy, qz);
                    const unsigned diff = (unsigned)(__builtin_bit_cast(int, d) - maxbits);
                    mask = __builtin_amdgcn_alignbit(mask, diff, 31);
                }
            } else {
                for (int i = 0; i < CHUNK; ++i) {
                    const int j = first + i < k_end ? first + i : k_end - 1;  // masked below
                    const float d = tk_dist2<float>(K[(int64_t)j * 3 + 0], K[(int64_t)j * 3 + 1],
                                                    K[(int64_t)j * 3 + 2], qx, qy, qz);
                    const unsigned diff = (unsigned)(__builtin_bit_cast(int, d) - maxbits);
                    mask = __builtin_amdgcn_alignbit(mask, diff, 31);
                }
            }
            int lo = skip_below - first;
            lo = lo < 0 ? 0 : (lo > CHUNK ? CHUNK : lo);
            int hi = k_end - first;
            hi = hi > CHUNK ? CHUNK : hi;
            unsigned valid = (lo >= CHUNK) ? 0u : (0xffffffffu >> lo);
            valid &= (hi >= CHUNK) ? 0xffffffffu : ~(0xffffffffu >> hi);
            mask &= valid;
            const float *__restrict__ ck = K + (int64_t)first * 3;
            bool has = mask != 0u;
            int i = has ? __builtin_clz(mask) : 0;
            float ex = ck[3 * i + 0], ey = ck[3 * i + 1], ez = ck[3 * i + 2];
            while (__builtin_amdgcn_ballot_w64(has)) {  // wave-uniform
                mask &= ~(0x80000000u >> i);
                const bool has_next = mask != 0u;
                const int i_next = has_next ? __builtin_clz(mask) : 0;
                const float nx = ck[3 * i_next + 0], ny = ck[3 * i_next + 1],
                            nz = ck[3 * i_next + 2];
                const float d = tk_dist2<float>(ex, ey, ez, qx, qy, qz);
                if (has && d < max_key) {
                    insert(d, first + i);
                    if (write_log) {
                        if (logged < CAP)
                            log[logged * NT] = (LogIdx)(first + i - log_base);
                        ++logged;
                    }
                }
                has = has_next;
                i = i_next;
                ex = nx;
                ey = ny;
                ez = nz;
            }
        }
    };

    // The keys are taken in groups of S slices (one group unless the cloud is longer than
    // S slices of 65536 keys): wave 0 carries its slots from group to group, the others
    // start every group from empty slots.
    for (int g0 = 0; g0 < n2; g0 += S * slice_len) {  // uniform over the workgroup
        const int k_begin = g0 + wave * slice_len;
        const int k_end = (k_begin + slice_len < n2) ? k_begin + slice_len : n2;
        log_base = k_begin;
        if (wave == 0) {
            sweep(k_begin, k_end, g0 == 0 ? k : 0, false);
        } else {
            if (g0 > 0)
                start_slots();
            logged = 0;
            if (k_begin < n2)
                sweep(k_begin, k_end, 0, true);
        }
        s_count[wave][lane] = logged;
        __syncthreads();
        if (wave == 0) {
            // ---- wave 0 replays the other slices of the group in key order ----
            for (int w = 1; w < S; ++w) {
                const int w_begin = g0 + w * slice_len;
                if (w_begin >= n2)
                    break;
                const int w_end = (w_begin + slice_len < n2) ? w_begin + slice_len : n2;
                const int count = s_count[w][lane];
                if (__builtin_amdgcn_ballot_w64(count > CAP)) {  // uniform: a log overflowed
                    sweep(w_begin, w_end, 0, false);
                    continue;
                }
                const LogIdx *__restrict__ wl = log_of(w);
                int r = 0;
                bool has = r < count;
                int j = w_begin + (has ? (int)wl[0] : 0);
                float ex = K[(int64_t)j * 3 + 0], ey = K[(int64_t)j * 3 + 1],
                      ez = K[(int64_t)j * 3 + 2];
                while (__builtin_amdgcn_ballot_w64(has)) {  // wave-uniform
                    const bool has_next = r + 1 < count;
                    const int j_next = w_begin + (has_next ? (int)wl[(r + 1) * NT] : 0);
                    const float nx = K[(int64_t)j_next * 3 + 0], ny = K[(int64_t)j_next * 3 + 1],
                                nz = K[(int64_t)j_next * 3 + 2];
                    const float d = tk_dist2<float>(ex, ey, ez, qx, qy, qz);
                    if (has && d < max_key)
                        insert(d, j);
                    ++r;
                    has = has_next;
                    j = j_next;
                    ex = nx;
                    ey = ny;
                    ez = nz;
                }
            }
        }
        if (g0 + S * slice_len < n2)  // uniform
            __syncthreads();  // the logs are free for the next group
    }
    if (wave != 0)
        return;

    if (active) {
        float *od = distance + ((int64_t)b * n1 + qi) * k;
        int64_t *oi = index + ((int64_t)b * n1 + qi) * k;
        for (int s = 0; s < k; ++s) {
            float d = leaf[s * NT];
            if (d == -__builtin_huge_valf())  // a NaN of the fill phase, still in its slot
                d = tk_dist2<float>(K[s * 3 + 0], K[s * 3 + 1], K[s * 3 + 2], qx, qy, qz);
            od[s] = d;
            oi[s] = (int64_t)kidx[s * NT];
        }
    }
}

// Launch with S waves per 64 queries when the plain launch would leave most SIMDs
// without a wave; returns TK3D_ERR_UNSUPPORTED when it does not apply.
template <int KMAX, int S, int CAP>
int knn_tree_split_launch(const float *query, const float *key, float *distance,
                          int64_t *index, int64_t B, int n1, int n2, int k, hipStream_t s)
{
    // a log holds 16-bit positions within its slice: slices of at most 65536 keys, in as
    // many groups of S slices as that takes
    const int groups = (int)(((int64_t)n2 + (int64_t)S * 65536 - 1) / ((int64_t)S * 65536));
    int slice_len = (int)(((int64_t)n2 + (int64_t)S * groups - 1) / ((int64_t)S * groups));
    slice_len = (slice_len + 31) / 32 * 32;
    const int64_t bpb = ((int64_t)n1 + 63) / 64;
    // Worth it when sweeping dominates the insertions (timed on an MI355X): from 2048 keys
    // for k <= 8, 4096 for k <= 16, 8192 for k <= 32, and only while every workgroup has a
    // CU to itself.
    constexpr int MIN_KEYS = KMAX <= 8 ? 2048 : KMAX <= 16 ? 4096 : 8192;
    if (n2 < MIN_KEYS || slice_len < k || B * bpb > 256)
        return TK3D_ERR_UNSUPPORTED;
    auto launch = [&](auto wide) {
        // key indices of the slots in LDS: 16 bits up to 65536 keys, else 32 bits and
        // slightly shorter logs (a slice whose log overflows is swept again by wave 0)
        constexpr bool IDX16 = !decltype(wide)::value;
        constexpr int LOG = IDX16 ? CAP : CAP - 16 * S;
        using Split = KnnSplitLayout<KMAX, IDX16, S, LOG>;
        static_assert(Split::BYTES + 64 * S * 4 <= 160 * 1024, "LDS of one CU");
        constexpr auto kernel = knn_tree_split_kernel_f32<KMAX, IDX16, S, LOG>;
        const int allowed = tk_allow_dynamic_lds<kernel>(Split::BYTES);
        if (allowed != TK3D_OK)
            return allowed;
        hipLaunchKernelGGL(kernel, dim3((unsigned)(B * bpb)), dim3(64 * S), Split::BYTES, s,
                           query, key, distance, index, (int)bpb, n1, n2, k, slice_len);
        return tk_launch_status();
    };
    if (n2 <= 65536)
        return launch(std::false_type{});
    return launch(std::true_type{});
}

template <int KMAX, bool IDX16, typename T = float, bool SOA = false>
int knn_tree_launch_as(const T *query, const T *key, T *distance, int64_t *index,
                       int64_t B, int n1, int n2, int k, hipStream_t s)
{
    constexpr int LDS_BYTES = KnnTreeLayout<KMAX, IDX16, T>::BYTES;
    if (LDS_BYTES > 48 * 1024) {
        const int allowed =
            tk_allow_dynamic_lds<knn_tree_kernel<T, KMAX, IDX16, SOA>>(LDS_BYTES);
        if (allowed != TK3D_OK)
            return allowed;
    }
    const int64_t bpb = ((int64_t)n1 + 63) / 64;
    if (B * bpb > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((knn_tree_kernel<T, KMAX, IDX16, SOA>), dim3((unsigned)(B * bpb)), dim3(64),
                       LDS_BYTES, s, query, key, distance, index, (int)bpb, n1, n2, k);
    return tk_launch_status();
}

template <int KMAX, typename T = float, bool SOA = false>
int knn_tree_launch(const T *query, const T *key, T *distance, int64_t *index,
                    int64_t B, int n1, int n2, int k, hipStream_t s)
{
    if (n2 <= 65536)
        return knn_tree_launch_as<KMAX, true, T, SOA>(query, key, distance, index, B, n1, n2, k, s);
    return knn_tree_launch_as<KMAX, false, T, SOA>(query, key, distance, index, B, n1, n2, k, s);
}

// The tree kernel with the matrix-core sweep: pays where the launch fills the chip and the
// key cloud amortises the prologue (two passes over the keys per workgroup).
// Timed against the plain tree kernel on an MI355X for k = 17..32: 1.1-1.5 times faster
// for 32768 to 65536 queries against 4096 keys or more, slower with more queries (fewer
// waves fit beside the staged terms, and a workgroup's waves wait for each other at every
// stage) and no faster on shorter key clouds; for k <= 16 the register kernel above wins.
template <int KMAX, int NW>
int knn_tree_matrix_launch(const float *query, const float *key, float *distance,
                           int64_t *index, int64_t B, int n1, int n2, int k, hipStream_t s)
{
    if (n2 > 65536 || n2 < 4096 || B * n1 < 32768 || B * n1 >= 131072)
        return TK3D_ERR_UNSUPPORTED;
    constexpr int LDS_BYTES = 2 * 256 * 32 + NW * KnnTreeLayout<KMAX, true>::BYTES;
    constexpr auto kernel = knn_tree_matrix_kernel_f32<KMAX, true, NW>;
    const int allowed = tk_allow_dynamic_lds<kernel>(LDS_BYTES);
    if (allowed != TK3D_OK)
        return allowed;
    const int64_t bpb = ((int64_t)n1 + 64 * NW - 1) / (64 * NW);
    if (B * bpb > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(B * bpb)), dim3(64 * NW), LDS_BYTES, s, query, key,
                       distance, index, (int)bpb, n1, n2, k);
    return tk_launch_status();
}

// Any k: the structure lives in the output rows in global memory.
template <typename T>
__global__ __launch_bounds__(KNN_BLOCK) void knn_global_kernel(
    const T *__restrict__ query, const T *__restrict__ key, T *distance, int64_t *index,
    int blocks_per_batch, int n1, int n2, int k)
{
    __shared__ T skey[KNN_STAGE * 4];
    const int tid = threadIdx.x;
    const int b = blockIdx.x / blocks_per_batch;
    const int qi = (blockIdx.x - b * blocks_per_batch) * KNN_BLOCK + tid;
    const bool active = qi < n1;
    const T *__restrict__ K = key + (int64_t)b * n2 * 3;
    T qx = 0, qy = 0, qz = 0;
    T *kd = distance;
    int64_t *ki = index;
    if (active) {
        const T *q = query + ((int64_t)b * n1 + qi) * 3;
        qx = q[0];
        qy = q[1];
        qz = q[2];
        kd = distance + ((int64_t)b * n1 + qi) * k;
        ki = index + ((int64_t)b * n1 + qi) * k;
    }
    T max_key = (T)0;
    int max_idx = 0;
    int size = 0;
    for (int stage0 = 0; stage0 < n2; stage0 += KNN_STAGE) {
        __syncthreads();
        for (int j = tid; j < KNN_STAGE; j += KNN_BLOCK) {
            const int kj = stage0 + j;
            T x = 0, y = 0, z = 0;
            if (kj < n2) {
                x = K[(int64_t)kj * 3 + 0];
                y = K[(int64_t)kj * 3 + 1];
                z = K[(int64_t)kj * 3 + 2];
            }
            skey[j * 4 + 0] = x;
            skey[j * 4 + 1] = y;
            skey[j * 4 + 2] = z;
            skey[j * 4 + 3] = (T)0;
        }
        __syncthreads();
        if (!active)
            continue;
        const int left = n2 - stage0;
        const int cnt = left < KNN_STAGE ? left : KNN_STAGE;
        for (int j = 0; j < cnt; ++j) {
            const T d = tk_dist2<T>(skey[j * 4 + 0], skey[j * 4 + 1], skey[j * 4 + 2], qx, qy,
                                    qz);
            const int kj = stage0 + j;
            if (size < k) {
                kd[size] = d;
                ki[size] = kj;
                if (size == 0 || d > max_key) {
                    max_key = d;
                    max_idx = size;
                }
                ++size;
            } else if (d < max_key) {
                kd[max_idx] = d;
                ki[max_idx] = kj;
                max_key = d;
                for (int s = 0; s < k; ++s) {
                    const T cur = kd[s];
                    if (cur > max_key) {
                        max_key = cur;
                        max_idx = s;
                    }
                }
            }
        }
    }
}

template <typename T, int KMAX, bool SOA = false, bool WEIGHTS = false>
void knn_launch(const T *query, const T *key, T *distance, int64_t *index, int64_t B,
                int bpb, int n1, int n2, int k, hipStream_t s, T *weight = nullptr,
                T eps = (T)0)
{
    if constexpr (sizeof(T) == 4)
        hipLaunchKernelGGL((knn_batched_kernel_f32<KMAX, SOA, WEIGHTS>),
                           dim3((unsigned)(B * bpb)), dim3(KNN_BLOCK), 0, s, query, key, distance,
                           index, weight, eps, bpb, n1, n2, k);
    else
        hipLaunchKernelGGL((knn_register_kernel<T, KMAX, SOA, WEIGHTS>),
                           dim3((unsigned)(B * bpb)), dim3(KNN_BLOCK), 0, s, query, key, distance,
                           index, weight, eps, bpb, n1, n2, k);
}

// Where the pre-filtered kernel is the fastest route for k <= 16, from timing it against
// every other kernel here on an MI355X (k = 1..16, 128 to 524288 queries, 128 to 65536
// keys, 1100 shapes): 1.1-2.0 times faster inside these bounds, 0.7-1.0 outside. Short key
// clouds do not amortise its prologue (two passes over the keys per workgroup); with few
// queries and very long clouds the kernels that share the keys of 64 queries among several
// waves win, from k = 5 on.
inline bool knn_filter_pays(int64_t queries, int n2, int k)
{
    if (k <= 4)
        return n2 >= 512 || (n2 >= 256 && queries >= 4096);
    if (k > 16)  // 32 slots as a sorted list, key indices in LDS; the tree kernel keeps
                 // short clouds with many queries (B=24, 4096 x 700: 117 against 137 us)
        return n2 <= 65536 && queries >= 4096 && (n2 >= 1024 || (n2 >= 512 && queries <= 32768));
    if (queries < 32768 && n2 > (k <= 8 ? 8192 : 32768))
        return false;
    return n2 >= (k <= 8 ? 512 : 1024) || (n2 >= 512 && queries >= 131072);
}

// Whether knn_filter_launch takes this launch: the one test both entry points and the
// launch itself go by.
inline bool knn_filter_takes(int64_t B, int n1, int n2, int k)
{
    const int64_t bpb = ((int64_t)n1 + 511) / 512;
    return k <= 32 && knn_filter_pays(B * n1, n2, k) && B * bpb <= TK_MAX_I32;
}

template <int KMAX, bool SOA, bool WEIGHTS, int LANES>
int knn_filter_launch_as(const float *query, const float *key, float *distance, int64_t *index,
                         float *weight, float eps, int64_t B, int n1, int n2, int k, hipStream_t s)
{
    const int64_t bpb = ((int64_t)n1 + LANES - 1) / LANES;
    if constexpr (KMAX >= 8) {  // (4 slots: the slot-ordered registers are 2-7 % faster)
        if (n2 <= 65536) {  // the slots' key indices in LDS, 16 bits each
            constexpr auto kernel =
                knn_filter_kernel_f32<KMAX, 1, SOA, WEIGHTS, true, LANES, true, !WEIGHTS>;
            constexpr int lds = KMAX * LANES * (int)sizeof(unsigned short);
            const int allowed = tk_allow_dynamic_lds<kernel>(lds);
            if (allowed != TK3D_OK)
                return allowed;
            hipLaunchKernelGGL(kernel, dim3((unsigned)(B * bpb)), dim3(LANES), lds, s, query, key,
                               distance, index, weight, eps, (int)bpb, n1, n2, k);
            return tk_launch_status();
        }
        if constexpr (KMAX > 16)
            return TK3D_ERR_UNSUPPORTED;  // 32 slots exist as a sorted list only
    }
    if constexpr (KMAX <= 16)
        hipLaunchKernelGGL((knn_filter_kernel_f32<KMAX, 1, SOA, WEIGHTS, true, LANES>),
                           dim3((unsigned)(B * bpb)), dim3(LANES), 0, s, query, key, distance,
                           index, weight, eps, (int)bpb, n1, n2, k);
    return tk_launch_status();
}

template <int KMAX, bool SOA, bool WEIGHTS>
int knn_filter_launch(const float *query, const float *key, float *distance, int64_t *index,
                      float *weight, float eps, int64_t B, int n1, int n2, int k, hipStream_t s,
                      bool whatever_the_size = false)
{
    // One query per lane, 512 lanes: two workgroups (16 waves) per CU. Two queries per lane
    // in 256 lanes need twice the registers, which leaves two waves per SIMD, and were 1.1
    // to 1.4 times slower on every shape (k = 16 at B=32, 8192 x 2048: 222 -> 191 us).
    // A launch of few such workgroups leaves CUs without one: 256 lanes then (128 workgroups,
    // B=8, 8192 x 2048: k = 3 52 -> 48 us, k = 16 96 -> 85 us, k = 32 189 -> 142 us; at 160
    // workgroups with up to 8 slots, at 192 with more, the larger workgroup wins: its staged
    // keys serve more queries).
    const int64_t bpb = ((int64_t)n1 + 511) / 512;
    if (B * bpb > TK_MAX_I32 || !(whatever_the_size || knn_filter_takes(B, n1, n2, k)))
        return TK3D_ERR_UNSUPPORTED;
    if (B * bpb <= (KMAX <= 8 ? 128 : 160))
        return knn_filter_launch_as<KMAX, SOA, WEIGHTS, 256>(query, key, distance, index, weight,
                                                             eps, B, n1, n2, k, s);
    return knn_filter_launch_as<KMAX, SOA, WEIGHTS, 512>(query, key, distance, index, weight, eps,
                                                         B, n1, n2, k, s);
}

template <typename T>
int knn(const T *query, const T *key, int64_t B, int64_t N1, int64_t N2, int64_t k,
        int version, T *distance, int64_t *index, void *stream)
{
    if (B < 0 || N1 < 0 || N2 < 0)
        return TK3D_ERR_BAD_SIZE;
    if (version != 0 && version != 1)
        return TK3D_ERR_BAD_VERSION;
    if (k <= 0 || k > N2)
        return TK3D_ERR_BAD_K;
    if (N1 > TK_MAX_I32 / 4 || N2 > TK_MAX_I32 / 4 || !tk_fits(TK_MAX_ELEMS, B, N1, k) ||
        !tk_fits(TK_MAX_ELEMS, B, N2, 3))
        return TK3D_ERR_UNSUPPORTED;
    if (B * N1 == 0)
        return TK3D_OK;
    if (!query || !key || !distance || !index)
        return TK3D_ERR_NULL_POINTER;
    const int64_t bpb = (N1 + KNN_BLOCK - 1) / KNN_BLOCK;
    if (B * bpb > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    const int n1 = (int)N1, n2 = (int)N2, kk = (int)k;
    if (k <= 4) {
        // the pre-filtered kernel wherever it pays (512 keys or more), else the batched kernel
        if constexpr (sizeof(T) == 4) {
            const int rc = knn_filter_launch<4, false, false>(query, key, distance, index, nullptr,
                                                              0.0f, B, n1, n2, kk, s);
            if (rc != TK3D_ERR_UNSUPPORTED)
                return rc;
        }
        knn_launch<T, 4>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
    } else if constexpr (sizeof(T) == 4) {
        // fp32, k >= 5: slots in LDS as a tournament tree (k = 16 at B=32, 8192 x 2048:
        // 0.30 ms against 0.41 ms with the slots in registers). Small launches with k <= 8
        // are a little faster in registers.
        if (k <= 32) {
            // pre-filtered sweep on the matrix cores, slots in registers: wherever it pays
            const int rc =
                k <= 8 ? knn_filter_launch<8, false, false>(query, key, distance, index, nullptr,
                                                            0.0f, B, n1, n2, kk, s)
                : k <= 16
                    ? knn_filter_launch<16, false, false>(query, key, distance, index, nullptr,
                                                          0.0f, B, n1, n2, kk, s)
                    : knn_filter_launch<32, false, false>(query, key, distance, index, nullptr,
                                                          0.0f, B, n1, n2, kk, s);
            if (rc != TK3D_ERR_UNSUPPORTED)
                return rc;
        }
        if (k <= 16) {
            // few queries: four waves share the keys of every 64 queries (1.2-3.3 times
            // faster from 2048 / 4096 keys on)
            const int rc = k <= 8 ? knn_tree_split_launch<8, 4, 352>(query, key, distance, index,
                                                                     B, n1, n2, kk, s)
                                  : knn_tree_split_launch<16, 4, 320>(query, key, distance,
                                                                      index, B, n1, n2, kk, s);
            if (rc != TK3D_ERR_UNSUPPORTED)
                return rc;
        }
        if (k > 16 && k <= 32) {
            // k = 17..32 logs more insertions: two waves per 64 queries, the second wave's
            // log gets all the spare LDS (1.15-1.5 times faster from 8192 keys on)
            const int rc = knn_tree_split_launch<32, 2, 896>(query, key, distance, index, B, n1,
                                                             n2, kk, s);
            if (rc != TK3D_ERR_UNSUPPORTED)
                return rc;
        }
        if (k > 16 && k <= 32) {
            // a chip's worth of queries on long key clouds: matrix-core sweep into the tree
            const int rc = knn_tree_matrix_launch<32, 2>(query, key, distance, index, B, n1, n2,
                                                         kk, s);
            if (rc != TK3D_ERR_UNSUPPORTED)
                return rc;
        }
        if (k <= 8 && B * N1 < 131072)
            knn_launch<T, 8>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
        else if (k <= 8)
            return knn_tree_launch<8>(query, key, distance, index, B, n1, n2, kk, s);
        else if (k <= 16)
            return knn_tree_launch<16>(query, key, distance, index, B, n1, n2, kk, s);
        else if (k <= 32)
            return knn_tree_launch<32>(query, key, distance, index, B, n1, n2, kk, s);
        else if (k <= 64)
            return knn_tree_launch<64>(query, key, distance, index, B, n1, n2, kk, s);
        else if (k <= 128)
            return knn_tree_launch<128>(query, key, distance, index, B, n1, n2, kk, s);
        else if (k <= 256 && n2 <= 65536)
            // 136 KiB of LDS per wave with 16-bit key indices: one wave per CU, still some
            // twenty times faster than keeping the slots in global memory
            return knn_tree_launch_as<256, true>(query, key, distance, index, B, n1, n2, kk, s);
        else
            hipLaunchKernelGGL((knn_global_kernel<T>), dim3((unsigned)(B * bpb)),
                               dim3(KNN_BLOCK), 0, s, query, key, distance, index, (int)bpb,
                               n1, n2, kk);
    } else {
        // fp64: slots in registers up to k = 16, the LDS tree beyond (k = 64 at B=32,
        // 2048 x 8192: the register variant pays 2 k selects per insertion on 64-bit values)
        if (k <= 8)
            knn_launch<T, 8>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
        else if (k <= 16)
            knn_launch<T, 16>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
        else if (k <= 32)
            return knn_tree_launch<32, T>(query, key, distance, index, B, n1, n2, kk, s);
        else if (k <= 64)
            return knn_tree_launch<64, T>(query, key, distance, index, B, n1, n2, kk, s);
        else if (k <= 128)
            return knn_tree_launch<128, T>(query, key, distance, index, B, n1, n2, kk, s);
        else
            hipLaunchKernelGGL((knn_global_kernel<T>), dim3((unsigned)(B * bpb)),
                               dim3(KNN_BLOCK), 0, s, query, key, distance, index, (int)bpb,
                               n1, n2, kk);
    }
    return tk_launch_status();
}

// KNN on [B,3,N] clouds with the kernels that read either layout, k <= 64 (beyond:
// TK3D_ERR_UNSUPPORTED before anything is launched; the caller copies the clouds and calls
// knn()). fp32: the pre-filtered sweep where knn() would launch it, the register kernel for
// k <= 4, else the LDS tree kernel (the variants of it that share keys among several waves,
// or sweep on the matrix cores, read [B,N,3] only). fp64 runs the same kernels on either
// layout.
template <typename T>
int knn_bcn(const T *query, const T *key, int64_t B, int64_t N1, int64_t N2, int64_t k,
            int version, T *distance, int64_t *index, void *stream)
{
    if (B < 0 || N1 < 0 || N2 < 0)
        return TK3D_ERR_BAD_SIZE;
    if (version != 0 && version != 1)
        return TK3D_ERR_BAD_VERSION;
    if (k <= 0 || k > N2)
        return TK3D_ERR_BAD_K;
    if (N1 > TK_MAX_I32 / 4 || N2 > TK_MAX_I32 / 4 || !tk_fits(TK_MAX_ELEMS, B, N1, k) ||
        !tk_fits(TK_MAX_ELEMS, B, N2, 3) || k > 64)
        return TK3D_ERR_UNSUPPORTED;
    const int64_t bpb = (N1 + KNN_BLOCK - 1) / KNN_BLOCK;
    if (B * bpb > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    const int n1 = (int)N1, n2 = (int)N2, kk = (int)k;
    if (B * N1 == 0)
        return TK3D_OK;
    if (!query || !key || !distance || !index)
        return TK3D_ERR_NULL_POINTER;
    hipStream_t s = (hipStream_t)stream;
    if constexpr (sizeof(T) == 4) {
        if (k > 4 && !knn_filter_takes(B, n1, n2, kk)) {
            // k = 17..64, or a launch the pre-filtered sweep does not pay for: the LDS tree,
            // reading the coordinate planes
            if (k <= 8)
                return knn_tree_launch<8, float, true>(query, key, distance, index, B, n1, n2, kk, s);
            if (k <= 16)
                return knn_tree_launch<16, float, true>(query, key, distance, index, B, n1, n2, kk, s);
            if (k <= 32)
                return knn_tree_launch<32, float, true>(query, key, distance, index, B, n1, n2, kk, s);
            return knn_tree_launch<64, float, true>(query, key, distance, index, B, n1, n2, kk, s);
        }
        int rc = TK3D_ERR_UNSUPPORTED;
        if (k <= 4) {
            rc = knn_filter_launch<4, true, false>(query, key, distance, index, nullptr, 0.0f, B,
                                                   n1, n2, kk, s);
            if (rc == TK3D_ERR_UNSUPPORTED) {
                knn_launch<T, 4, true>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
                rc = tk_launch_status();
            }
        } else if (k <= 8) {
            rc = knn_filter_launch<8, true, false>(query, key, distance, index, nullptr, 0.0f, B,
                                                   n1, n2, kk, s);
        } else if (k <= 16) {
            rc = knn_filter_launch<16, true, false>(query, key, distance, index, nullptr, 0.0f, B,
                                                    n1, n2, kk, s);
        } else {
            rc = knn_filter_launch<32, true, false>(query, key, distance, index, nullptr, 0.0f, B,
                                                    n1, n2, kk, s);
        }
        return rc;
    } else {
        if (k <= 4)
            knn_launch<T, 4, true>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
        else if (k <= 8)
            knn_launch<T, 8, true>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
        else if (k <= 16)
            knn_launch<T, 16, true>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
        else if (k <= 32)
            knn_launch<T, 32, true>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
        else
            knn_launch<T, 64, true>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
        return tk_launch_status();
    }
}

// 3 nearest neighbours with the interpolation weights formed in the same kernel.
template <typename T>
int three_nn(const T *query, const T *key, bool channels_first, int64_t B, int64_t N1,
             int64_t N2, double eps, T *distance, int64_t *index, T *weight, void *stream)
{
    if (B < 0 || N1 < 0 || N2 < 0)
        return TK3D_ERR_BAD_SIZE;
    if (N2 < 3)
        return TK3D_ERR_BAD_K;
    if (N1 > TK_MAX_I32 / 4 || N2 > TK_MAX_I32 / 4 || !tk_fits(TK_MAX_ELEMS, B, N1, 3) ||
        !tk_fits(TK_MAX_ELEMS, B, N2, 3))
        return TK3D_ERR_UNSUPPORTED;
    if (B * N1 == 0)
        return TK3D_OK;
    if (!query || !key || !distance || !index || !weight)
        return TK3D_ERR_NULL_POINTER;
    const int64_t bpb = (N1 + KNN_BLOCK - 1) / KNN_BLOCK;
    if (B * bpb > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    if constexpr (sizeof(T) == 4) {
        const int rf = channels_first
                           ? knn_filter_launch<4, true, true>(query, key, distance, index, weight,
                                                              (float)eps, B, (int)N1, (int)N2, 3, s)
                           : knn_filter_launch<4, false, true>(query, key, distance, index, weight,
                                                               (float)eps, B, (int)N1, (int)N2, 3,
                                                               s);
        if (rf != TK3D_ERR_UNSUPPORTED)
            return rf;
    }
    if (channels_first)
        knn_launch<T, 4, true, true>(query, key, distance, index, B, (int)bpb, (int)N1, (int)N2,
                                     3, s, weight, (T)eps);
    else
        knn_launch<T, 4, false, true>(query, key, distance, index, B, (int)bpb, (int)N1,
                                      (int)N2, 3, s, weight, (T)eps);
    return tk_launch_status();
}

}  // namespace

extern "C" {

int tk3d_three_nn_f32(const float *query, const float *key, int channels_first, int64_t B,
                      int64_t N1, int64_t N2, double eps, float *distance, int64_t *index,
                      float *weight, void *stream)
{
    return three_nn<float>(query, key, channels_first != 0, B, N1, N2, eps, distance, index,
                           weight, stream);
}

int tk3d_three_nn_f64(const double *query, const double *key, int channels_first, int64_t B,
                      int64_t N1, int64_t N2, double eps, double *distance, int64_t *index,
                      double *weight, void *stream)
{
    return three_nn<double>(query, key, channels_first != 0, B, N1, N2, eps, distance, index,
                            weight, stream);
}

int tk3d_knn_distance_bcn_f32(const float *query, const float *key, int64_t B, int64_t N1,
                              int64_t N2, int64_t k, int version, float *distance,
                              int64_t *index, void *stream)
{
    return knn_bcn<float>(query, key, B, N1, N2, k, version, distance, index, stream);
}

int tk3d_knn_distance_bcn_f64(const double *query, const double *key, int64_t B, int64_t N1,
                              int64_t N2, int64_t k, int version, double *distance,
                              int64_t *index, void *stream)
{
    return knn_bcn<double>(query, key, B, N1, N2, k, version, distance, index, stream);
}

int tk3d_knn_distance_f32(const float *query, const float *key, int64_t B, int64_t N1,
                          int64_t N2, int64_t k, int version, float *distance,
                          int64_t *index, void *stream)
{
    return knn<float>(query, key, B, N1, N2, k, version, distance, index, stream);
}

int tk3d_knn_distance_f64(const double *query, const double *key, int64_t B, int64_t N1,
                          int64_t N2, int64_t k, int version, double *distance,
                          int64_t *index, void *stream)
{
    return knn<double>(query, key, B, N1, N2, k, version, distance, index, stream);
}

int tk3d_debug_knn_filter_f32(const float *query, const float *key, int64_t B, int64_t N1,
                              int64_t N2, int64_t k, float *distance, int64_t *index,
                              void *stream)
{
    if (B < 0 || N1 < 0 || N2 < 0)
        return TK3D_ERR_BAD_SIZE;
    if (k <= 0 || k > N2)
        return TK3D_ERR_BAD_K;
    if (k > 16 || N2 < 256 || N1 > TK_MAX_I32 / 4 || N2 > TK_MAX_I32 / 4 ||
        !tk_fits(TK_MAX_ELEMS, B, N1, k) || !tk_fits(TK_MAX_ELEMS, B, N2, 3))
        return TK3D_ERR_UNSUPPORTED;
    if (B * N1 == 0)
        return TK3D_OK;
    if (!query || !key || !distance || !index)
        return TK3D_ERR_NULL_POINTER;
    hipStream_t s = (hipStream_t)stream;
    const int n1 = (int)N1, n2 = (int)N2, kk = (int)k;
    if (k <= 4)
        return knn_filter_launch<4, false, false>(query, key, distance, index, nullptr, 0.0f, B,
                                                  n1, n2, kk, s, true);
    if (k <= 8)
        return knn_filter_launch<8, false, false>(query, key, distance, index, nullptr, 0.0f, B,
                                                  n1, n2, kk, s, true);
    return knn_filter_launch<16, false, false>(query, key, distance, index, nullptr, 0.0f, B, n1,
                                               n2, kk, s, true);
}

}  // extern "C"

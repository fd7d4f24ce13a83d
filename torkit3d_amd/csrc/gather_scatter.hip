// Group points (gather) and feature interpolation for gfx950, forward and backward.
//
// Both ops are the same two memory-bound patterns over feature rows [B,C,N1]:
//
//   gather :  out[b,c,p]            = sum_{i<KK} in[b,c,idx[b,p,i]] * w[b,p,i]
//   scatter:  gin[b,c,idx[b,p,i]] += gout[b,c,p] * w[b,p,i]
//
// group points is KK = 1 without weights over p = (m,s) flattened (N2*K points);
// interpolation is KK = K (3 in the reference) with weights over p = n.
//
// gather: a workgroup owns a tile of p and a group of channels. The indices (and
// weights) of the tile are read once, checked, narrowed to 32 bits and kept in
// registers; the channel loop then issues only the row gathers and one coalesced
// store per channel, where the reference re-reads index and weight for every
// channel (interpolate_kernel.cu:34-41) or pays ATen's generic gather
// (group_points_kernel.cu:26-29).
//
// scatter: a workgroup owns CG destination rows [CG][N1] in LDS, streams its
// share of p with coalesced reads of gout and accumulates with LDS atomics, then
// writes the rows out with plain coalesced stores - no global atomics and no
// zero-fill when one workgroup covers all p. fp32 accumulates in 64-bit fixed point
// (integer LDS atomics: fast, and the sums do not depend on the order of arrival);
// fp64, and fp32 rows holding NaN or inf, use floating-point LDS atomics, whose
// summation order differs from run to run exactly as in the reference (one global
// atomicAdd per element, group_points_kernel.cu:63, interpolate_kernel.cu:142).
// When B*C is too small to fill the chip the p range is split over several
// workgroups that merge into a zero-filled output with global atomics. Rows too
// long for LDS are accumulated in windows of destinations or, longer still, with
// global atomics directly.

#include "tk3d_common.h"
#include <type_traits>

namespace {

constexpr int GS_BLOCK = 256;

// ---- gather -------------------------------------------------------------------

template <typename T, int KK, bool HAS_W, int V>
__global__ __launch_bounds__(GS_BLOCK) void gather_kernel(
    const T *__restrict__ in, const int64_t *__restrict__ idx, const T *__restrict__ w,
    T *__restrict__ out, int c_total, int wc_total, int wc_off, int n1, int64_t np, int cg, int vec_ok)
{
    const int b = blockIdx.z;
    const int c0 = blockIdx.y * cg;
    const int c1 = (c0 + cg < c_total) ? c0 + cg : c_total;
    const int64_t p0 = ((int64_t)blockIdx.x * GS_BLOCK + threadIdx.x) * V;
    if (p0 >= np)
        return;

    int src[V][KK];
    T wt[V][KK];
#pragma unroll
    for (int v = 0; v < V; ++v) {
#pragma unroll
        for (int i = 0; i < KK; ++i) {
            const int64_t p = p0 + v;
            int64_t j = -1;
            T ww = (T)0;
            if (p < np) {
                j = idx[((int64_t)b * np + p) * KK + i];
                if (HAS_W)
                    ww = w[((int64_t)b * np + p) * KK + i];
            }
            const bool ok = j >= 0 && j < n1;
            src[v][i] = ok ? (int)j : -1;
            wt[v][i] = ww;
        }
    }

    const bool full = (p0 + V <= np);
    for (int c = c0; c < c1; ++c) {
        const T *__restrict__ row = in + ((int64_t)b * c_total + c) * n1;
        T *__restrict__ orow = out + ((int64_t)b * wc_total + wc_off + c) * np;
        T val[V];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            if (HAS_W) {
                // out = 0; out = fma(in, w, out) per neighbour, in slot order
                // (interpolate_kernel.cu:31-42 under default contraction).
                T acc = (T)0;
#pragma unroll
                for (int i = 0; i < KK; ++i)
                    if (src[v][i] >= 0)
                        acc = tk_fma<T>(row[src[v][i]], wt[v][i], acc);
                val[v] = acc;
            } else {
                val[v] = src[v][0] >= 0 ? row[src[v][0]] : (T)0;
            }
        }
        if (full && vec_ok && V == 4 && sizeof(T) == 4) {
            float4 pack;
            pack.x = (float)val[0];
            pack.y = (float)val[1 % V];
            pack.z = (float)val[2 % V];
            pack.w = (float)val[3 % V];
            *reinterpret_cast<float4 *>(orow + p0) = pack;
        } else if (full && vec_ok && V == 2 && sizeof(T) == 8) {
            double2 pack;
            pack.x = (double)val[0];
            pack.y = (double)val[1 % V];
            *reinterpret_cast<double2 *>(orow + p0) = pack;
        } else {
#pragma unroll
            for (int v = 0; v < V; ++v)
                if (p0 + v < np)
                    orow[p0 + v] = val[v];
        }
    }
}


// Same gather with the source rows staged in LDS. Row gathers through the vector
// cache cost one cache line per lane (64 lanes -> 64 lines per load instruction),
// which caps the plain kernel near 2 TB/s of output; LDS serves the same random
// reads at bank rate. grid = (point chunks, channel groups, B); LDS = cg*n1 elements.
//
// A wave covers 64*V consecutive points and lane l takes points l, l+64, ... of that
// span: every index, weight and output access of the wave is then a run of
// consecutive elements (indices: 24-byte stride for three neighbours), instead of
// each lane walking its own 96 bytes of the index array, which costs the vector
// cache one line lookup per lane and load.
template <typename T, int KK, bool HAS_W, int V, int NT>
__global__ __launch_bounds__(NT) void gather_lds_kernel(
    const T *__restrict__ in, const int64_t *__restrict__ idx, const T *__restrict__ w,
    T *__restrict__ out, int c_total, int wc_total, int wc_off, int n1, int64_t np, int cg, int64_t chunk_len, int vec_ok)
{
    extern __shared__ __align__(16) unsigned char gather_smem[];
    T *rows = reinterpret_cast<T *>(gather_smem);  // [cg][n1]
    const int b = blockIdx.z;
    const int c0 = blockIdx.y * cg;
    const int nc = (c0 + cg < c_total) ? cg : c_total - c0;
    const T *__restrict__ src_rows = in + ((int64_t)b * c_total + c0) * n1;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t ps = (int64_t)blockIdx.x * chunk_len;
    const int64_t pe = (ps + chunk_len < np) ? ps + chunk_len : np;

    // Indices and weights are fetched one iteration ahead (the first set while the rows
    // are staged) and only decoded when their iteration starts.
    int64_t jn[V][KK];
    T wn[V][KK];
    auto fetch = [&](int64_t p0) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const int64_t p = p0 + v * 64;
            if constexpr (KK == 3) {
                // a point's three indices and three weights as one run each: element by
                // element a wave's request touches every cache line of the run three times
                struct __attribute__((aligned(8))) Idx3 { int64_t a, b, c; };
                struct __attribute__((aligned(sizeof(T)))) W3 { T a, b, c; };
                Idx3 ji = {-1, -1, -1};
                W3 wi = {(T)0, (T)0, (T)0};
                if (p < pe) {
                    ji = *reinterpret_cast<const Idx3 *>(idx + ((int64_t)b * np + p) * 3);
                    if (HAS_W)
                        wi = *reinterpret_cast<const W3 *>(w + ((int64_t)b * np + p) * 3);
                }
                jn[v][0] = ji.a;
                jn[v][1] = ji.b;
                jn[v][2] = ji.c;
                wn[v][0] = wi.a;
                wn[v][1] = wi.b;
                wn[v][2] = wi.c;
            } else {
#pragma unroll
                for (int i = 0; i < KK; ++i) {
                    jn[v][i] = -1;
                    wn[v][i] = (T)0;
                    if (p < pe) {
                        jn[v][i] = idx[((int64_t)b * np + p) * KK + i];
                        if (HAS_W)
                            wn[v][i] = w[((int64_t)b * np + p) * KK + i];
                    }
                }
            }
        }
    };
    const int64_t pfirst = ps + (int64_t)wave * (64 * V) + lane;
    fetch(pfirst);
    {
        // the staged rows are contiguous in global memory: 16-byte copies when aligned
        constexpr int E = 16 / (int)sizeof(T);
        const int total = nc * n1;
        const bool wide = ((uintptr_t)src_rows & 15) == 0;
        const int nwide = wide ? total / E : 0;
        const float4 *__restrict__ s4 = reinterpret_cast<const float4 *>(src_rows);
        float4 *d4 = reinterpret_cast<float4 *>(rows);
#pragma unroll 4
        for (int i = threadIdx.x; i < nwide; i += NT)
            d4[i] = s4[i];
        for (int i = nwide * E + threadIdx.x; i < total; i += NT)
            rows[i] = src_rows[i];
    }
    __syncthreads();

    for (int64_t p0 = pfirst; p0 < pe; p0 += (int64_t)NT * V) {
        int src[V][KK];
        T wt[V][KK];
#pragma unroll
        for (int v = 0; v < V; ++v) {
#pragma unroll
            for (int i = 0; i < KK; ++i) {
                const int64_t j = jn[v][i];
                src[v][i] = (j >= 0 && j < n1) ? (int)j : -1;
                wt[v][i] = wn[v][i];
            }
        }
        if (p0 + (int64_t)NT * V < pe)
            fetch(p0 + (int64_t)NT * V);
        // Every lane of the wave inside the points and every index inside the row (the
        // usual case): all LDS reads of a channel are issued together and nothing is
        // predicated. Otherwise each read sits behind a test of its own.
        bool plain = p0 + (V - 1) * 64 < pe;
#pragma unroll
        for (int v = 0; v < V; ++v)
#pragma unroll
            for (int i = 0; i < KK; ++i)
                plain = plain && src[v][i] >= 0;
        if (__all(plain)) {
#pragma unroll 4
            for (int c = 0; c < nc; ++c) {
                const T *row = rows + c * n1;
                T *__restrict__ orow = out + ((int64_t)b * wc_total + wc_off + c0 + c) * np;
                T x[V][KK];
#pragma unroll
                for (int v = 0; v < V; ++v)
#pragma unroll
                    for (int i = 0; i < KK; ++i)
                        x[v][i] = row[src[v][i]];
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    T val = x[v][0];
                    if (HAS_W) {
                        // out = 0; out = fma(in, w, out) per neighbour, in slot order
                        // (interpolate_kernel.cu:31-42 under default contraction).
                        val = (T)0;
#pragma unroll
                        for (int i = 0; i < KK; ++i)
                            val = tk_fma<T>(x[v][i], wt[v][i], val);
                    }
                    __builtin_nontemporal_store(val, &orow[p0 + v * 64]);
                }
            }
            continue;
        }
#pragma unroll 4
        for (int c = 0; c < nc; ++c) {
            const T *row = rows + c * n1;
            T *__restrict__ orow = out + ((int64_t)b * wc_total + wc_off + c0 + c) * np;
#pragma unroll
            for (int v = 0; v < V; ++v) {
                T val;
                if (HAS_W) {
                    // out = 0; out = fma(in, w, out) per neighbour, in slot order
                    // (interpolate_kernel.cu:31-42 under default contraction).
                    T acc = (T)0;
#pragma unroll
                    for (int i = 0; i < KK; ++i)
                        if (src[v][i] >= 0)
                            acc = tk_fma<T>(row[src[v][i]], wt[v][i], acc);
                    val = acc;
                } else {
                    val = src[v][0] >= 0 ? row[src[v][0]] : (T)0;
                }
                if (p0 + v * 64 < pe)
                    __builtin_nontemporal_store(val, &orow[p0 + v * 64]);
            }
        }
    }
}

// ---- scatter ---------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(GS_BLOCK) void fill_zero_kernel(T *__restrict__ p, int64_t n)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        p[i] = (T)0;
}

// Streams the points [ps, pe) of one batch for `nc` channels starting at c0 and hands
// every contribution whose destination lies in [d0, d0 + nr) to
// `sink(ctx, c, dst - d0, value, weight)`, where `ctx = prep(c)` is evaluated once per
// channel and lane iteration. A lane takes V points 64 apart,
// and the channel loop is unrolled to keep several loads in flight.
template <typename T, int KK, bool HAS_W, int V, int NT, typename Prep, typename Sink>
__device__ __forceinline__ void scatter_stream(const T *__restrict__ gout,
                                               const int64_t *__restrict__ idx,
                                               const T *__restrict__ w, int b, int wc_total,
                                               int c0, int nc, int d0, int nr, int64_t np,
                                               int64_t ps, int64_t pe, int vec_ok, Prep prep,
                                               Sink sink)
{
    (void)vec_ok;
    // A wave covers 64*V consecutive points, lane l the points l, l+64, ...: every load
    // of the wave is a run of consecutive elements (24-byte stride for the indices of
    // three neighbours).
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    for (int64_t p0 = ps + (int64_t)wave * (64 * V) + lane; p0 < pe; p0 += (int64_t)NT * V) {
        int dst[V][KK];
        T wt[V][KK];
#pragma unroll
        for (int v = 0; v < V; ++v) {
#pragma unroll
            for (int i = 0; i < KK; ++i) {
                const int64_t p = p0 + v * 64;
                int64_t j = -1;
                T ww = (T)1;
                if (p < pe) {
                    j = idx[((int64_t)b * np + p) * KK + i];
                    if (HAS_W)
                        ww = w[((int64_t)b * np + p) * KK + i];
                }
                dst[v][i] = (j >= d0 && j < (int64_t)d0 + nr) ? (int)(j - d0) : -1;
                wt[v][i] = ww;
            }
        }
#pragma unroll 4
        for (int c = 0; c < nc; ++c) {
            const T *__restrict__ grow = gout + ((int64_t)b * wc_total + c0 + c) * np;
            T g[V];
#pragma unroll
            for (int v = 0; v < V; ++v)
                g[v] = (p0 + v * 64 < pe) ? grow[p0 + v * 64] : (T)0;
            const auto ctx = prep(c);
#pragma unroll
            for (int v = 0; v < V; ++v)
#pragma unroll
                for (int i = 0; i < KK; ++i)
                    if (dst[v][i] >= 0)
                        sink(ctx, c, dst[v][i], g[v], wt[v][i]);
        }
    }
}

// LDS-resident destination rows with floating-point LDS atomics.
// grid = (segments, channel groups, B).
template <typename T, int KK, bool HAS_W, int V, int NT>
__global__ __launch_bounds__(NT) void scatter_lds_kernel(
    const T *__restrict__ gout, const int64_t *__restrict__ idx, const T *__restrict__ w,
    T *__restrict__ gin, int c_total, int wc_total, int wc_off, int n1, int64_t np, int cg, int64_t seg_len,
    int merge_with_atomics, int vec_ok)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *rows = reinterpret_cast<T *>(smem_raw);  // [cg][n1]
    const int b = blockIdx.z;
    const int c0 = blockIdx.y * cg;
    const int nc = (c0 + cg < c_total) ? cg : c_total - c0;
    const int64_t ps = (int64_t)blockIdx.x * seg_len;
    const int64_t pe = (ps + seg_len < np) ? ps + seg_len : np;

    for (int i = threadIdx.x; i < nc * n1; i += NT)
        rows[i] = (T)0;
    __syncthreads();
    scatter_stream<T, KK, HAS_W, V, NT>(
        gout, idx, w, b, wc_total, c0 + wc_off, nc, 0, n1, np, ps, pe, vec_ok,
        [](int) { return 0; },
        [&](int, int c, int dst, T g, T ww) { atomicAdd(&rows[c * n1 + dst], HAS_W ? g * ww : g); });
    __syncthreads();

    T *__restrict__ dstrows = gin + ((int64_t)b * c_total + c0) * n1;
    if (merge_with_atomics) {
        for (int i = threadIdx.x; i < nc * n1; i += NT) {
            const T v = rows[i];
            if (v != (T)0)
                unsafeAtomicAdd(&dstrows[i], v);
        }
    } else {
        for (int i = threadIdx.x; i < nc * n1; i += NT)
            dstrows[i] = rows[i];
    }
}

// fp32 scatter with 64-bit fixed-point accumulators in LDS.
//
// Floating-point LDS atomics on this GPU retire about one lane every three clocks
// (measured: 195 clocks per wave instruction, conflicts or not); integer LDS
// atomics run at the rate of a plain LDS write, 13 times faster. So each
// contribution g*w (rounded to fp32 as the reference rounds it) is converted to an
// integer at a per-row power-of-two scale and added with ds_add_u64:
//   * magnitudes: the workgroup samples an eighth of its share of gout for max|g| per
//     row and an eighth of w for max|w| (runs of 64 consecutive loads, one run in
//     eight), and allows 8 times their product as the bound B_c of a row;
//   * scale: 2^k with k the largest integer keeping B_c * 2^k below 2^50 and
//     count * B_c * 2^k below 2^62, i.e. one term is resolved to 2^-43 of the row's
//     largest term or better for up to 2^16 terms per row. The resolution is absolute
//     within a row where fp32 accumulation's is relative to each sum: a row whose
//     terms span more than 2^20 resolves its small sums worse than fp32 would;
//   * conversion: fma(double(term), 2^k, 1.5 * 2^52) leaves the rounded integer in
//     the low mantissa bits (one cvt, one fma, one 64-bit subtract);
//   * a term above its row's bound (the sample missed an outlier) raises a flag;
//     the workgroup then repeats the pass with bounds from the full data.
// Integer addition is associative, so unlike the reference the result does not
// depend on the order in which the contributions arrive. A row holding NaN or inf
// has no usable scale; the workgroup then takes the floating-point path.
// Largest value of a wave, in every lane. Called by whole waves only.
__device__ __forceinline__ unsigned wave_max_u32(unsigned v)
{
    // within rows of 16 lanes through the data-parallel-primitive lane selects (lane ^ 1,
    // lane ^ 2, mirrored in 8, mirrored in 16), then the four rows through scalar registers
    auto fold = [&](auto ctrl) {
        const unsigned t =
            (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, decltype(ctrl)::value, 0xf, 0xf, false);
        v = t > v ? t : v;
    };
    fold(std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
    fold(std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
    fold(std::integral_constant<int, 0x141>{});  // row_half_mirror
    fold(std::integral_constant<int, 0x140>{});  // row_mirror
    const unsigned r0 = (unsigned)__builtin_amdgcn_readlane((int)v, 0);
    const unsigned r1 = (unsigned)__builtin_amdgcn_readlane((int)v, 16);
    const unsigned r2 = (unsigned)__builtin_amdgcn_readlane((int)v, 32);
    const unsigned r3 = (unsigned)__builtin_amdgcn_readlane((int)v, 48);
    const unsigned a = r0 > r1 ? r0 : r1, b = r2 > r3 ? r2 : r3;
    return a > b ? a : b;
}


template <int CGMAX>
struct ScatterFixedShared {
    unsigned maxg[CGMAX];  // bit patterns of non-negative floats order as integers
    unsigned maxw;
    int kexp[CGMAX];
    double scale[CGMAX];
    float bound[CGMAX];
    int finite, exceeded;
};

// Workgroups are handed to the 8 XCDs round-robin by linear id. Every workgroup of a
// batch streams that batch's index and weight arrays, so each XCD takes a contiguous
// range of logical workgroups (batch slowest): a batch's arrays then come from HBM
// once and from one XCD's L2 afterwards, instead of once per XCD.
__device__ __forceinline__ void scatter_fixed_block(int &b, int &by, int &bx)
{
    const unsigned long long gx = gridDim.x, gyy = gridDim.y;
    const unsigned long long total = gx * gyy * gridDim.z;
    unsigned long long lin = blockIdx.x + gx * (blockIdx.y + gyy * blockIdx.z);
    const unsigned long long per = total >> 3, full = per << 3;
    if (lin < full)
        lin = (lin & 7ull) * per + (lin >> 3);
    const unsigned long long rest = lin / gx;
    bx = (int)(lin - rest * gx);
    by = (int)(rest % gyy);
    b = (int)(rest / gyy);
}

// Clears `acc_elems` accumulators and the shared magnitudes; barriers before and after.
template <bool HAS_W, int NT, int CGMAX>
__device__ __forceinline__ void scatter_fixed_clear(ScatterFixedShared<CGMAX> &sh,
                                                    unsigned long long *acc, int acc_elems)
{
    __syncthreads();
    for (int i = threadIdx.x; i < acc_elems; i += NT)
        acc[i] = 0ull;
    if (threadIdx.x < CGMAX)
        sh.maxg[threadIdx.x] = 0u;
    if (threadIdx.x == 0) {
        sh.finite = 1;
        sh.exceeded = 0;
        sh.maxw = HAS_W ? 0u : 0x3f800000u;
    }
    __syncthreads();
}

// Bound and scale of each row from the magnitudes in sh.maxg / sh.maxw, which came from a
// sample (`headroom` 8) or from all the data (just above 1); barriers before and after.
// sh.finite tells whether every bound is a finite number.
template <int CGMAX>
__device__ __forceinline__ void scatter_fixed_scales(ScatterFixedShared<CGMAX> &sh,
                                                     float headroom, int log2_count)
{
    __syncthreads();
    if (threadIdx.x < CGMAX) {  // lane c works out row c
        const float maxw = __builtin_bit_cast(float, sh.maxw);
        const float bound = __builtin_bit_cast(float, sh.maxg[threadIdx.x]) * maxw * headroom;
        if (!(bound < 3.0e38f))  // NaN or inf (NaN has the largest bit pattern)
            sh.finite = 0;
        int e = 0;
        (void)__builtin_frexpf(bound, &e);  // bound < 2^e (bound == 0 gives e = 0)
        // one term stays below 2^50 (the conversion is exact to 2^51) and the sum of
        // `count` terms below 2^62
        sh.kexp[threadIdx.x] = (62 - log2_count < 50 ? 62 - log2_count : 50) - e;
        sh.scale[threadIdx.x] = __builtin_ldexp(1.0, sh.kexp[threadIdx.x]);
        sh.bound[threadIdx.x] = bound;
    }
    __syncthreads();
}

// Clears `acc_elems` accumulators and works out the bound and scale of each of the `nc`
// rows starting at row `row0` of batch b (points [ps, pe)): from a sample on attempt 0
// (every 8th run of 64 loads, 8 times headroom), from all the data on attempt 1. Ends
// with a barrier; sh.finite tells whether every bound is a finite number.
template <int KK, bool HAS_W, int NT, int CGMAX>
__device__ __forceinline__ void scatter_fixed_prepare(
    ScatterFixedShared<CGMAX> &sh, unsigned long long *acc, int acc_elems, int attempt,
    const float *__restrict__ gout, const float *__restrict__ w, int b, int wc_total, int row0,
    int nc, int64_t np, int64_t ps, int64_t pe, int vec_ok, int log2_count)
{
    constexpr int V = 4;  // points per 16-byte load of the sampler
    scatter_fixed_clear<HAS_W, NT, CGMAX>(sh, acc, acc_elems);

    if (HAS_W) {
        // first attempt: one run of 64 consecutive weights in every 512
        unsigned mw = 0u;
        const int64_t ne = (pe - ps) * KK;
        for (int64_t t = threadIdx.x;; t += NT) {
            const int64_t e = attempt == 0 ? (t >> 6) * 512 + (t & 63) : t;
            if (e >= ne)
                break;
            const unsigned bits =
                __builtin_bit_cast(unsigned, w[((int64_t)b * np + ps) * KK + e]) & 0x7fffffffu;
            mw = bits > mw ? bits : mw;
        }
        // one LDS atomic per wave: 64 lanes on one address would be served one by one
        mw = wave_max_u32(mw);
        if ((threadIdx.x & 63) == 0 && mw != 0u)
            atomicMax(&sh.maxw, mw);
    }
    {
        // first attempt: one run of 64 consecutive 16-byte groups in every 512
        unsigned mg[CGMAX];
#pragma unroll
        for (int c = 0; c < CGMAX; ++c)
            mg[c] = 0u;
        for (int64_t t = threadIdx.x;; t += NT) {
            const int64_t gi = attempt == 0 ? (t >> 6) * 512 + (t & 63) : t;
            const int64_t p0 = ps + gi * V;
            if (p0 >= pe)
                break;
            const bool full = (p0 + V <= pe);
#pragma unroll
            for (int c = 0; c < CGMAX; ++c) {
                if (c >= nc)
                    break;
                const float *__restrict__ grow = gout + ((int64_t)b * wc_total + row0 + c) * np;
                float g[V];
                if (full && vec_ok) {
                    const float4 pack = *reinterpret_cast<const float4 *>(grow + p0);
                    g[0] = pack.x;
                    g[1] = pack.y;
                    g[2] = pack.z;
                    g[3] = pack.w;
                } else {
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        g[v] = (p0 + v < pe) ? grow[p0 + v] : 0.0f;
                }
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    const unsigned bits = __builtin_bit_cast(unsigned, g[v]) & 0x7fffffffu;
                    mg[c] = bits > mg[c] ? bits : mg[c];
                }
            }
        }
#pragma unroll
        for (int c = 0; c < CGMAX; ++c) {
            if (c >= nc)  // uniform
                break;
            const unsigned m = wave_max_u32(mg[c]);
            if ((threadIdx.x & 63) == 0 && m != 0u)
                atomicMax(&sh.maxg[c], m);
        }
    }
    scatter_fixed_scales<CGMAX>(sh, attempt == 0 ? 8.0f : 1.000001f, log2_count);
}

// Rows of fixed-point sums back to fp32 and out to memory; `stride` accumulators per row
// in LDS, the first `nr` of them destinations d0, d0 + 1, ...
template <int NT, int CGMAX>
__device__ __forceinline__ void scatter_fixed_write(const ScatterFixedShared<CGMAX> &sh,
                                                    const unsigned long long *acc, int stride,
                                                    float *__restrict__ gin, int64_t row0,
                                                    int nc, int n1, int d0, int nr,
                                                    int merge_with_atomics)
{
    for (int c = 0; c < nc; ++c) {
        float *__restrict__ dstrow = gin + (row0 + c) * n1 + d0;
        const unsigned long long *__restrict__ row = acc + c * stride;
        const int kexp = sh.kexp[c];
        for (int i = threadIdx.x; i < nr; i += NT) {
            const float v = (float)__builtin_ldexp((double)(long long)row[i], -kexp);
            if (merge_with_atomics) {
                if (v != 0.0f)
                    unsafeAtomicAdd(&dstrow[i], v);
            } else {
                dstrow[i] = v;
            }
        }
    }
}

// The general procedure for the destinations [d0, d0 + nr) of rows c0 .. c0 + nc - 1 of
// batch b: attempts `first_attempt` .. 1 in fixed point, then floating point.
template <int KK, bool HAS_W, int V, int NT, int CGMAX>
__device__ __forceinline__ void scatter_fixed_attempts(
    ScatterFixedShared<CGMAX> &sh, unsigned char *smem_raw, int first_attempt,
    const float *__restrict__ gout, const int64_t *__restrict__ idx,
    const float *__restrict__ w, float *__restrict__ gin, int b, int c_total, int wc_total,
    int wc_off, int c0, int nc, int n1, int d0, int nr, int64_t np, int64_t ps, int64_t pe,
    int merge_with_atomics, int vec_ok, int log2_count)
{
    unsigned long long *acc = reinterpret_cast<unsigned long long *>(smem_raw);  // [nc][nr]
    const double MAGIC = 6755399441055744.0;  // 1.5 * 2^52
    for (int attempt = first_attempt; attempt < 2; ++attempt) {  // uniform over the workgroup
        scatter_fixed_prepare<KK, HAS_W, NT, CGMAX>(sh, acc, nc * nr, attempt, gout, w, b,
                                                    wc_total, wc_off + c0, nc, np, ps, pe,
                                                    vec_ok, log2_count);
        if (!sh.finite)
            break;
        struct RowScale {
            double scale;
            float bound;
        };
        bool exceeded = false;
        scatter_stream<float, KK, HAS_W, V, NT>(
            gout, idx, w, b, wc_total, c0 + wc_off, nc, d0, nr, np, ps, pe, vec_ok,
            [&](int c) {
                RowScale r;
                r.scale = sh.scale[c];
                r.bound = sh.bound[c];
                return r;
            },
            [&](const RowScale &r, int c, int dst, float g, float ww) {
                const float term = HAS_W ? g * ww : g;
                exceeded = exceeded || !(__builtin_fabsf(term) <= r.bound);  // also NaN
                const double d = __builtin_fma((double)term, r.scale, MAGIC);
                const unsigned long long q = __builtin_bit_cast(unsigned long long, d) -
                                             __builtin_bit_cast(unsigned long long, MAGIC);
                atomicAdd(&acc[c * nr + dst], q);
            });
        if (exceeded)
            sh.exceeded = 1;
        __syncthreads();
        if (!sh.exceeded) {
            scatter_fixed_write<NT, CGMAX>(sh, acc, nr, gin, (int64_t)b * c_total + c0, nc, n1,
                                           d0, nr, merge_with_atomics);
            return;
        }
    }

    // ---- non-finite input: floating-point accumulation in the same LDS ----
    float *rows = reinterpret_cast<float *>(smem_raw);
    __syncthreads();
    for (int i = threadIdx.x; i < nc * nr; i += NT)
        rows[i] = 0.0f;
    __syncthreads();
    scatter_stream<float, KK, HAS_W, V, NT>(
        gout, idx, w, b, wc_total, c0 + wc_off, nc, d0, nr, np, ps, pe, vec_ok,
        [](int) { return 0; },
        [&](int, int c, int dst, float g, float ww) {
            atomicAdd(&rows[c * nr + dst], HAS_W ? g * ww : g);
        });
    __syncthreads();
    for (int c = 0; c < nc; ++c) {
        float *__restrict__ dstrow = gin + ((int64_t)b * c_total + c0 + c) * n1 + d0;
        for (int i = threadIdx.x; i < nr; i += NT) {
            const float v = rows[c * nr + i];
            if (merge_with_atomics) {
                if (v != 0.0f)
                    unsafeAtomicAdd(&dstrow[i], v);
            } else {
                dstrow[i] = v;
            }
        }
    }
}

// Any number of neighbours, rows of any length (in windows of destinations).
// grid = (segments, windows * channel groups, B).
template <int KK, bool HAS_W, int V, int NT, int CGMAX>
__global__ __launch_bounds__(NT) void scatter_fixed_kernel(
    const float *__restrict__ gout, const int64_t *__restrict__ idx,
    const float *__restrict__ w, float *__restrict__ gin, int c_total, int wc_total, int wc_off, int n1, int64_t np, int cg,
    int64_t seg_len, int merge_with_atomics, int vec_ok, int log2_count, int groups, int window)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    __shared__ ScatterFixedShared<CGMAX> sh;
    int b, by, bx;
    scatter_fixed_block(b, by, bx);
    // by = destination window * groups + channel group; a workgroup accumulates the
    // destinations [d0, d0 + nr) of its channels (the whole row when it fits in LDS)
    const int win = by / groups;
    const int c0 = (by - win * groups) * cg;
    const int nc = (c0 + cg < c_total) ? cg : c_total - c0;
    const int d0 = win * window;
    const int nr = (d0 + window < n1) ? window : n1 - d0;
    const int64_t ps = (int64_t)bx * seg_len;
    const int64_t pe = (ps + seg_len < np) ? ps + seg_len : np;
    scatter_fixed_attempts<KK, HAS_W, V, NT, CGMAX>(sh, smem_raw, 0, gout, idx, w, gin, b, c_total,
                                                    wc_total, wc_off, c0, nc, n1, d0, nr, np, ps,
                                                    pe, merge_with_atomics, vec_ok, log2_count);
}

// A value every lane holds, moved to scalar registers.
__device__ __forceinline__ double scatter_uniform(double v)
{
    const unsigned long long bits = __builtin_bit_cast(unsigned long long, v);
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)bits);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(bits >> 32));
    return __builtin_bit_cast(double, ((unsigned long long)hi << 32) | lo);
}

// Whole rows in LDS, the shapes the layers produce (one neighbour without weights, three
// with). The general kernel above spends its time waiting: every contribution sits in a
// branch of its own behind a wait for all loads and all LDS traffic in flight, and each
// workgroup pays the latencies of clearing, sampling, streaming and writing one after the
// other. Here:
//   * a wave takes a run of consecutive chunks of 64 * V points, lane l the points l,
//     l + 64, ... of a chunk. The indices, weights and the values of all rows for the
//     next chunk are requested before the current chunk is accumulated; the loop over a
//     chunk has no branch and no wait on LDS;
//   * a lane past the end of the points, or an index outside the row, adds into a spare
//     accumulator of its lane behind the row (64 per row, never read) instead of being
//     skipped;
//   * the first chunk of every wave doubles as the sample for the magnitudes (runs of
//     64 * V points spread evenly over the points), so no separate sampling pass;
//   * instead of comparing every term with the bound of its row, a lane keeps the largest
//     |value| per row and the largest |weight| it has seen and compares their product at
//     the end (NaN and inf have the largest bit patterns). That is stricter than the
//     term-by-term test, so a pass may be repeated where the general kernel would not
//     repeat it; a pass that is kept adds exactly the same integers;
//   * a workgroup works through several jobs (a job = the rows of one channel group of
//     one batch over one segment of points). Writing a job's rows out also clears the
//     accumulators, and the first chunks of the next job are requested before that, so
//     clearing and the first trip to memory cost nothing from the second job on.
// A repeated pass, and rows with NaN or inf, take the general procedure.
// grid = (workgroups); jobs = segments * channel groups * B, job j of `gx * gy * gz` has
// x fastest; LDS = cg * (n1 + 64) accumulators.
template <int KK, bool HAS_W, int NT, int CG, int V>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 4))) void
scatter_fixed_rows_kernel(const float *__restrict__ gout, const int64_t *__restrict__ idx,
                          const float *__restrict__ w, float *__restrict__ gin, int c_total,
                          int wc_total, int wc_off, int n1, int64_t np, int cg, int64_t seg_len,
                          int merge_with_atomics, int vec_ok, int log2_count, unsigned gx,
                          unsigned gy, unsigned gz)
{
    constexpr int NW = NT / 64, SPARE = 64;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    unsigned long long *acc = reinterpret_cast<unsigned long long *>(smem_raw);
    __shared__ ScatterFixedShared<CG> sh;
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int stride = n1 + SPARE;

    // Workgroups go to the 8 XCDs round-robin by id. Every job of a batch streams that
    // batch's index and weight arrays, so each XCD takes a contiguous range of the jobs
    // (batch slowest) and a batch's arrays come from HBM once, then from one XCD's L2.
    const unsigned total = gx * gy * gz;
    unsigned job, job_end, job_step;
    if (gridDim.x % 8 == 0 && total % 8 == 0) {
        const unsigned per = total / 8, x = blockIdx.x & 7;
        job = x * per + (blockIdx.x >> 3);
        job_end = (x + 1) * per;
        job_step = gridDim.x >> 3;
    } else {
        job = blockIdx.x;
        job_end = total;
        job_step = gridDim.x;
    }

    // what a lane has asked for and not yet used: one chunk of indices, weights and values
    struct Stage {
        int64_t j[V][KK];
        float w[V][KK], g[CG][V];
    };
    struct Job {
        int b, c0, nc;
        int64_t ps;
        unsigned len, first, last;  // points, and this wave's chunks [first, last)
        const float *gbase, *wbase;
        const int64_t *ibase;
    };
    auto decode = [&](unsigned j) {
        Job jb;
        const unsigned rest = j / gx;
        const int bx = (int)(j - rest * gx);
        jb.b = (int)(rest / gy);
        jb.c0 = (int)(rest % gy) * cg;
        jb.nc = (jb.c0 + cg < c_total) ? cg : c_total - jb.c0;
        jb.ps = (int64_t)bx * seg_len;
        const int64_t pe = (jb.ps + seg_len < np) ? jb.ps + seg_len : np;
        jb.len = (unsigned)(pe - jb.ps);  // the host keeps len * KK below 2^31
        const unsigned nchunks = (jb.len + 64 * V - 1) / (64 * V);
        const unsigned per_wave = (nchunks + NW - 1) / NW;
        jb.first = wave * per_wave;
        jb.last = jb.first + per_wave < nchunks ? jb.first + per_wave : nchunks;
        jb.gbase = gout + ((int64_t)jb.b * wc_total + wc_off + jb.c0) * np + jb.ps;
        jb.ibase = idx + ((int64_t)jb.b * np + jb.ps) * KK;
        jb.wbase = HAS_W ? w + ((int64_t)jb.b * np + jb.ps) * KK : nullptr;
        return jb;
    };
    auto request = [&](Stage &st, const Job &jb, unsigned chunk) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            unsigned po = chunk * (64 * V) + v * 64 + lane;
            po = po < jb.len ? po : jb.len - 1;
            if constexpr (KK == 3) {
                // a point's three indices and three weights as one run each (a 16-byte and an
                // 8-byte load, a 12-byte load): loaded one element at a time, a wave's
                // request touches every cache line of the run three times
                struct __attribute__((aligned(8))) Idx3 { int64_t a, b, c; };
                struct __attribute__((aligned(4))) W3 { float a, b, c; };
                const Idx3 ji = *reinterpret_cast<const Idx3 *>(jb.ibase + (int64_t)po * 3);
                st.j[v][0] = ji.a;
                st.j[v][1] = ji.b;
                st.j[v][2] = ji.c;
                if constexpr (HAS_W) {
                    const W3 wi = *reinterpret_cast<const W3 *>(jb.wbase + (int64_t)po * 3);
                    st.w[v][0] = wi.a;
                    st.w[v][1] = wi.b;
                    st.w[v][2] = wi.c;
                } else {
                    st.w[v][0] = st.w[v][1] = st.w[v][2] = 1.0f;
                }
            } else {
#pragma unroll
                for (int i = 0; i < KK; ++i) {
                    st.j[v][i] = jb.ibase[po * KK + i];
                    st.w[v][i] = HAS_W ? jb.wbase[po * KK + i] : 1.0f;
                }
            }
#pragma unroll
            for (int c = 0; c < CG; ++c)
                if (c < jb.nc)  // uniform
                    st.g[c][v] = (jb.gbase + (int64_t)c * np)[po];
        }
    };

    Stage sa;
    bool prepared = false;  // accumulators are zero and the first chunk is on its way
    for (; job < job_end; job += job_step) {
        const Job jb = decode(job);
        const int nc = jb.nc;
        if (!prepared) {
            if (jb.first < jb.last)
                request(sa, jb, jb.first);
            scatter_fixed_clear<HAS_W, NT, CG>(sh, acc, cg * stride);
        } else {
            // the barrier that ended the last job's writing is behind us
            if (threadIdx.x < CG)
                sh.maxg[threadIdx.x] = 0u;
            if (threadIdx.x == 0) {
                sh.finite = 1;
                sh.exceeded = 0;
                sh.maxw = HAS_W ? 0u : 0x3f800000u;
            }
            __syncthreads();
        }
        prepared = false;
        // magnitudes from the first chunk of every wave
        if (jb.first < jb.last) {
            if (HAS_W) {
                unsigned mw = 0u;
#pragma unroll
                for (int v = 0; v < V; ++v)
#pragma unroll
                    for (int i = 0; i < KK; ++i) {
                        const unsigned bits = __builtin_bit_cast(unsigned, sa.w[v][i]) & 0x7fffffffu;
                        mw = bits > mw ? bits : mw;
                    }
                mw = wave_max_u32(mw);
                if (lane == 0 && mw != 0u)
                    atomicMax(&sh.maxw, mw);
            }
#pragma unroll
            for (int c = 0; c < CG; ++c) {
                if (c >= nc)  // uniform
                    break;
                unsigned m = 0u;
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    const unsigned bits = __builtin_bit_cast(unsigned, sa.g[c][v]) & 0x7fffffffu;
                    m = bits > m ? bits : m;
                }
                m = wave_max_u32(m);
                if (lane == 0 && m != 0u)
                    atomicMax(&sh.maxg[c], m);
            }
        }
        scatter_fixed_scales<CG>(sh, 8.0f, log2_count);
        bool done = false;
        if (sh.finite) {
            const double MAGIC = 6755399441055744.0;  // 1.5 * 2^52
            double scale[CG];
#pragma unroll
            for (int c = 0; c < CG; ++c)
                scale[c] = scatter_uniform(sh.scale[c < nc ? c : 0]);
            unsigned gbits[CG];
#pragma unroll
            for (int c = 0; c < CG; ++c)
                gbits[c] = 0u;
            unsigned wbits = HAS_W ? 0u : 0x3f800000u;
            for (unsigned chunk = jb.first; chunk < jb.last; ++chunk) {
                // copy the chunk out of `sa`, ask for the next one into it, accumulate
                unsigned slot[V][KK];
                float wt[V][KK], g[CG][V];
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    const bool inside = chunk * (64 * V) + v * 64 + lane < jb.len;
#pragma unroll
                    for (int i = 0; i < KK; ++i) {
                        const int64_t j = sa.j[v][i];
                        slot[v][i] = (inside && (unsigned long long)j < (unsigned long long)n1)
                                         ? (unsigned)j
                                         : (unsigned)n1 + lane;
                        wt[v][i] = sa.w[v][i];
                        if (HAS_W) {
                            const unsigned bits =
                                __builtin_bit_cast(unsigned, wt[v][i]) & 0x7fffffffu;
                            wbits = bits > wbits ? bits : wbits;
                        }
                    }
#pragma unroll
                    for (int c = 0; c < CG; ++c)
                        g[c][v] = sa.g[c][v];
                }
                if (chunk + 1 < jb.last)  // uniform
                    request(sa, jb, chunk + 1);
#pragma unroll
                for (int c = 0; c < CG; ++c) {
                    if (c >= nc)  // uniform
                        break;
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        const unsigned bits = __builtin_bit_cast(unsigned, g[c][v]) & 0x7fffffffu;
                        gbits[c] = bits > gbits[c] ? bits : gbits[c];
#pragma unroll
                        for (int i = 0; i < KK; ++i) {
                            const float term = HAS_W ? g[c][v] * wt[v][i] : g[c][v];
                            const double d = __builtin_fma((double)term, scale[c], MAGIC);
                            const unsigned long long q =
                                __builtin_bit_cast(unsigned long long, d) -
                                __builtin_bit_cast(unsigned long long, MAGIC);
                            atomicAdd(&acc[(unsigned)c * (unsigned)stride + slot[v][i]], q);
                        }
                    }
                }
            }
            bool exceeded = false;
#pragma unroll
            for (int c = 0; c < CG; ++c)
                if (c < nc)
                    exceeded = exceeded || !(__builtin_bit_cast(float, gbits[c]) *
                                                 __builtin_bit_cast(float, wbits) <=
                                             sh.bound[c]);  // also NaN
            if (exceeded)
                sh.exceeded = 1;
            __syncthreads();
            done = !sh.exceeded;
        }
        const bool more = job + job_step < job_end;
        if (done) {
            // the next job's first chunks fly while this job's rows are written and cleared
            if (more) {
                const Job nx = decode(job + job_step);
                if (nx.first < nx.last)
                    request(sa, nx, nx.first);
                prepared = true;
            }
            for (int c = 0; c < nc; ++c) {
                float *__restrict__ dstrow = gin + ((int64_t)jb.b * c_total + jb.c0 + c) * n1;
                unsigned long long *__restrict__ row = acc + c * stride;
                const int kexp = sh.kexp[c];
                constexpr int U = 4;  // accumulators fetched together
                for (int i0 = threadIdx.x; i0 < n1; i0 += NT * U) {
                    unsigned long long q[U];
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        q[u] = i0 + u * NT < n1 ? row[i0 + u * NT] : 0ull;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int i = i0 + u * NT;
                        if (i >= n1)
                            break;
                        row[i] = 0ull;
                        // (double)(long long)q in one rounding: high word times 2^32 is exact
                        const double d = __builtin_fma((double)(int)(unsigned)(q[u] >> 32),
                                                       4294967296.0, (double)(unsigned)q[u]);
                        const float v = (float)__builtin_ldexp(d, -kexp);
                        if (merge_with_atomics) {
                            if (v != 0.0f)
                                unsafeAtomicAdd(&dstrow[i], v);
                        } else {
                            dstrow[i] = v;
                        }
                    }
                }
            }
            __syncthreads();
        } else {
            const int64_t pe = jb.ps + jb.len;
            scatter_fixed_attempts<KK, HAS_W, 4, NT, CG>(sh, smem_raw, 1, gout, idx, w, gin, jb.b,
                                                         c_total, wc_total, wc_off, jb.c0, nc, n1,
                                                         0, n1, np, jb.ps, pe, merge_with_atomics,
                                                         vec_ok, log2_count);
        }
    }
}

// The kernel above as a type, for the launch helper of the host code.
template <int KK, bool HAS_W, int NT, int CG, int V>
using ScatterRowsKernel =
    std::integral_constant<decltype(&scatter_fixed_rows_kernel<KK, HAS_W, NT, CG, V>),
                           &scatter_fixed_rows_kernel<KK, HAS_W, NT, CG, V>>;

// Rows too long for LDS: one global atomic per contribution into a zero-filled
// output.
template <typename T, int KK, bool HAS_W>
__global__ __launch_bounds__(GS_BLOCK) void scatter_global_kernel(
    const T *__restrict__ gout, const int64_t *__restrict__ idx, const T *__restrict__ w,
    T *__restrict__ gin, int c_total, int wc_total, int wc_off, int n1, int64_t np, int cg)
{
    const int b = blockIdx.z;
    const int c0 = blockIdx.y * cg;
    const int c1 = (c0 + cg < c_total) ? c0 + cg : c_total;
    const int64_t p = (int64_t)blockIdx.x * GS_BLOCK + threadIdx.x;
    if (p >= np)
        return;
    int dst[KK];
    T wt[KK];
#pragma unroll
    for (int i = 0; i < KK; ++i) {
        const int64_t j = idx[((int64_t)b * np + p) * KK + i];
        dst[i] = (j >= 0 && j < n1) ? (int)j : -1;
        wt[i] = HAS_W ? w[((int64_t)b * np + p) * KK + i] : (T)1;
    }
    for (int c = c0; c < c1; ++c) {
        const T g = gout[((int64_t)b * wc_total + wc_off + c) * np + p];
        T *row = gin + ((int64_t)b * c_total + c) * n1;
#pragma unroll
        for (int i = 0; i < KK; ++i)
            if (dst[i] >= 0)
                unsafeAtomicAdd(&row[dst[i]], HAS_W ? g * wt[i] : g);
    }
}

// ---- host ------------------------------------------------------------------------------

int check_shape(int64_t B, int64_t C, int64_t N1, int64_t NP, int64_t KK)
{
    if (B < 0 || C < 0 || N1 < 0 || NP < 0 || KK < 0)
        return TK3D_ERR_BAD_SIZE;
    if (N1 > TK_MAX_I32 / 4 || C > TK_MAX_I32 / 4 || B > 65535 ||
        !tk_fits(TK_MAX_ELEMS, B, C, N1) || !tk_fits(TK_MAX_ELEMS, B, C, NP) ||
        !tk_fits(TK_MAX_ELEMS, B, NP, KK > 0 ? KK : 1))
        return TK3D_ERR_UNSUPPORTED;
    return TK3D_OK;
}

template <typename T, int KK, bool HAS_W>
int gather(const T *in, const int64_t *idx, const T *w, int64_t B, int64_t C, int64_t N1,
           int64_t NP, T *out, hipStream_t s, int64_t wc_total = -1, int64_t wc_off = 0)
{
    // The output may be a channel slice [wc_off, wc_off + C) of a tensor with wc_total
    // channels (same B and NP); by default it is exactly [B, C, NP].
    if (wc_total < 0)
        wc_total = C;
    if (B * C * NP == 0)
        return TK3D_OK;
    if (!in && N1 > 0)
        return TK3D_ERR_NULL_POINTER;
    if (!idx || !out || (HAS_W && !w))
        return TK3D_ERR_NULL_POINTER;
    constexpr int V = (sizeof(T) == 4) ? 4 : 2;
    // 16-byte stores need every output row to start on a 16-byte boundary.
    const int vec_ok = (((uintptr_t)out & 15) == 0) && ((NP * (int64_t)sizeof(T)) % 16 == 0);

    // Rows are staged in LDS: up to 64 KiB per workgroup (two workgroups per CU), or one
    // row of up to 128 KiB when a row alone is longer than that (32768 fp32 elements).
    const int64_t row_bytes = N1 * (int64_t)sizeof(T);
    const int64_t LDS_BUDGET = row_bytes > 64 * 1024 ? 128 * 1024 : 64 * 1024;
    if (row_bytes > 0 && row_bytes <= LDS_BUDGET && NP >= 1024) {
        constexpr int NT = 512;
        int cg = 8;
        while (cg > 1 && (cg * row_bytes > LDS_BUDGET || cg > C))
            cg /= 2;
        if (cg * row_bytes > 48 * 1024) {
            const int allowed =
                tk_allow_dynamic_lds<gather_lds_kernel<T, KK, HAS_W, V, NT>>(128 * 1024);
            if (allowed != TK3D_OK)
                return allowed;
        }
        const int64_t gy = (C + cg - 1) / cg;
        // Split the points until the chip is full; every chunk re-stages its rows, so
        // keep a chunk well above the staged size.
        int64_t chunks = 1;
        const int64_t min_chunk = (int64_t)NT * V * 4;
        while (B * gy * chunks < 512 && NP / (chunks * 2) >= min_chunk &&
               (NP / (chunks * 2)) * KK >= (cg * N1) / 2)
            chunks *= 2;
        int64_t chunk_len = (NP + chunks - 1) / chunks;
        chunk_len = (chunk_len + 15) / 16 * 16;  // keeps 16-byte alignment of chunk starts
        chunks = (NP + chunk_len - 1) / chunk_len;
        if (gy > 65535 || chunks > TK_MAX_I32)
            return TK3D_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((gather_lds_kernel<T, KK, HAS_W, V, NT>),
                           dim3((unsigned)chunks, (unsigned)gy, (unsigned)B), dim3(NT),
                           (size_t)(cg * row_bytes), s, in, idx, w, out, (int)C, (int)wc_total, (int)wc_off, (int)N1, NP, cg,
                           chunk_len, vec_ok);
        return tk_launch_status();
    }

    const int64_t tiles = (NP + (int64_t)GS_BLOCK * V - 1) / ((int64_t)GS_BLOCK * V);
    // Channels per workgroup: enough to amortise the index reads, few enough to
    // keep at least ~2k workgroups in flight.
    int cg = 16;
    while (cg > 1 && tiles * ((C + cg - 1) / cg) * B < 2048)
        cg /= 2;
    const int64_t gy = (C + cg - 1) / cg;
    if (tiles > TK_MAX_I32 || gy > 65535)
        return TK3D_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gather_kernel<T, KK, HAS_W, V>),
                       dim3((unsigned)tiles, (unsigned)gy, (unsigned)B), dim3(GS_BLOCK), 0, s,
                       in, idx, w, out, (int)C, (int)wc_total, (int)wc_off, (int)N1, NP, cg, vec_ok);
    return tk_launch_status();
}

template <typename T, int KK, bool HAS_W>
int scatter(const T *gout, const int64_t *idx, const T *w, int64_t B, int64_t C, int64_t N1,
            int64_t NP, T *gin, hipStream_t s, int64_t wc_total = -1, int64_t wc_off = 0)
{
    // gout may be a channel slice [wc_off, wc_off + C) of a tensor with wc_total
    // channels (same B and NP); by default it is exactly [B, C, NP].
    if (wc_total < 0)
        wc_total = C;
    const int64_t out_elems = B * C * N1;
    if (out_elems == 0)
        return TK3D_OK;
    if (!gin)
        return TK3D_ERR_NULL_POINTER;
    if (NP > 0 && (!gout || !idx || (HAS_W && !w)))
        return TK3D_ERR_NULL_POINTER;
    int64_t zero_blocks = (out_elems + GS_BLOCK - 1) / GS_BLOCK;
    if (zero_blocks > 16384)
        zero_blocks = 16384;
    if (NP == 0) {
        hipLaunchKernelGGL((fill_zero_kernel<T>), dim3((unsigned)zero_blocks), dim3(GS_BLOCK),
                           0, s, gin, out_elems);
        return tk_launch_status();
    }

    if constexpr (sizeof(T) == 4) {
        // fp32: 64-bit fixed-point accumulators, up to 128 KiB of LDS per workgroup.
        constexpr int64_t FIXED_LDS = 128 * 1024;
        constexpr int NT = 1024, V = 4, CGMAX = 8;
        // Rows longer than the LDS holds are accumulated in windows of destinations, each
        // by workgroups of its own that stream the whole input and keep what lands in
        // their window. Up to 16 windows this beats global atomics (the input is read once
        // per window); longer rows take the global path below.
        constexpr int64_t MAX_WINDOW = FIXED_LDS / 8, MAX_WINDOWS = 16;
        const int64_t windows = (N1 + MAX_WINDOW - 1) / MAX_WINDOW;
        const int64_t window = ((N1 + windows - 1) / windows + 3) / 4 * 4;
        const int64_t acc_row = window * 8;
        const int vec_ok = (((uintptr_t)gout & 15) == 0) && ((NP * 4) % 16 == 0);
        if constexpr ((KK == 1 && !HAS_W) || (KK == 3 && HAS_W)) {
            // Whole rows in LDS: the branch-free kernel, as two workgroups of 512 lanes and
            // up to 4 rows per CU when four rows fit in 72 KiB, else one workgroup of 1024
            // lanes with as many rows (4 at most) as fit in 132 KiB. The grid is what the
            // chip holds at once; the workgroups share out the jobs.
            constexpr int64_t ROWS_LDS = 132 * 1024, HALF_LDS = 72 * 1024;
            constexpr int PTS = KK == 1 ? 2 : 1;  // points per lane and chunk
            const int64_t row = (N1 + 64) * 8;
            if (windows == 1 && row <= ROWS_LDS) {
                const bool two = 4 * row <= HALF_LDS;
                const int64_t nt = two ? 512 : 1024;
                int cg = 4;
                while (cg > 1 && (cg * row > (two ? HALF_LDS : ROWS_LDS) || cg > C))
                    cg /= 2;
                // Prefer more jobs over wider channel groups until every CU has work.
                while (cg > 2 && B * ((C + cg - 1) / cg) < (two ? 512 : 256))
                    cg /= 2;
                const int64_t gy = (C + cg - 1) / cg;
                int64_t nseg = 1;
                const int64_t groups = B * gy;
                if (groups < 128) {
                    nseg = (256 + groups - 1) / groups;
                    const int64_t max_seg = (NP + 8 * nt - 1) / (8 * nt);
                    if (nseg > max_seg)
                        nseg = max_seg;
                    if (nseg < 1)
                        nseg = 1;
                }
                int64_t seg_len = (NP + nseg - 1) / nseg;
                seg_len = (seg_len + 15) / 16 * 16;
                nseg = (NP + seg_len - 1) / seg_len;
                const int64_t jobs = nseg * gy * B;
                if (jobs < ((int64_t)1 << 31) && seg_len * KK < ((int64_t)1 << 31)) {
                    int log2_count = 1;
                    while (((int64_t)1 << log2_count) < seg_len * KK + 1)
                        ++log2_count;
                    if (nseg > 1)
                        hipLaunchKernelGGL((fill_zero_kernel<T>), dim3((unsigned)zero_blocks),
                                           dim3(GS_BLOCK), 0, s, gin, out_elems);
                    const int64_t resident = (int64_t)tk_cu_count() * (two ? 2 : 1);
                    const int64_t wgs = jobs < resident ? jobs : resident;
                    auto launch = [&](auto kernel_tag, int threads) {
                        constexpr auto kernel = decltype(kernel_tag)::value;
                        const int allowed = tk_allow_dynamic_lds<kernel>((int)ROWS_LDS);
                        if (allowed != TK3D_OK)
                            return allowed;
                        hipLaunchKernelGGL(kernel, dim3((unsigned)wgs), dim3(threads),
                                           (size_t)(cg * row), s, gout, idx, w, gin, (int)C,
                                           (int)wc_total, (int)wc_off, (int)N1, NP, cg, seg_len,
                                           nseg > 1 ? 1 : 0, vec_ok, log2_count, (unsigned)nseg,
                                           (unsigned)gy, (unsigned)B);
                        return tk_launch_status();
                    };
                    if (two)
                        return launch(ScatterRowsKernel<KK, HAS_W, 512, 4, PTS>{}, 512);
                    return launch(ScatterRowsKernel<KK, HAS_W, 1024, 4, PTS>{}, 1024);
                }
            }
        }
        if (windows <= MAX_WINDOWS) {
            int cg = CGMAX;
            while (cg > 1 && (cg * acc_row > FIXED_LDS || cg > C))
                cg /= 2;
            // Prefer more workgroups over wider channel groups until every CU has one.
            while (cg > 2 && B * windows * ((C + cg - 1) / cg) < 256)
                cg /= 2;
            const int64_t gy = (C + cg - 1) / cg;
            int64_t nseg = 1;
            const int64_t groups = B * gy * windows;
            if (groups < 128) {
                nseg = (256 + groups - 1) / groups;
                const int64_t max_seg = (NP + 4 * NT * V - 1) / (4 * NT * V);
                if (nseg > max_seg)
                    nseg = max_seg;
                if (nseg < 1)
                    nseg = 1;
            }
            int64_t seg_len = (NP + nseg - 1) / nseg;
            seg_len = (seg_len + 15) / 16 * 16;
            nseg = (NP + seg_len - 1) / seg_len;
            if (gy * windows > 65535 || nseg > TK_MAX_I32)
                return TK3D_ERR_UNSUPPORTED;
            int log2_count = 1;
            while (((int64_t)1 << log2_count) < seg_len * KK + 1)
                ++log2_count;
            constexpr auto kernel = scatter_fixed_kernel<KK, HAS_W, V, NT, CGMAX>;
            const int allowed = tk_allow_dynamic_lds<kernel>((int)FIXED_LDS);
            if (allowed != TK3D_OK)
                return allowed;
            if (nseg > 1)
                hipLaunchKernelGGL((fill_zero_kernel<T>), dim3((unsigned)zero_blocks),
                                   dim3(GS_BLOCK), 0, s, gin, out_elems);
            hipLaunchKernelGGL(kernel, dim3((unsigned)nseg, (unsigned)(gy * windows), (unsigned)B),
                               dim3(NT), (size_t)(cg * acc_row), s, gout, idx, w, gin, (int)C,
                               (int)wc_total, (int)wc_off, (int)N1, NP, cg, seg_len,
                               nseg > 1 ? 1 : 0, vec_ok, log2_count, (int)gy, (int)window);
            return tk_launch_status();
        }
    }

    constexpr int64_t LDS_BUDGET = 64 * 1024;
    const int64_t row_bytes = N1 * (int64_t)sizeof(T);
    if (row_bytes <= LDS_BUDGET) {
        constexpr int NT = 512;
        constexpr int V = (sizeof(T) == 4) ? 4 : 2;
        const int vec_ok =
            (((uintptr_t)gout & 15) == 0) && ((NP * (int64_t)sizeof(T)) % 16 == 0);
        int cg = 8;
        while (cg > 1 && (cg * row_bytes > LDS_BUDGET || cg > C))
            cg /= 2;
        // Prefer more workgroups over wider channel groups until the chip is full.
        while (cg > 2 && B * ((C + cg - 1) / cg) < 512)
            cg /= 2;
        const int64_t gy = (C + cg - 1) / cg;
        int64_t nseg = 1;
        const int64_t groups = B * gy;
        if (groups < 256) {
            nseg = (512 + groups - 1) / groups;
            const int64_t max_seg = (NP + 4 * NT * V - 1) / (4 * NT * V);  // >= 4 rounds per lane
            if (nseg > max_seg)
                nseg = max_seg;
            if (nseg < 1)
                nseg = 1;
        }
        int64_t seg_len = (NP + nseg - 1) / nseg;
        seg_len = (seg_len + 15) / 16 * 16;  // keeps 16-byte alignment of segment starts
        nseg = (NP + seg_len - 1) / seg_len;
        if (gy > 65535 || nseg > TK_MAX_I32)
            return TK3D_ERR_UNSUPPORTED;
        if (nseg > 1)
            hipLaunchKernelGGL((fill_zero_kernel<T>), dim3((unsigned)zero_blocks),
                               dim3(GS_BLOCK), 0, s, gin, out_elems);
        hipLaunchKernelGGL((scatter_lds_kernel<T, KK, HAS_W, V, NT>),
                           dim3((unsigned)nseg, (unsigned)gy, (unsigned)B), dim3(NT),
                           (size_t)(cg * row_bytes), s, gout, idx, w, gin, (int)C, (int)wc_total, (int)wc_off, (int)N1, NP,
                           cg, seg_len, nseg > 1 ? 1 : 0, vec_ok);
        return tk_launch_status();
    }

    hipLaunchKernelGGL((fill_zero_kernel<T>), dim3((unsigned)zero_blocks), dim3(GS_BLOCK), 0, s,
                       gin, out_elems);
    const int64_t tiles = (NP + GS_BLOCK - 1) / GS_BLOCK;
    int cg = 8;
    while (cg > 1 && tiles * ((C + cg - 1) / cg) * B < 2048)
        cg /= 2;
    const int64_t gy = (C + cg - 1) / cg;
    if (tiles > TK_MAX_I32 || gy > 65535)
        return TK3D_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((scatter_global_kernel<T, KK, HAS_W>),
                       dim3((unsigned)tiles, (unsigned)gy, (unsigned)B), dim3(GS_BLOCK), 0, s,
                       gout, idx, w, gin, (int)C, (int)wc_total, (int)wc_off, (int)N1, NP, cg);
    return tk_launch_status();
}

template <typename T>
int interpolate_forward(const T *in, const int64_t *idx, const T *w, int64_t B, int64_t C,
                        int64_t N1, int64_t N2, int64_t K, T *out, void *stream)
{
    const int rc = check_shape(B, C, N1, N2, K);
    if (rc != TK3D_OK)
        return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (K) {
    case 1: return gather<T, 1, true>(in, idx, w, B, C, N1, N2, out, s);
    case 2: return gather<T, 2, true>(in, idx, w, B, C, N1, N2, out, s);
    case 3: return gather<T, 3, true>(in, idx, w, B, C, N1, N2, out, s);
    case 4: return gather<T, 4, true>(in, idx, w, B, C, N1, N2, out, s);
    case 5: return gather<T, 5, true>(in, idx, w, B, C, N1, N2, out, s);
    case 6: return gather<T, 6, true>(in, idx, w, B, C, N1, N2, out, s);
    case 7: return gather<T, 7, true>(in, idx, w, B, C, N1, N2, out, s);
    case 8: return gather<T, 8, true>(in, idx, w, B, C, N1, N2, out, s);
    default: return TK3D_ERR_BAD_K;
    }
}

template <typename T>
int interpolate_backward(const T *gout, const int64_t *idx, const T *w, int64_t B, int64_t C,
                         int64_t N1, int64_t N2, int64_t K, T *gin, void *stream)
{
    const int rc = check_shape(B, C, N1, N2, K);
    if (rc != TK3D_OK)
        return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (K) {
    case 1: return scatter<T, 1, true>(gout, idx, w, B, C, N1, N2, gin, s);
    case 2: return scatter<T, 2, true>(gout, idx, w, B, C, N1, N2, gin, s);
    case 3: return scatter<T, 3, true>(gout, idx, w, B, C, N1, N2, gin, s);
    case 4: return scatter<T, 4, true>(gout, idx, w, B, C, N1, N2, gin, s);
    case 5: return scatter<T, 5, true>(gout, idx, w, B, C, N1, N2, gin, s);
    case 6: return scatter<T, 6, true>(gout, idx, w, B, C, N1, N2, gin, s);
    case 7: return scatter<T, 7, true>(gout, idx, w, B, C, N1, N2, gin, s);
    case 8: return scatter<T, 8, true>(gout, idx, w, B, C, N1, N2, gin, s);
    default: return TK3D_ERR_BAD_K;
    }
}

template <typename T>
int group_forward(const T *in, const int64_t *idx, int64_t B, int64_t C, int64_t N1,
                  int64_t N2, int64_t K, T *out, void *stream)
{
    if (N2 < 0 || K < 0 || !tk_fits(TK_MAX_ELEMS, N2, K))
        return N2 < 0 || K < 0 ? TK3D_ERR_BAD_SIZE : TK3D_ERR_UNSUPPORTED;
    const int rc = check_shape(B, C, N1, N2 * K, 1);
    if (rc != TK3D_OK)
        return rc;
    return gather<T, 1, false>(in, idx, nullptr, B, C, N1, N2 * K, out, (hipStream_t)stream);
}

template <typename T>
int group_backward(const T *gout, const int64_t *idx, int64_t B, int64_t C, int64_t N1,
                   int64_t N2, int64_t K, T *gin, void *stream)
{
    if (N2 < 0 || K < 0 || !tk_fits(TK_MAX_ELEMS, N2, K))
        return N2 < 0 || K < 0 ? TK3D_ERR_BAD_SIZE : TK3D_ERR_UNSUPPORTED;
    const int rc = check_shape(B, C, N1, N2 * K, 1);
    if (rc != TK3D_OK)
        return rc;
    return scatter<T, 1, false>(gout, idx, nullptr, B, C, N1, N2 * K, gin,
                                (hipStream_t)stream);
}

// Grouped coordinates relative to their centre, written into the last three channels
// of a [B, wc_total, N2, K] tensor: out[b, wc_off+a, m, s] = xyz[b,a,idx[b,m,s]] -
// centre[b,a,m] (torkit3d/layers/pointnet2.py:55-58). The clouds are [B,3,N]; they
// are small (12 bytes per point), so the gathers hit in cache.
template <typename T>
__global__ __launch_bounds__(GS_BLOCK) void group_xyz_kernel(
    const T *__restrict__ xyz, const T *__restrict__ centre, const int64_t *__restrict__ idx,
    T *__restrict__ out, int wc_total, int wc_off, int n1, int n2, int k)
{
    const int b = blockIdx.y;
    const int64_t np = (int64_t)n2 * k;
    const int64_t p = (int64_t)blockIdx.x * GS_BLOCK + threadIdx.x;
    if (p >= np)
        return;
    const int64_t j = idx[(int64_t)b * np + p];
    const bool ok = j >= 0 && j < n1;
    const int m = (int)(p / k);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        const T v = ok ? xyz[((int64_t)b * 3 + a) * n1 + j] : (T)0;
        out[((int64_t)b * wc_total + wc_off + a) * np + p] =
            v - centre[((int64_t)b * 3 + a) * n2 + m];
    }
}

template <typename T>
int group_concat_forward(const T *feat, const T *xyz, const T *centre, const int64_t *idx,
                         int64_t B, int64_t C, int64_t N1, int64_t N2, int64_t K, T *out,
                         void *stream)
{
    if (N2 < 0 || K < 0 || !tk_fits(TK_MAX_ELEMS, N2, K))
        return N2 < 0 || K < 0 ? TK3D_ERR_BAD_SIZE : TK3D_ERR_UNSUPPORTED;
    const int rc = check_shape(B, C + 3, N1, N2 * K, 1);
    if (rc != TK3D_OK)
        return rc;
    if (B * N2 * K == 0)
        return TK3D_OK;
    if (!xyz || !centre || !idx || !out || (C > 0 && !feat))
        return TK3D_ERR_NULL_POINTER;
    hipStream_t s = (hipStream_t)stream;
    if (C > 0) {
        const int g = gather<T, 1, false>(feat, idx, nullptr, B, C, N1, N2 * K, out, s, C + 3, 0);
        if (g != TK3D_OK)
            return g;
    }
    const int64_t tiles = (N2 * K + GS_BLOCK - 1) / GS_BLOCK;
    if (tiles > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((group_xyz_kernel<T>), dim3((unsigned)tiles, (unsigned)B), dim3(GS_BLOCK),
                       0, s, xyz, centre, idx, out, (int)(C + 3), (int)C, (int)N1, (int)N2,
                       (int)K);
    return tk_launch_status();
}

template <typename T>
int group_concat_backward(const T *gout, const int64_t *idx, int64_t B, int64_t C, int64_t N1,
                          int64_t N2, int64_t K, T *gfeat, T *gxyz, void *stream)
{
    if (N2 < 0 || K < 0 || !tk_fits(TK_MAX_ELEMS, N2, K))
        return N2 < 0 || K < 0 ? TK3D_ERR_BAD_SIZE : TK3D_ERR_UNSUPPORTED;
    const int rc = check_shape(B, C + 3, N1, N2 * K, 1);
    if (rc != TK3D_OK)
        return rc;
    hipStream_t s = (hipStream_t)stream;
    if (C > 0 && gfeat) {
        const int g = scatter<T, 1, false>(gout, idx, nullptr, B, C, N1, N2 * K, gfeat, s, C + 3, 0);
        if (g != TK3D_OK)
            return g;
    }
    if (gxyz)
        return scatter<T, 1, false>(gout, idx, nullptr, B, 3, N1, N2 * K, gxyz, s, C + 3, C);
    return TK3D_OK;
}

}  // namespace

extern "C" {

int tk3d_group_points_concat_forward_f32(const float *feature, const float *xyz,
                                         const float *centre, const int64_t *index, int64_t B,
                                         int64_t C, int64_t N1, int64_t N2, int64_t K,
                                         float *output, void *stream)
{
    return group_concat_forward<float>(feature, xyz, centre, index, B, C, N1, N2, K, output,
                                       stream);
}
int tk3d_group_points_concat_forward_f64(const double *feature, const double *xyz,
                                         const double *centre, const int64_t *index,
                                         int64_t B, int64_t C, int64_t N1, int64_t N2,
                                         int64_t K, double *output, void *stream)
{
    return group_concat_forward<double>(feature, xyz, centre, index, B, C, N1, N2, K, output,
                                        stream);
}
int tk3d_group_points_concat_backward_f32(const float *grad_output, const int64_t *index,
                                          int64_t B, int64_t C, int64_t N1, int64_t N2,
                                          int64_t K, float *grad_feature, float *grad_xyz,
                                          void *stream)
{
    return group_concat_backward<float>(grad_output, index, B, C, N1, N2, K, grad_feature,
                                        grad_xyz, stream);
}
int tk3d_group_points_concat_backward_f64(const double *grad_output, const int64_t *index,
                                          int64_t B, int64_t C, int64_t N1, int64_t N2,
                                          int64_t K, double *grad_feature, double *grad_xyz,
                                          void *stream)
{
    return group_concat_backward<double>(grad_output, index, B, C, N1, N2, K, grad_feature,
                                         grad_xyz, stream);
}

int tk3d_group_points_forward_f32(const float *input, const int64_t *index, int64_t B,
                                  int64_t C, int64_t N1, int64_t N2, int64_t K,
                                  float *output, void *stream)
{
    return group_forward<float>(input, index, B, C, N1, N2, K, output, stream);
}
int tk3d_group_points_forward_f64(const double *input, const int64_t *index, int64_t B,
                                  int64_t C, int64_t N1, int64_t N2, int64_t K,
                                  double *output, void *stream)
{
    return group_forward<double>(input, index, B, C, N1, N2, K, output, stream);
}
int tk3d_group_points_backward_f32(const float *grad_output, const int64_t *index, int64_t B,
                                   int64_t C, int64_t N1, int64_t N2, int64_t K,
                                   float *grad_input, void *stream)
{
    return group_backward<float>(grad_output, index, B, C, N1, N2, K, grad_input, stream);
}
int tk3d_group_points_backward_f64(const double *grad_output, const int64_t *index,
                                   int64_t B, int64_t C, int64_t N1, int64_t N2, int64_t K,
                                   double *grad_input, void *stream)
{
    return group_backward<double>(grad_output, index, B, C, N1, N2, K, grad_input, stream);
}
int tk3d_interpolate_forward_f32(const float *input, const int64_t *index,
                                 const float *weight, int64_t B, int64_t C, int64_t N1,
                                 int64_t N2, int64_t K, float *output, void *stream)
{
    return interpolate_forward<float>(input, index, weight, B, C, N1, N2, K, output, stream);
}
int tk3d_interpolate_forward_f64(const double *input, const int64_t *index,
                                 const double *weight, int64_t B, int64_t C, int64_t N1,
                                 int64_t N2, int64_t K, double *output, void *stream)
{
    return interpolate_forward<double>(input, index, weight, B, C, N1, N2, K, output, stream);
}
int tk3d_interpolate_backward_f32(const float *grad_output, const int64_t *index,
                                  const float *weight, int64_t B, int64_t C, int64_t N1,
                                  int64_t N2, int64_t K, float *grad_input, void *stream)
{
    return interpolate_backward<float>(grad_output, index, weight, B, C, N1, N2, K,
                                       grad_input, stream);
}
int tk3d_interpolate_backward_f64(const double *grad_output, const int64_t *index,
                                  const double *weight, int64_t B, int64_t C, int64_t N1,
                                  int64_t N2, int64_t K, double *grad_input, void *stream)
{
    return interpolate_backward<double>(grad_output, index, weight, B, C, N1, N2, K,
                                        grad_input, stream);
}

}  // extern "C"

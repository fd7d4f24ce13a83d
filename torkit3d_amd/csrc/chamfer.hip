// Chamfer / nearest-neighbour distance for gfx950: forward (all-pairs minimum with
// argmin) and backward (closed-form gradient).
//
// Forward design
// --------------
// One workgroup owns QPL*BLOCK query points of one cloud and sweeps the opposite cloud -
// all of it, or one slice of it when the launch would otherwise leave most of the chip
// idle (the slices' results then meet in a packed 64-bit minimum, see chamfer_emit).
// Key points are staged through LDS as (x,y,z,pad) quads; every
// lane reads the same quad (a broadcast ds_read_b128) and applies it to the QPL
// queries it keeps in registers, so one LDS read feeds QPL distance evaluations.
//
// The inner loop tracks only the VALUE of the minimum: per pair three subtracts,
// one multiply, two fused multiply-adds and half a three-operand minimum. The
// argmin is recovered afterwards: the sweep is cut into tiles of TILE keys, each
// query remembers the first tile that lowered its minimum to the final value
// (one compare and two selects per tile, not per key), and a short epilogue
// re-evaluates that one tile to find the lowest key index whose distance equals
// the minimum bit for bit. This keeps the reference's tie rule (strict '<' over
// ascending j, chamfer_distance_kernel.cu:73) exactly.
//
// Both directions (cloud 1 -> 2 and 2 -> 1) run in one launch.
#include "tk3d_common.h"
#include "tk3d_debug.h"

#include <type_traits>

namespace {

template <typename T> struct ChamferDir {
    const T *query;   // [B, nq, 3]
    const T *key;     // [B, nk, 3]
    T *dist;          // [B, nq]
    int64_t *idx;     // [B, nq]
    int nq;
    int nk;
    int blocks_per_batch;  // query blocks x key slices
    int slices;            // key slices a query's sweep is split into (1: no split)
    int slice_len;         // keys per slice, a multiple of the tile length
};

template <typename T> struct ChamferFwdArgs {
    ChamferDir<T> dir[2];
    int nblocks0;  // workgroups of direction 0; the rest belong to direction 1
    // When set: [2, nbatch] flags, and a workgroup of direction w and batch element b
    // works only if only_if[w * nbatch + b] is non-zero (chamfer_forward_mfma_flagged_kernel only).
    const int *only_if;
    int nbatch;
};

template <typename T> __device__ __forceinline__ T chamfer_init_min();
// The reference starts from 1e40 (chamfer_distance_kernel.cu:42), which is +inf
// once stored in a float and a finite number in a double.
template <> __device__ __forceinline__ float chamfer_init_min<float>()
{
    return __builtin_huge_valf();
}
template <> __device__ __forceinline__ double chamfer_init_min<double>()
{
    return 1e40;
}

// A cloud as the kernels read it: coordinate a of point j of the cloud at `base` is
// base[j * 3 + a] in a [N,3] cloud and base[a * plane + j] in a [3,N] one (SOA; `plane` is
// the number of points of the whole cloud, also when `base` points at a slice of it).
template <bool SOA, typename T>
__device__ __forceinline__ T chamfer_coord(const T *__restrict__ base, int plane, int j, int a)
{
    return SOA ? base[(int64_t)a * plane + j] : base[(int64_t)j * 3 + a];
}
template <bool SOA, typename T>
__device__ __forceinline__ TkPoint3<T> chamfer_point(const T *__restrict__ base, int plane, int j)
{
    if constexpr (SOA) {
        TkPoint3<T> p;
        p.x = base[j];
        p.y = base[(int64_t)plane + j];
        p.z = base[(int64_t)2 * plane + j];
        return p;
    } else {
        return tk_load3<T>(base + (int64_t)j * 3);
    }
}
// Start of batch element b's key slice beginning at key k0, in either layout.
template <bool SOA, typename T>
__device__ __forceinline__ const T *chamfer_key_base(const T *key, int b, int nk_cloud, int k0)
{
    return SOA ? key + (int64_t)b * nk_cloud * 3 + k0 : key + ((int64_t)b * nk_cloud + k0) * 3;
}

// Decodes blockIdx into (direction, batch, query block). Workgroups are handed to
// the 8 XCDs round-robin by blockIdx; the remap gives each XCD a contiguous range of
// logical workgroups, so the workgroups that sweep the same key cloud share one L2
// instead of fetching it 8 times.
template <typename T>
__device__ __forceinline__ const ChamferDir<T> &chamfer_decode_block(
    const ChamferFwdArgs<T> &args, int &b, int &qblock, int &slice)
{
    int lb = blockIdx.x;
    const int nb = gridDim.x, per = nb >> 3, full = per << 3;
    if (lb < full)
        lb = (lb & 7) * per + (lb >> 3);
    const int which = lb >= args.nblocks0;
    if (which)
        lb -= args.nblocks0;
    const ChamferDir<T> &d = args.dir[which];
    b = lb / d.blocks_per_batch;
    const int rest = lb - b * d.blocks_per_batch;
    qblock = rest / d.slices;
    slice = rest - qblock * d.slices;
    return d;
}

// Result of one workgroup for query `qi` of batch `b`: distance `dist` to key `j` of the
// workgroup's slice (j < 0: the slice holds no key with a finite distance).
//
// Unsplit sweeps store it. With key slices several workgroups hold partial results for
// the same query; they meet in the index output, used as 64-bit words that hold
// (distance bits << 32 | key index): distances are non-negative, so their bit patterns
// order as unsigned integers and an unsigned minimum of the packed words keeps the
// smallest distance and, among equal distances, the lowest key index - the reference's
// strict '<' over ascending j. chamfer_split_init_kernel sets the words to (+inf, -1)
// beforehand and chamfer_split_finish_kernel unpacks them.
template <typename T>
__device__ __forceinline__ void chamfer_emit(const ChamferDir<T> &d, int b, int qi, int k0,
                                             T dist, int j)
{
    const int64_t o = (int64_t)b * d.nq + qi;
    if constexpr (sizeof(T) == 4) {
        if (d.slices > 1) {
            if (j >= 0) {
                const unsigned long long word =
                    ((unsigned long long)__builtin_bit_cast(unsigned, dist) << 32) |
                    (unsigned)(j + k0);
                atomicMin(reinterpret_cast<unsigned long long *>(d.idx) + o, word);
            }
            return;
        }
    }
    d.dist[o] = dist;
    d.idx[o] = (int64_t)j;
}

// Exact sweep of one workgroup: QPL*BLOCK queries against the whole key cloud.
// `skey` is STAGE*4 elements of LDS.
template <typename T, int QPL, int BLOCK, int TILE, int STAGE, bool SOA = false>
__device__ __forceinline__ void chamfer_exact_sweep(const ChamferDir<T> &d, int b, int qblock,
                                                    int slice, T *skey)
{
    static_assert(STAGE % TILE == 0 && TILE % 2 == 0, "tile shapes");
    const int tid = threadIdx.x;
    const int nq = d.nq;
    const int k0 = slice * d.slice_len;  // this workgroup sweeps keys [k0, k0 + nk)
    const int nk = (d.nk - k0 < d.slice_len) ? d.nk - k0 : d.slice_len;
    const T *__restrict__ Q = d.query + (int64_t)b * nq * 3;
    const T *__restrict__ K = chamfer_key_base<SOA, T>(d.key, b, d.nk, k0);

    T qx[QPL], qy[QPL], qz[QPL], best[QPL];
    int btile[QPL];
#pragma unroll
    for (int i = 0; i < QPL; ++i) {
        const int qi = (qblock * QPL + i) * BLOCK + tid;
        const bool ok = qi < nq;
        qx[i] = ok ? chamfer_coord<SOA, T>(Q, nq, qi, 0) : (T)0;
        qy[i] = ok ? chamfer_coord<SOA, T>(Q, nq, qi, 1) : (T)0;
        qz[i] = ok ? chamfer_coord<SOA, T>(Q, nq, qi, 2) : (T)0;
        best[i] = chamfer_init_min<T>();
        btile[i] = -1;
    }

    for (int stage0 = 0; stage0 < nk; stage0 += STAGE) {
        __syncthreads();
        for (int j = tid; j < STAGE; j += BLOCK) {
            const int kj = stage0 + j;
            T x = tk_inf<T>(), y = tk_inf<T>(), z = tk_inf<T>();
            if (kj < nk) {
                const TkPoint3<T> p = chamfer_point<SOA, T>(K, d.nk, kj);
                x = p.x, y = p.y, z = p.z;
            }
            // Keys past the end sit at +inf: their distance is +inf or NaN and
            // can never lower a minimum.
            skey[j * 4 + 0] = x;
            skey[j * 4 + 1] = y;
            skey[j * 4 + 2] = z;
            skey[j * 4 + 3] = (T)0;
        }
        __syncthreads();

        const int left = nk - stage0;
        const int ntiles = ((left < STAGE ? left : STAGE) + TILE - 1) / TILE;
        for (int t = 0; t < ntiles; ++t) {
            T tmin[QPL];
#pragma unroll
            for (int i = 0; i < QPL; ++i)
                tmin[i] = tk_inf<T>();
            const T *tk = skey + t * TILE * 4;
            // the next pair of keys is read while the current pair is evaluated (the last
            // read of a stage runs into the two pad keys behind the buffer)
            T ax = tk[0], ay = tk[1], az = tk[2], bx = tk[4], by = tk[5], bz = tk[6];
#pragma unroll
            for (int j = 0; j < TILE; j += 2) {
                const T nax = tk[j * 4 + 8], nay = tk[j * 4 + 9], naz = tk[j * 4 + 10];
                const T nbx = tk[j * 4 + 12], nby = tk[j * 4 + 13], nbz = tk[j * 4 + 14];
#pragma unroll
                for (int i = 0; i < QPL; ++i) {
                    const T da = tk_dist2<T>(ax, ay, az, qx[i], qy[i], qz[i]);
                    const T db = tk_dist2<T>(bx, by, bz, qx[i], qy[i], qz[i]);
                    tmin[i] = tk_min<T>(tk_min<T>(tmin[i], da), db);
                }
                ax = nax, ay = nay, az = naz;
                bx = nbx, by = nby, bz = nbz;
            }
            const int tile_id = stage0 / TILE + t;
#pragma unroll
            for (int i = 0; i < QPL; ++i) {
                const bool lower = tmin[i] < best[i];
                best[i] = lower ? tmin[i] : best[i];
                btile[i] = lower ? tile_id : btile[i];
            }
        }
    }

    // Epilogue: lowest key index inside the remembered tile whose distance equals
    // the minimum exactly (same operations on the same bits as the sweep).
#pragma unroll
    for (int i = 0; i < QPL; ++i) {
        const int qi = (qblock * QPL + i) * BLOCK + tid;
        if (qi >= nq)
            continue;
        int found = -1;
        if (btile[i] >= 0) {
            const int j0 = btile[i] * TILE;
            const int j1 = (j0 + TILE < nk) ? j0 + TILE : nk;
            for (int j = j1 - 1; j >= j0; --j) {
                const TkPoint3<T> p = chamfer_point<SOA, T>(K, d.nk, j);
                const T dd = tk_dist2<T>(p.x, p.y, p.z, qx[i], qy[i], qz[i]);
                found = (dd == best[i]) ? j : found;
            }
        }
        chamfer_emit<T>(d, b, qi, k0, best[i], found);
    }
}

template <typename T, int QPL, int BLOCK, int TILE, int STAGE, bool SOA = false>
__global__ __launch_bounds__(BLOCK) void chamfer_forward_kernel(ChamferFwdArgs<T> args)
{
    __shared__ T skey[STAGE * 4 + 8];  // + 2 keys for the read-ahead
    int b, qblock, slice;
    const ChamferDir<T> &d = chamfer_decode_block<T>(args, b, qblock, slice);
    chamfer_exact_sweep<T, QPL, BLOCK, TILE, STAGE, SOA>(d, b, qblock, slice, skey);
}

// ---- fp32 forward with a bounded-error pre-filter -------------------------------
//
// The exact sweep spends 6.5 VALU instructions per pair. Most pairs only need to be
// ruled out, which a cheaper score can do:
//
//     s(q,k) = |k'|^2 - 2 q'.k'   (k' = k - c, q' = q - c, c = centre of the key
//                                  cloud's bounding box; three fused multiply-adds
//                                  per pair, |k'|^2 staged with the key)
//
// d2(q,k) = s + |q'|^2 up to rounding. For one query the additive |q'|^2 is common to
// all keys, so minima of s locate minima of d2 up to the rounding error of both
// expressions. With u = 2^-24, rho = |k'| + |q'| and d the true distance:
//     canonical d2: three rounded differences, one product, two fmas, all terms
//         non-negative                      |canonical - d^2| <= 5.01 u d^2 <= 5.01 u rho^2
//     centring: k' and q' carry one rounding each, so k'-q' is off by at most
//         u rho and its squared norm by     2.01 u rho^2
//     |k'|^2: three non-negative rounded terms                   3 u |k'|^2
//     the three fmas of s: each rounds a partial sum of magnitude at most rho^2
//                                                                3.01 u rho^2
// hence |s + |q'|^2 - canonical d2| <= E = 13.1 u R with R = (max|k'| + |q'|)^2, and any
// key whose canonical distance equals the minimum has s <= min(s) + 2E. The kernel
// compares against min(s) + slack with slack = 32 u R: 26.2 u R for 2E, 1 u R for the
// rounding of that sum, the rest margin (max|k'| and |q'| are inflated by 1e-6 to
// cover their own rounding; 1e-37 is added against underflow).
//
// Sweep: per tile of TILE keys only min(s) is formed (3 fma + half a min3 per
// pair), and each query keeps the three smallest tile minima v0<=v1<=v2 with the
// tile ids of the first two. Afterwards:
//     v2 >  v0 + slack : at most two tiles can hold the argmin; they are
//                        re-evaluated with the exact canonical arithmetic in
//                        ascending key order (strict '<'), which yields exactly the
//                        reference's distance and lowest-index argmin;
//     v2 <= v0 + slack : three or more candidate tiles (heavy ties); the wave scans
//                        the whole key cloud for that query with exact arithmetic.
// Non-finite or huge coordinates (where the bound above does not hold) take the
// exact sweep for the whole workgroup or the exact scan for the query.
// Results are therefore bit-identical to the exact sweep for every input.

// Minimum / maximum over the wave, the same value in every lane (NaNs are passed over, as
// fminf / fmaxf do). A scan along rows of 16 lanes with row shifts, the rows' results carried
// on with row broadcasts, the total read from lane 63: six short steps on the vector ALU where
// six exchanges through the LDS crossbar (ds_bpermute) took a hundred clocks each.
template <bool MAX> __device__ __forceinline__ float wave_reduce_extreme(float v)
{
#define TK_WAVE_STEP(ctrl, rows)                                                              \
    {                                                                                         \
        const float o = __builtin_bit_cast(                                                   \
            float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v),                    \
                                               __builtin_bit_cast(int, v), ctrl, rows, 0xf,   \
                                               false));                                       \
        v = MAX ? __builtin_fmaxf(v, o) : __builtin_fminf(v, o);                              \
    }
    TK_WAVE_STEP(0x111, 0xf)  // row_shr:1
    TK_WAVE_STEP(0x112, 0xf)  // row_shr:2
    TK_WAVE_STEP(0x114, 0xf)  // row_shr:4
    TK_WAVE_STEP(0x118, 0xf)  // row_shr:8
    TK_WAVE_STEP(0x142, 0xa)  // row_bcast:15 into rows 1 and 3
    TK_WAVE_STEP(0x143, 0xc)  // row_bcast:31 into rows 2 and 3
#undef TK_WAVE_STEP
    return __builtin_bit_cast(float,
                              __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), TK_WAVE - 1));
}
__device__ __forceinline__ float wave_reduce_min(float v)
{
    return wave_reduce_extreme<false>(v);
}
__device__ __forceinline__ float wave_reduce_max(float v)
{
    return wave_reduce_extreme<true>(v);
}

// Exact nearest neighbour of one query, the whole workgroup cooperating: lane t scans
// keys t, t+BLOCK, ... in ascending order with strict '<'; the workgroup keeps the
// smallest distance and, among equal distances, the lowest key index. Every lane
// returns the result. `sval` / `sidx` hold one entry per wave.
template <int BLOCK, bool SOA = false>
__device__ __forceinline__ void chamfer_block_exact_scan(const float *__restrict__ K, int nk,
                                                         float qx, float qy, float qz,
                                                         float *sval, int *sidx, float &out_d,
                                                         int &out_j, int kplane = 0)
{
    constexpr int NW = BLOCK / TK_WAVE;
    const int tid = threadIdx.x;
    float best = __builtin_huge_valf();
    int bj = -1;
#pragma unroll 8
    for (int j = tid; j < nk; j += BLOCK) {
        const TkPoint3<float> p = chamfer_point<SOA, float>(K, kplane, j);
        const float d = tk_dist2<float>(p.x, p.y, p.z, qx, qy, qz);
        if (d < best) {
            best = d;
            bj = j;
        }
    }
    const float wmin = wave_reduce_min(best);
    int cand = (best == wmin && bj >= 0) ? bj : 0x7fffffff;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const int other = __shfl_xor(cand, o);
        cand = other < cand ? other : cand;
    }
    __syncthreads();
    if ((tid & (TK_WAVE - 1)) == 0) {
        sval[tid / TK_WAVE] = wmin;
        sidx[tid / TK_WAVE] = cand;
    }
    __syncthreads();
    float g = __builtin_huge_valf();
#pragma unroll
    for (int w = 0; w < NW; ++w)
        g = __builtin_fminf(g, sval[w]);
    int gj = 0x7fffffff;
#pragma unroll
    for (int w = 0; w < NW; ++w)
        gj = (sval[w] == g && sidx[w] < gj) ? sidx[w] : gj;
    out_d = g;
    out_j = gj == 0x7fffffff ? -1 : gj;
}

template <int QPL, int BLOCK, int TILE, int STAGE>
__global__ __launch_bounds__(BLOCK) void chamfer_forward_filter_kernel(ChamferFwdArgs<float> args)
{
    static_assert(STAGE % TILE == 0 && TILE % 2 == 0, "tile shapes");
    constexpr int NW = BLOCK / TK_WAVE;
    // More queries than this with three or more candidate tiles: the cloud is full of
    // ties (quantised coordinates) and the exact sweep is the cheaper way out.
    constexpr int MAX_SCANS = 96;
    __shared__ __align__(16) float skey[2 * STAGE * 4 + 8];  // + 2 keys for the read-ahead
    __shared__ float sred[NW][8];
    __shared__ int sidx[NW];
    __shared__ int s_list[MAX_SCANS];
    __shared__ int s_count;

    const int tid = threadIdx.x;
    const int lane = tid & (TK_WAVE - 1);
    const int wave = tid / TK_WAVE;
    int b, qblock, slice;
    const ChamferDir<float> &d = chamfer_decode_block<float>(args, b, qblock, slice);
    const int nq = d.nq;
    // This workgroup sweeps keys [k0, k0 + nk); to the filter that slice is the key cloud.
    const int k0 = slice * d.slice_len;
    const int nk = (d.nk - k0 < d.slice_len) ? d.nk - k0 : d.slice_len;
    const float *__restrict__ Q = d.query + (int64_t)b * nq * 3;
    const float *__restrict__ K = d.key + ((int64_t)b * d.nk + k0) * 3;
    const float INF = __builtin_huge_valf();

    // ---- bounding box of the key cloud -> centre ----
    float lo[3] = {INF, INF, INF}, hi[3] = {-INF, -INF, -INF};
    for (int j = tid; j < nk; j += BLOCK) {
        const TkPoint3<float> p = tk_load3<float>(K + (int64_t)j * 3);
        const float v[3] = {p.x, p.y, p.z};
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            lo[a] = __builtin_fminf(lo[a], v[a]);
            hi[a] = __builtin_fmaxf(hi[a], v[a]);
        }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        lo[a] = wave_reduce_min(lo[a]);
        hi[a] = wave_reduce_max(hi[a]);
    }
    if (lane == 0) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            sred[wave][a] = lo[a];
            sred[wave][3 + a] = hi[a];
        }
    }
    if (tid == 0)
        s_count = 0;
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
    // ---- largest centred squared norm, computed as the staging below computes it ----
    float kmax2 = 0.0f;
    for (int j = tid; j < nk; j += BLOCK) {
        const TkPoint3<float> p = tk_load3<float>(K + (int64_t)j * 3);
        const float x = p.x - c0;
        const float y = p.y - c1;
        const float z = p.z - c2;
        kmax2 = __builtin_fmaxf(kmax2, __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x)));
    }
    kmax2 = wave_reduce_max(kmax2);
    if (lane == 0)
        sred[wave][6] = kmax2;
    __syncthreads();
    kmax2 = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w)
        kmax2 = __builtin_fmaxf(kmax2, sred[w][6]);

    // The error bound needs finite, moderate magnitudes; otherwise do the exact sweep.
    const bool safe = (c0 - c0 == 0.0f) && (c1 - c1 == 0.0f) && (c2 - c2 == 0.0f) &&
                      (kmax2 < 1e30f);
    if (!safe) {  // uniform over the workgroup
        chamfer_exact_sweep<float, QPL, BLOCK, TILE, STAGE>(d, b, qblock, slice, skey);
        return;
    }
    // sqrt and the norm carry a few u of rounding; 1e-6 covers them.
    const float kmax = __builtin_sqrtf(kmax2) * 1.000001f;

    // ---- queries: a = -2 (q - c) ----
    float ax[QPL], ay[QPL], az[QPL];
    float v0[QPL], v1[QPL], v2[QPL];
    int id0[QPL], id1[QPL];
#pragma unroll
    for (int i = 0; i < QPL; ++i) {
        const int qi = (qblock * QPL + i) * BLOCK + tid;
        const bool ok = qi < nq;
        ax[i] = -2.0f * ((ok ? Q[(int64_t)qi * 3 + 0] : c0) - c0);
        ay[i] = -2.0f * ((ok ? Q[(int64_t)qi * 3 + 1] : c1) - c1);
        az[i] = -2.0f * ((ok ? Q[(int64_t)qi * 3 + 2] : c2) - c2);
        v0[i] = v1[i] = v2[i] = INF;
        id0[i] = id1[i] = -1;
    }
    // slack = 32 u (max|k'| + |q'|)^2, from a = -2 q'. NaN / inf for a non-finite or
    // huge query; the epilogue tests for that.
    auto slack_of = [&](int i) {
        const float qn = 0.5f * 1.000001f *
                         __builtin_sqrtf(__builtin_fmaf(az[i], az[i],
                                                        __builtin_fmaf(ay[i], ay[i], ax[i] * ax[i])));
        const float r = kmax + qn;
        return r * r * 1.9073486e-06f + 1e-37f;
    };

    // ---- sweep ----
    // Keys are centred and staged as (x', y', z', |k'|^2) in two LDS buffers: the next
    // stage is fetched into registers before the current one is consumed and stored
    // to the other buffer afterwards, so a stage costs one barrier and its global
    // loads overlap the arithmetic.
    constexpr int PER = STAGE / BLOCK;
    static_assert(STAGE % BLOCK == 0, "whole keys per lane and stage");
    const int nstages = (nk + STAGE - 1) / STAGE;
    float4 pre[PER];
    auto fetch = [&](int st) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int kj = st * STAGE + r * BLOCK + tid;
            float4 e = make_float4(0.0f, 0.0f, 0.0f, INF);  // past the end: s = +inf
            if (kj < nk) {
                const TkPoint3<float> p = tk_load3<float>(K + (int64_t)kj * 3);
                e.x = p.x - c0;
                e.y = p.y - c1;
                e.z = p.z - c2;
                e.w = __builtin_fmaf(e.z, e.z, __builtin_fmaf(e.y, e.y, e.x * e.x));
            }
            pre[r] = e;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int r = 0; r < PER; ++r)
            reinterpret_cast<float4 *>(skey)[buf * STAGE + r * BLOCK + tid] = pre[r];
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

        const int left = nk - stage0;
        const int ntiles = ((left < STAGE ? left : STAGE) + TILE - 1) / TILE;
        for (int t = 0; t < ntiles; ++t) {
            float tmin[QPL];
#pragma unroll
            for (int i = 0; i < QPL; ++i)
                tmin[i] = INF;
            const float4 *tk = sbuf + t * TILE;
            // The pair after the current one is read from LDS before the current pair's
            // 28 vector instructions, so its latency hides behind them (the last read of
            // a tile runs into the next tile or the pad behind the buffers). Reading two
            // pairs ahead was slower (more registers).
            float4 ka = tk[0], kb = tk[1];
#pragma unroll
            for (int j = 0; j < TILE; j += 2) {
                const float4 na = tk[j + 2], nb = tk[j + 3];
#pragma unroll
                for (int i = 0; i < QPL; ++i) {
                    const float sa = __builtin_fmaf(
                        ka.x, ax[i], __builtin_fmaf(ka.y, ay[i], __builtin_fmaf(ka.z, az[i], ka.w)));
                    const float sb = __builtin_fmaf(
                        kb.x, ax[i], __builtin_fmaf(kb.y, ay[i], __builtin_fmaf(kb.z, az[i], kb.w)));
                    tmin[i] = __builtin_fminf(__builtin_fminf(tmin[i], sa), sb);
                }
                ka = na;
                kb = nb;
            }
            // Three smallest tile minima (ties keep the earlier tile in front).
            const int tile_id = stage0 / TILE + t;
#pragma unroll
            for (int i = 0; i < QPL; ++i) {
                const float x = tmin[i];
                const bool lt0 = x < v0[i];
                const bool lt1 = x < v1[i];
                id1[i] = lt1 ? tile_id : id1[i];
                id1[i] = lt0 ? id0[i] : id1[i];
                id0[i] = lt0 ? tile_id : id0[i];
                v2[i] = __builtin_amdgcn_fmed3f(v1[i], v2[i], x);
                v1[i] = __builtin_amdgcn_fmed3f(v0[i], v1[i], x);
                v0[i] = __builtin_amdgcn_fmed3f(-INF, v0[i], x);
            }
        }

        if (st + 1 < nstages)
            stash((st + 1) & 1);
        __syncthreads();

        // One look, an eighth of the way in: if a quarter of the queries already see
        // three tiles within the slack, the cloud is quantised and will not get better.
        if (nstages >= 8 && st == (nstages >> 3)) {
            int tied = 0;
#pragma unroll
            for (int i = 0; i < QPL; ++i) {
                const int qi = (qblock * QPL + i) * BLOCK + tid;
                const bool t3 = qi < nq && v2[i] <= v0[i] + slack_of(i);
                tied += __builtin_popcountll(__builtin_amdgcn_ballot_w64(t3));
            }
            if (lane == 0)
                atomicAdd(&s_count, tied);
            __syncthreads();
            const int total = s_count;
            __syncthreads();
            if (tid == 0)
                s_count = 0;
            if (total * 4 > QPL * BLOCK) {  // uniform over the workgroup
                chamfer_exact_sweep<float, QPL, BLOCK, TILE, STAGE>(d, b, qblock, slice, skey);
                return;
            }
        }
    }

    // ---- epilogue: exact evaluation of the candidate tiles ----
    static_assert(TILE % 4 == 0, "tile of whole 16-byte groups");
    const bool k_aligned = (reinterpret_cast<uintptr_t>(K) & 15) == 0;  // tiles are 768 B
#pragma unroll
    for (int i = 0; i < QPL; ++i) {
        const int qi = (qblock * QPL + i) * BLOCK + tid;
        const bool ok = qi < nq;
        const float slack = slack_of(i);
        const float thr = v0[i] + slack;
        const bool usable = slack < 1e30f;  // false for NaN / inf / huge
        // No finite score at all (nk == 0 or every key NaN): the exact result is (+inf, -1).
        const bool none = !(v0[i] < INF);
        const bool second = v1[i] <= thr;
        const bool over = ok && !none && (!usable || v2[i] <= thr);
        float bestd = INF;
        int bestj = -1;
        if (ok && !none && !over) {
            const float qx = Q[(int64_t)qi * 3 + 0], qy = Q[(int64_t)qi * 3 + 1],
                        qz = Q[(int64_t)qi * 3 + 2];
            int ta = id0[i], tb = second ? id1[i] : -1;
            if (tb >= 0 && tb < ta) {
                const int tmp = ta;
                ta = tb;
                tb = tmp;
            }
            for (int pass = 0; pass < 2; ++pass) {
                const int tile = pass == 0 ? ta : tb;
                if (tile < 0)
                    continue;
                const int j0 = tile * TILE;
                if (k_aligned && j0 + TILE <= nk) {
                    // 16-byte loads: four keys per three quads.
                    const float4 *p4 = reinterpret_cast<const float4 *>(K + (int64_t)j0 * 3);
#pragma unroll 2
                    for (int g = 0; g < TILE / 4; ++g) {
                        const float4 f0 = p4[g * 3 + 0], f1 = p4[g * 3 + 1], f2 = p4[g * 3 + 2];
                        const float dd0 = tk_dist2<float>(f0.x, f0.y, f0.z, qx, qy, qz);
                        const float dd1 = tk_dist2<float>(f0.w, f1.x, f1.y, qx, qy, qz);
                        const float dd2 = tk_dist2<float>(f1.z, f1.w, f2.x, qx, qy, qz);
                        const float dd3 = tk_dist2<float>(f2.y, f2.z, f2.w, qx, qy, qz);
                        const int j = j0 + g * 4;
                        if (dd0 < bestd) { bestd = dd0; bestj = j; }
                        if (dd1 < bestd) { bestd = dd1; bestj = j + 1; }
                        if (dd2 < bestd) { bestd = dd2; bestj = j + 2; }
                        if (dd3 < bestd) { bestd = dd3; bestj = j + 3; }
                    }
                } else if (j0 + TILE <= nk) {
                    // Rows of this cloud are not 16-byte aligned: one 12-byte load per key.
#pragma unroll 2
                    for (int g = 0; g < TILE / 4; ++g) {
                        const int j = j0 + g * 4;
                        const TkPoint3<float> p0 = tk_load3<float>(K + (int64_t)j * 3);
                        const TkPoint3<float> p1 = tk_load3<float>(K + (int64_t)j * 3 + 3);
                        const TkPoint3<float> p2 = tk_load3<float>(K + (int64_t)j * 3 + 6);
                        const TkPoint3<float> p3 = tk_load3<float>(K + (int64_t)j * 3 + 9);
                        const float dd0 = tk_dist2<float>(p0.x, p0.y, p0.z, qx, qy, qz);
                        const float dd1 = tk_dist2<float>(p1.x, p1.y, p1.z, qx, qy, qz);
                        const float dd2 = tk_dist2<float>(p2.x, p2.y, p2.z, qx, qy, qz);
                        const float dd3 = tk_dist2<float>(p3.x, p3.y, p3.z, qx, qy, qz);
                        if (dd0 < bestd) { bestd = dd0; bestj = j; }
                        if (dd1 < bestd) { bestd = dd1; bestj = j + 1; }
                        if (dd2 < bestd) { bestd = dd2; bestj = j + 2; }
                        if (dd3 < bestd) { bestd = dd3; bestj = j + 3; }
                    }
                } else {
                    for (int j = j0; j < nk; ++j) {
                        const TkPoint3<float> p = tk_load3<float>(K + (int64_t)j * 3);
                        const float dd = tk_dist2<float>(p.x, p.y, p.z, qx, qy, qz);
                        if (dd < bestd) {
                            bestd = dd;
                            bestj = j;
                        }
                    }
                }
            }
        }
        if (ok && !over)
            chamfer_emit<float>(d, b, qi, k0, bestd, bestj);
        if (over) {
            const int slot = atomicAdd(&s_count, 1);
            if (slot < MAX_SCANS)
                s_list[slot] = i * BLOCK + tid;
        }
    }

    // ---- queries with three or more candidate tiles ----
    __syncthreads();
    const int nscan = s_count;
    if (nscan > MAX_SCANS) {  // uniform over the workgroup
        chamfer_exact_sweep<float, QPL, BLOCK, TILE, STAGE>(d, b, qblock, slice, skey);
        return;
    }
    for (int e = 0; e < nscan; ++e) {
        const int slot = s_list[e];
        const int qi = (qblock * QPL + slot / BLOCK) * BLOCK + (slot % BLOCK);
        float bd;
        int bj;
        chamfer_block_exact_scan<BLOCK>(K, nk, Q[(int64_t)qi * 3 + 0], Q[(int64_t)qi * 3 + 1],
                                        Q[(int64_t)qi * 3 + 2], &sred[0][0], sidx, bd, bj);
        if (tid == 0)
            chamfer_emit<float>(d, b, qi, k0, bd, bj);
    }
}

// ---- fp32 forward, pre-filter on the matrix cores --------------------------------
//
// The score s(q,k) = |k'|^2 - 2 q'.k' of the kernel above is a dot product, and the
// pre-filter only has to be accurate to a stated bound, so it can run as an fp16 matrix
// product with fp32 accumulation (v_mfma_f32_32x32x16_f16: 32 keys x 32 queries x 16
// terms in 32 clocks, against 3 x 2 clocks of vector FMAs per 64 pairs).
//
// Coordinates are centred on c and multiplied by a power of two 2^-e (exact), so that the
// key cloud's extent is of order 1 and fp16's range is not an issue; c and e come from a
// strided sample of 1024 keys and need not be accurate: the bound below uses the largest
// centred norm of *all* keys, which the staging computes on the way, and input that leaves
// the range (|k'| > 181, the extent's exponent outside [-40, 40], anything non-finite in
// the sample) takes the exact sweep. From here on k', q' are the centred, scaled points.
// Every coordinate is split into two fp16 pieces, x = xh + xl + e with |e| <= 2^-23 |x|
// + 2^-25 (fp16 has 11 significant bits: |x - xh| <= 2^-11 |x| to nearest and xl, again
// to nearest, is within 2^-12 of that, or within half the subnormal spacing 2^-24; the
// matrix cores of this GPU take subnormal fp16 input as it is - measured, and flushing
// would put errors of 2^-14 |X| into the scores of every uniform cloud, far beyond the
// slack, so the parity tests on such clouds would fail), and |k'|^2 into
// three. The 16 terms of a pair are
//     key   : xh xh xl xl  yh yh yl yl  zh zh zl zl  n0 n1 n2 0
//     query : Xh Xl Xh Xl  Yh Yl Yh Yl  Zh Zl Zh Zl  1  1  1  0      (X = -2 q'x, ...)
// i.e. all four piece products of every coordinate plus |k'|^2. Products of two fp16
// values are exact in fp32. With u = 2^-24, R = (max|k'| + |q'|)^2:
//     pieces dropped from 2 q'.k'    2 * 2^-23 * sum |x||X| <= 2^-21 |q'||k'| <=    2 u R
//     the pieces' absolute floor     2^-25 * (sum |X| + sum |x|) <= 1.75 u (max|k'| + |q'|)
//                                    <= 7 u R given max|k'| >= 1/4                   7 u R
//     |k'|^2 as staged                                                            3.2 u R
//     the matrix core's 16 additions                                               33 u R
//     canonical d2 against the exact distance of the centred points               7.1 u R
// so |s + |q'|^2 - canonical d2| <= E = 52.3 u R, and a key whose canonical distance
// equals the minimum has s <= min(s) + 2 E. The kernel uses slack = 128 u R = 2^-17 R
// (+ 1e-36 in the caller's units against underflow of the canonical distance).
// A query beyond fp16's range (|q'| > 16000) goes to the exact scan.
//
// The floor of the pieces is why max|k'| >= 1/4 is required and checked: a key cloud whose
// keys all sit within 0.02 of the centre at this scale has scores off by a thousand u R. Here
// the scale comes from the sampled extent, a sampled key lies on the sample's bounding box,
// so max|k'| >= 1 unless the sample has no extent; then (scale 1) a cloud with
// 0 < max|k'| < 1/2 takes the exact sweep.
//
// The additions. The matrix core aligns the 16 products to the largest exponent among them
// and cuts them off about 25 bits below it, where a product's exponent is the sum of its
// factors' exponent fields: a subnormal fp16 factor counts as 2^-14 however small it is.
// With m(v) = max(|v|, 2^-14) for v != 0, the budget is one unit in the last place of the
// running sum per addition, |result - sum a_i b_i| <= 32 u sum m(a_i) m(b_i) (measured: 4.5 u;
// against true magnitudes the error reaches 147 u times the largest product when subnormal
// and huge factors meet). For the terms above a subnormal piece is seen as at most 2^-14 times
// the other factor, below 2^-10 R per term given max|k'| >= 1/4, so the sum of seen magnitudes
// is below 1.02 R. tests/test_gpu_mfma_bound.py checks the budget and the whole score against
// exact arithmetic on this GPU.
//
// Layout. In the 32 x 32 result a lane holds 16 keys (rows 8a + 4h + c, a, c < 4, h =
// lane / 32) of one query (column lane % 32): lanes l and l + 32 serve the same query
// on disjoint halves of the keys, each with its own three smallest group minima, and
// their exact results are merged at the end (smaller distance, then lower index). A
// wave keeps NQB blocks of 32 queries, so one LDS read of a key tile (16 bytes per
// lane, conflict-free) feeds NQB matrix instructions. The vector ALU only folds the 16
// results of an instruction into the running minimum (8 v_min3) and, every 4 tiles
// (a group of 128 keys), updates the three smallest group minima as above. A matrix
// instruction and its 8 v_min3 take 32 clocks each on a SIMD and run side by side: the
// loop issues the matrix instruction of the next step into a second set of result
// registers before it folds the current set.
//
// Everything after the sweep is the scheme of the kernel above: at most two candidate
// groups per half are re-evaluated with the canonical arithmetic in ascending key
// order, three or more send the query to the exact scan, non-finite or out-of-range input
// takes the exact sweep. Results are bit-identical to the exact sweep for every input.
// The two 16-byte halves of a key's 16 terms; n = |k'|^2. A key past the end gets
// |k'|^2 = +inf.
__device__ __forceinline__ void chamfer_key_terms(float x, float y, float z, float n, bool exists,
                                                  uint4 &half0, uint4 &half1)
{
    const unsigned sx = tk_f16_split2(x), sy = tk_f16_split2(y), sz = tk_f16_split2(z);
    const unsigned n0 = tk_f16_bits(n);
    const float r1 = n - tk_f16_value(n0);
    const unsigned n1 = tk_f16_bits(r1);
    const unsigned n2 = tk_f16_bits(r1 - tk_f16_value(n1));
    const unsigned xh = sx & 0xffffu, xl = sx >> 16, yh = sy & 0xffffu, yl = sy >> 16;
    const unsigned zh = sz & 0xffffu, zl = sz >> 16;
    half0 = make_uint4(xh * 0x10001u, xl * 0x10001u, yh * 0x10001u, yl * 0x10001u);
    half1 = make_uint4(zh * 0x10001u, zl * 0x10001u, n0 | (n1 << 16), n2);
    if (!exists) {
        half0 = make_uint4(0u, 0u, 0u, 0u);
        half1 = make_uint4(0u, 0u, 0x7c00u, 0u);  // n0 = +inf
    }
}

// The query side of the 16 terms for half h of the lanes (q' = centred, scaled query).
__device__ __forceinline__ uint4 chamfer_query_terms(float qx, float qy, float qz, int h)
{
    const unsigned sx = tk_f16_split2(-2.0f * qx), sy = tk_f16_split2(-2.0f * qy);
    const unsigned sz = tk_f16_split2(-2.0f * qz);
    return h == 0 ? make_uint4(sx, sx, sy, sy) : make_uint4(sz, sz, 0x3c003c00u, 0x00003c00u);
}

// Folds the 16 results of a matrix instruction into m.
__device__ __forceinline__ float chamfer_fold16(float m, const tk_f32x16 &acc)
{
#pragma unroll
    for (int r = 0; r < 16; r += 2)
        m = __builtin_fminf(__builtin_fminf(m, acc[r]), acc[r + 1]);
    return m;
}

// One workgroup's share: query block `qblock` of batch element `b` against key slice
// `slice` of direction `d`.
template <int NQB, int BLOCK, int STAGE, bool SOA = false>
__device__ __forceinline__ void chamfer_mfma_block(const ChamferDir<float> &d, const int b,
                                                   const int qblock, const int slice)
{
    constexpr int NW = BLOCK / TK_WAVE;
    constexpr int QB = NW * NQB * 32;  // queries per workgroup
    constexpr int GROUP = 128;         // keys per group: 4 tiles of 32
    constexpr int TILES = STAGE / 32;
    constexpr int PER = STAGE / BLOCK;
    constexpr int MAX_SCANS = 96;
    constexpr int SAMPLES = 4;         // keys per lane in the sample that places the centre
    static_assert(STAGE % GROUP == 0 && STAGE % BLOCK == 0 && QB % BLOCK == 0, "shapes");
    static_assert(NQB % 2 == 0, "the loop alternates between two sets of result registers");
    // Two stage buffers of key terms, [tile][half][key in tile] x 16 bytes; the exact
    // sweep (the way out for input the bound does not cover) reuses them.
    __shared__ __align__(16) uint4 sterm[2 * STAGE * 2];
    static_assert(sizeof(uint4) * 2 * STAGE * 2 >= sizeof(float) * (512 * 4 + 8), "exact sweep stage");
    __shared__ float sred[NW][8];
    __shared__ int sidx[NW];
    __shared__ int s_list[MAX_SCANS];
    __shared__ int s_count;

    const int tid = threadIdx.x;
    const int lane = tid & (TK_WAVE - 1);
    const int wave = tid / TK_WAVE;
    const int col = lane & 31, half = lane >> 5;
    const int nq = d.nq;
    const int k0 = slice * d.slice_len;
    const int nk = (d.nk - k0 < d.slice_len) ? d.nk - k0 : d.slice_len;
    const float *__restrict__ Q = d.query + (int64_t)b * nq * 3;
    const float *__restrict__ K = chamfer_key_base<SOA, float>(d.key, b, d.nk, k0);
    const float INF = __builtin_huge_valf();

    // ---- centre and scale from a strided sample of the key cloud ----
    float lo[3] = {INF, INF, INF}, hi[3] = {-INF, -INF, -INF};
    if (nk > 0) {
        TkPoint3<float> sp[SAMPLES];
#pragma unroll
        for (int r = 0; r < SAMPLES; ++r) {
            const int j = (int)(((int64_t)(r * BLOCK + tid) * nk) / (SAMPLES * BLOCK));
            sp[r] = chamfer_point<SOA, float>(K, d.nk, j);
        }
#pragma unroll
        for (int r = 0; r < SAMPLES; ++r) {
            const float v[3] = {sp[r].x, sp[r].y, sp[r].z};
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                // (not fmin / fmax: a NaN must reach the test below)
                lo[a] = v[a] < lo[a] ? v[a] : (v[a] == v[a] ? lo[a] : v[a]);
                hi[a] = v[a] > hi[a] ? v[a] : (v[a] == v[a] ? hi[a] : v[a]);
            }
        }
    }
    // NaN-propagating reductions: min / max of (value, partner) written with compares
#pragma unroll
    for (int a = 0; a < 3; ++a) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ol = __shfl_xor(lo[a], o), oh = __shfl_xor(hi[a], o);
            lo[a] = (ol < lo[a] || ol != ol) ? ol : lo[a];
            hi[a] = (oh > hi[a] || oh != oh) ? oh : hi[a];
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            sred[wave][a] = lo[a];
            sred[wave][3 + a] = hi[a];
        }
    }
    if (tid == 0)
        s_count = 0;
    __syncthreads();
    float cc[3], ext = 0.0f;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        float l = sred[0][a], h = sred[0][3 + a];
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            const float ol = sred[w][a], oh = sred[w][3 + a];
            l = (ol < l || ol != ol) ? ol : l;
            h = (oh > h || oh != oh) ? oh : h;
        }
        cc[a] = 0.5f * l + 0.5f * h;
        const float e = 0.5f * h - 0.5f * l;
        ext = (e > ext || e != e) ? e : ext;
    }
    const float c0 = cc[0], c1 = cc[1], c2 = cc[2];
    // scale = 2^-(exponent of the sampled half extent), the exponent within [-40, 40]
    // (a sample of identical points: scale 1). Outside, or with anything non-finite in
    // the sample: exact sweep.
    const int ebits = (int)((__builtin_bit_cast(unsigned, ext) >> 23) & 0xffu) - 127;
    const bool safe = nk > 0 && (c0 - c0 == 0.0f) && (c1 - c1 == 0.0f) && (c2 - c2 == 0.0f) &&
                      (ext - ext == 0.0f) && (ext == 0.0f || (ebits >= -40 && ebits <= 40));
    if (!safe) {  // uniform over the workgroup
        chamfer_exact_sweep<float, QB / BLOCK, BLOCK, 64, 512, SOA>(
            d, b, qblock, slice, reinterpret_cast<float *>(sterm));
        return;
    }
    const float scale =
        ext == 0.0f ? 1.0f : __builtin_bit_cast(float, (unsigned)(127 - ebits) << 23);

    // ---- queries: block g of the wave, column `col`; both halves of the lanes load it ----
    tk_f16x8 qterm[NQB];
    float qnorm[NQB];  // |q'| with a margin for its rounding; > 16000 or NaN: not filtered
    float v0[NQB], v1[NQB], v2[NQB];
    int id0[NQB], id1[NQB];
#pragma unroll
    for (int g = 0; g < NQB; ++g) {
        const int qi = qblock * QB + (wave * NQB + g) * 32 + col;
        const bool ok = qi < nq;
        const float px = ((ok ? chamfer_coord<SOA, float>(Q, nq, qi, 0) : c0) - c0) * scale;
        const float py = ((ok ? chamfer_coord<SOA, float>(Q, nq, qi, 1) : c1) - c1) * scale;
        const float pz = ((ok ? chamfer_coord<SOA, float>(Q, nq, qi, 2) : c2) - c2) * scale;
        qnorm[g] =
            1.000001f * __builtin_sqrtf(__builtin_fmaf(pz, pz, __builtin_fmaf(py, py, px * px)));
        const bool in_range = qnorm[g] <= 16000.0f;  // false for NaN
        qterm[g] = __builtin_bit_cast(
            tk_f16x8, chamfer_query_terms(in_range ? px : 0.0f, in_range ? py : 0.0f,
                                          in_range ? pz : 0.0f, half));
        v0[g] = v1[g] = v2[g] = INF;
        id0[g] = id1[g] = -1;
    }

    // ---- sweep ----
    const int nstages = (nk + STAGE - 1) / STAGE;
    float pre[PER][3];
    float kmax2 = 0.0f;  // largest |k'|^2 this lane has staged (NaN keys never match: skipped)
    auto fetch = [&](int st) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int kj = st * STAGE + r * BLOCK + tid;
            pre[r][0] = c0;
            pre[r][1] = c1;
            pre[r][2] = c2;
            if (kj < nk) {
                const TkPoint3<float> p = chamfer_point<SOA, float>(K, d.nk, kj);
                pre[r][0] = p.x;
                pre[r][1] = p.y;
                pre[r][2] = p.z;
            }
        }
    };
    auto stash = [&](int st, int buf) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int j = r * BLOCK + tid;  // key within the stage
            const float x = (pre[r][0] - c0) * scale;
            const float y = (pre[r][1] - c1) * scale;
            const float z = (pre[r][2] - c2) * scale;
            const float n = __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x));
            kmax2 = __builtin_fmaxf(kmax2, n);
            uint4 h0, h1;
            chamfer_key_terms(x, y, z, n, st * STAGE + j < nk, h0, h1);
            uint4 *tile = sterm + buf * (STAGE * 2) + (j >> 5) * 64 + (j & 31);
            tile[0] = h0;
            tile[32] = h1;
        }
    };
    __syncthreads();
    fetch(0);
    stash(0, 0);
    __syncthreads();
    const tk_f32x16 zero = {};
    for (int st = 0; st < nstages; ++st) {
        if (st + 1 < nstages)
            fetch(st + 1);
        const uint4 *sbuf = sterm + (st & 1) * (STAGE * 2) + lane;
        const int left = nk - st * STAGE;
        const int cnt = left < STAGE ? left : STAGE;
        const int ntiles = (cnt + GROUP - 1) / GROUP * (GROUP / 32);  // whole groups
        float tmin[NQB];
#pragma unroll
        for (int g = 0; g < NQB; ++g)
            tmin[g] = INF;
        // Two sets of result registers: the matrix instruction of the next step is
        // issued before the minima of the current one are taken (the barriers keep the
        // compiler from putting the two back in sequence on one set).
        tk_f16x8 ka = __builtin_bit_cast(tk_f16x8, sbuf[0]);
        tk_f32x16 acc[2];
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qterm[0], zero, 0, 0, 0);
#pragma unroll 4
        for (int t = 0; t < ntiles; ++t) {
            // (the read after the last tile wraps to tile 0: one wasted instruction)
            const tk_f16x8 kn =
                __builtin_bit_cast(tk_f16x8, sbuf[((t + 1) & (TILES - 1)) * 64]);
#pragma unroll
            for (int g = 0; g < NQB; ++g) {
                acc[(g + 1) & 1] =
                    g + 1 < NQB
                        ? __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qterm[g + 1 < NQB ? g + 1 : 0],
                                                                  zero, 0, 0, 0)
                        : __builtin_amdgcn_mfma_f32_32x32x16_f16(kn, qterm[0], zero, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                const float m = chamfer_fold16(tmin[g], acc[g & 1]);
                tmin[g] = m;
                if ((t & 3) == 3) {
                    // three smallest group minima (ties keep the earlier group in front)
                    const int group_id = st * (STAGE / GROUP) + (t >> 2);
                    const float x = m;
                    const bool lt0 = x < v0[g];
                    const bool lt1 = x < v1[g];
                    id1[g] = lt1 ? group_id : id1[g];
                    id1[g] = lt0 ? id0[g] : id1[g];
                    id0[g] = lt0 ? group_id : id0[g];
                    v2[g] = __builtin_amdgcn_fmed3f(v1[g], v2[g], x);
                    v1[g] = __builtin_amdgcn_fmed3f(v0[g], v1[g], x);
                    v0[g] = __builtin_amdgcn_fmed3f(-INF, v0[g], x);
                    tmin[g] = INF;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            ka = kn;
        }

        if (st + 1 < nstages) {
            __syncthreads();  // (the other buffer was read during the previous stage)
            stash(st + 1, (st + 1) & 1);
        }
        __syncthreads();

        // One look, an eighth of the way in: if a quarter of the lanes already see three
        // groups within the slack (taken with the largest key norm so far), the cloud is
        // quantised and will not get better.
        if (nstages >= 8 && st == (nstages >> 3)) {
            const float kmax_wave = wave_reduce_max(kmax2);
            if (lane == 0)
                sred[wave][6] = kmax_wave;
            __syncthreads();
            float kmax_now = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w)
                kmax_now = __builtin_fmaxf(kmax_now, sred[w][6]);
            kmax_now = __builtin_sqrtf(kmax_now) * 1.000001f;
            int tied = 0;
#pragma unroll
            for (int g = 0; g < NQB; ++g) {
                const int qi = qblock * QB + (wave * NQB + g) * 32 + col;
                const float r = kmax_now + qnorm[g];
                const bool t3 = qi < nq && v2[g] <= v0[g] + r * r * 7.6293945e-06f;
                tied += __builtin_popcountll(__builtin_amdgcn_ballot_w64(t3));
            }
            if (lane == 0)
                atomicAdd(&s_count, tied);
            __syncthreads();
            const int total = s_count;
            __syncthreads();
            if (tid == 0)
                s_count = 0;
            if (total * 4 > 2 * QB) {  // uniform over the workgroup
                chamfer_exact_sweep<float, QB / BLOCK, BLOCK, 64, 512, SOA>(
                    d, b, qblock, slice, reinterpret_cast<float *>(sterm));
                return;
            }
        }
    }

    // ---- the largest centred key norm; a key cloud that left fp16's range ----
    kmax2 = wave_reduce_max(kmax2);
    if (lane == 0)
        sred[wave][6] = kmax2;
    __syncthreads();
    kmax2 = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w)
        kmax2 = __builtin_fmaxf(kmax2, sred[w][6]);
    // (also +inf; and keys that all differ from the centre by far less than 1 - a sample of
    // identical keys, scale 1, beside keys that differ a little: the fp16 terms have no
    // precision for those; with a sample that has an extent max|k'| >= 1)
    if (!(kmax2 <= 32768.0f) || (kmax2 > 0.0f && kmax2 < 0.25f)) {  // uniform
        chamfer_exact_sweep<float, QB / BLOCK, BLOCK, 64, 512, SOA>(
            d, b, qblock, slice, reinterpret_cast<float *>(sterm));
        return;
    }
    const float kmax = __builtin_sqrtf(kmax2) * 1.000001f;
    const float guard = 1e-36f * scale * scale;  // scale^2 <= 2^80

    // ---- epilogue: exact evaluation of each half's candidate groups, then the merge ----
    // runs of 4 keys: 48 bytes of a [N,3] cloud, 16 bytes of each coordinate of a [3,N] one
    const bool k_aligned =
        (reinterpret_cast<uintptr_t>(K) & 15) == 0 && (!SOA || (d.nk & 3) == 0);
    float qx[NQB], qy[NQB], qz[NQB];
#pragma unroll
    for (int g = 0; g < NQB; ++g) {
        const int qi = qblock * QB + (wave * NQB + g) * 32 + col;
        const bool ok = qi < nq;
        qx[g] = ok ? chamfer_coord<SOA, float>(Q, nq, qi, 0) : 0.0f;
        qy[g] = ok ? chamfer_coord<SOA, float>(Q, nq, qi, 1) : 0.0f;
        qz[g] = ok ? chamfer_coord<SOA, float>(Q, nq, qi, 2) : 0.0f;
    }
#pragma unroll
    for (int g = 0; g < NQB; ++g) {
        const int slot = (wave * NQB + g) * 32 + col;
        const int qi = qblock * QB + slot;
        const bool ok = qi < nq;
        const float best_score = __builtin_fminf(v0[g], __shfl_xor(v0[g], 32));
        const float r = kmax + qnorm[g];
        const float thr = best_score + (r * r * 7.6293945e-06f + guard);  // 2^-17 R
        const bool filtered = qnorm[g] <= 16000.0f;  // false for NaN / inf / out of range
        // No finite score at all (nk == 0 or every key NaN): the exact result is (+inf, -1).
        const bool none = filtered && !(best_score < INF);
        const bool crowded = v2[g] <= thr;  // three or more candidate groups in this half
        const bool over =
            ok && !none && (!filtered || (__builtin_amdgcn_ballot_w64(crowded) >> col & 0x100000001ull));
        float bestd = INF;
        int bestj = -1;
        if (ok && !none && !over) {
            int ta = v0[g] <= thr ? id0[g] : -1, tb = v1[g] <= thr ? id1[g] : -1;
            if (tb >= 0 && (ta < 0 || tb < ta)) {
                const int tmp = ta;
                ta = tb;
                tb = tmp;
            }
            for (int pass = 0; pass < 2; ++pass) {
                const int group = pass == 0 ? ta : tb;
                if (group < 0)
                    continue;
                // this half's keys of the group: runs of 4 keys, 8 keys apart
                if (k_aligned && (group + 1) * GROUP <= nk) {
                    const float4 *p4 = reinterpret_cast<const float4 *>(
                        K + (int64_t)(group * GROUP + half * 4) * (SOA ? 1 : 3));
                    const int plane4 = d.nk >> 2;  // ([3,N]: quads between the coordinates)
#pragma unroll
                    for (int r0 = 0; r0 < GROUP / 8; r0 += 4) {
                        float4 f[4][3];
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr) {
                            if constexpr (SOA) {  // x, y, z of 4 keys; runs 32 bytes apart
                                f[rr][0] = p4[(r0 + rr) * 2];
                                f[rr][1] = p4[(r0 + rr) * 2 + plane4];
                                f[rr][2] = p4[(r0 + rr) * 2 + 2 * plane4];
                            } else {  // a run is 48 bytes, runs 96 bytes apart
                                f[rr][0] = p4[(r0 + rr) * 6 + 0];
                                f[rr][1] = p4[(r0 + rr) * 6 + 1];
                                f[rr][2] = p4[(r0 + rr) * 6 + 2];
                            }
                        }
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr) {
                            const int j = group * GROUP + (r0 + rr) * 8 + half * 4;
                            const float4 f0 = f[rr][0], f1 = f[rr][1], f2 = f[rr][2];
                            const float dd0 = SOA ? tk_dist2<float>(f0.x, f1.x, f2.x, qx[g], qy[g], qz[g])
                                                  : tk_dist2<float>(f0.x, f0.y, f0.z, qx[g], qy[g], qz[g]);
                            const float dd1 = SOA ? tk_dist2<float>(f0.y, f1.y, f2.y, qx[g], qy[g], qz[g])
                                                  : tk_dist2<float>(f0.w, f1.x, f1.y, qx[g], qy[g], qz[g]);
                            const float dd2 = SOA ? tk_dist2<float>(f0.z, f1.z, f2.z, qx[g], qy[g], qz[g])
                                                  : tk_dist2<float>(f1.z, f1.w, f2.x, qx[g], qy[g], qz[g]);
                            const float dd3 = SOA ? tk_dist2<float>(f0.w, f1.w, f2.w, qx[g], qy[g], qz[g])
                                                  : tk_dist2<float>(f2.y, f2.z, f2.w, qx[g], qy[g], qz[g]);
                            if (dd0 < bestd) { bestd = dd0; bestj = j; }
                            if (dd1 < bestd) { bestd = dd1; bestj = j + 1; }
                            if (dd2 < bestd) { bestd = dd2; bestj = j + 2; }
                            if (dd3 < bestd) { bestd = dd3; bestj = j + 3; }
                        }
                    }
                } else {
                    for (int run = 0; run < GROUP / 8; ++run) {
                        const int j = group * GROUP + run * 8 + half * 4;
                        for (int e = j; e < j + 4 && e < nk; ++e) {
                            const TkPoint3<float> p = chamfer_point<SOA, float>(K, d.nk, e);
                            const float dd = tk_dist2<float>(p.x, p.y, p.z, qx[g], qy[g], qz[g]);
                            if (dd < bestd) {
                                bestd = dd;
                                bestj = e;
                            }
                        }
                    }
                }
            }
        }
        // the other half's result: smaller distance, then lower key index
        const float od = __shfl_xor(bestd, 32);
        const int oj = __shfl_xor(bestj, 32);
        if (oj >= 0 && (bestj < 0 || od < bestd || (od == bestd && oj < bestj))) {
            bestd = od;
            bestj = oj;
        }
        if (half == 0) {
            if (ok && !over)
                chamfer_emit<float>(d, b, qi, k0, bestd, bestj);
            if (over) {
                const int at = atomicAdd(&s_count, 1);
                if (at < MAX_SCANS)
                    s_list[at] = slot;
            }
        }
    }

    // ---- queries with three or more candidate groups in a half, or out of range ----
    __syncthreads();
    const int nscan = s_count;
    if (nscan > MAX_SCANS) {  // uniform over the workgroup
        chamfer_exact_sweep<float, QB / BLOCK, BLOCK, 64, 512, SOA>(
            d, b, qblock, slice, reinterpret_cast<float *>(sterm));
        return;
    }
    for (int e = 0; e < nscan; ++e) {
        const int qi = qblock * QB + s_list[e];
        float bd;
        int bj;
        chamfer_block_exact_scan<BLOCK, SOA>(K, nk, chamfer_coord<SOA, float>(Q, nq, qi, 0),
                                             chamfer_coord<SOA, float>(Q, nq, qi, 1),
                                             chamfer_coord<SOA, float>(Q, nq, qi, 2), &sred[0][0],
                                             sidx, bd, bj, d.nk);
        if (tid == 0)
            chamfer_emit<float>(d, b, qi, k0, bd, bj);
    }
}

template <int NQB, int BLOCK, int STAGE, bool SOA = false>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(4, 4))) void
chamfer_forward_mfma_kernel(ChamferFwdArgs<float> args)
{
    int b, qblock, slice;
    const ChamferDir<float> &d = chamfer_decode_block<float>(args, b, qblock, slice);
    chamfer_mfma_block<NQB, BLOCK, STAGE, SOA>(d, b, qblock, slice);
}

// The same sweep for the clouds another kernel has flagged (args.only_if: a word per
// direction and batch element, then one that is set when any of them is): a fixed, small
// number of workgroups go through all (direction, batch element, query block) shares and
// work on those whose cloud carries a flag; a launch that finds no flag at all leaves at
// once.
template <int NQB, int BLOCK, int STAGE, bool SOA = false>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(4, 4))) void
chamfer_forward_mfma_flagged_kernel(ChamferFwdArgs<float> args, int total)
{
    if (args.only_if[2 * args.nbatch] == 0)  // no cloud carries a flag: nothing to do
        return;
    // Shares of the two directions alternate (as far as the shorter one reaches): often only
    // one direction carries flags, and its workgroups should not be neighbours on the chip.
    const int n0 = args.nblocks0, n1 = total - args.nblocks0, both = n0 < n1 ? n0 : n1;
    for (int lb = blockIdx.x; lb < total; lb += gridDim.x) {
        const int which = lb < 2 * both ? (lb & 1) : (n0 > n1 ? 0 : 1);
        const int rest0 = lb < 2 * both ? (lb >> 1) : lb - both;
        const ChamferDir<float> &d = args.dir[which];
        const int b = rest0 / d.blocks_per_batch;
        const int rest = rest0 - b * d.blocks_per_batch;
        const int qblock = rest / d.slices, slice = rest - qblock * d.slices;
        if (args.only_if[which * args.nbatch + b] == 0)  // uniform over the workgroup
            continue;
        chamfer_mfma_block<NQB, BLOCK, STAGE, SOA>(d, b, qblock, slice);
        __syncthreads();  // the next share reuses the stage buffers
    }
}

// ---- backward ----------------------------------------------------------------
// Pass A ("own" terms): every point i of cloud 1 has exactly one term
// 2*gd1[i]*(x1[i]-x2[idx1[i]]) addressed to itself, so it is written with a plain
// store; same for cloud 2. Pass B ("scattered" terms): the negated term goes to
// the matched point of the other cloud, where several sources can meet, and is
// added with a hardware fp atomic. Pass B runs after pass A on the same stream.
template <typename T>
__global__ __launch_bounds__(256) void chamfer_backward_own_kernel(
    const T *__restrict__ gd1, const T *__restrict__ gd2, const T *__restrict__ xyz1,
    const T *__restrict__ xyz2, const int64_t *__restrict__ idx1,
    const int64_t *__restrict__ idx2, int64_t total1, int64_t total2, int n1, int n2,
    T *__restrict__ gx1, T *__restrict__ gx2)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
         lin < total1 + total2; lin += stride) {
        const bool second = lin >= total1;
        const int64_t p = second ? lin - total1 : lin;
        const int na = second ? n2 : n1, nb = second ? n1 : n2;
        const T *__restrict__ xa = second ? xyz2 : xyz1;
        const T *__restrict__ xb = second ? xyz1 : xyz2;
        const T *__restrict__ gd = second ? gd2 : gd1;
        const int64_t *__restrict__ ix = second ? idx2 : idx1;
        T *__restrict__ ga = second ? gx2 : gx1;
        const int64_t b = p / na;
        const int64_t j = ix[p];
        T vx = 0, vy = 0, vz = 0;
        if (j >= 0 && j < nb) {
            const T g = gd[p] * 2;
            const T *pa = xa + p * 3;
            const T *pb = xb + (b * nb + j) * 3;
            vx = g * (pa[0] - pb[0]);
            vy = g * (pa[1] - pb[1]);
            vz = g * (pa[2] - pb[2]);
        }
        ga[p * 3 + 0] = vx;
        ga[p * 3 + 1] = vy;
        ga[p * 3 + 2] = vz;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void chamfer_backward_scatter_kernel(
    const T *__restrict__ gd1, const T *__restrict__ gd2, const T *__restrict__ xyz1,
    const T *__restrict__ xyz2, const int64_t *__restrict__ idx1,
    const int64_t *__restrict__ idx2, int64_t total1, int64_t total2, int n1, int n2,
    T *gx1, T *gx2)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
         lin < total1 + total2; lin += stride) {
        const bool second = lin >= total1;
        const int64_t p = second ? lin - total1 : lin;
        const int na = second ? n2 : n1, nb = second ? n1 : n2;
        const T *__restrict__ xa = second ? xyz2 : xyz1;
        const T *__restrict__ xb = second ? xyz1 : xyz2;
        const T *__restrict__ gd = second ? gd2 : gd1;
        const int64_t *__restrict__ ix = second ? idx2 : idx1;
        T *gb = second ? gx1 : gx2;
        const int64_t b = p / na;
        const int64_t j = ix[p];
        if (j < 0 || j >= nb)
            continue;
        const T g = gd[p] * 2;
        const T *pa = xa + p * 3;
        const T *pb = xb + (b * nb + j) * 3;
        T *dst = gb + (b * nb + j) * 3;
        unsafeAtomicAdd(dst + 0, -(g * (pa[0] - pb[0])));
        unsafeAtomicAdd(dst + 1, -(g * (pa[1] - pb[1])));
        unsafeAtomicAdd(dst + 2, -(g * (pa[2] - pb[2])));
    }
}

// fp32 backward without global atomics, in one launch. A workgroup owns a range of
// R points of one cloud X in one batch and produces their gradients completely:
//   grad_X[j] = 2 gX[j] (x_j - y_{idxX[j]})                     the point's own term
//             - sum_{i : idxY[i] = j} 2 gY[i] (y_i - x_j)       terms sent by cloud Y
// It scans all of cloud Y's matches, accumulates those that land in its range in
// 64-bit fixed-point LDS accumulators (integer LDS atomics run an order of
// magnitude faster than floating-point ones on this GPU, and make the sum
// independent of arrival order), adds the own term and stores each gradient once.
// The senders are taken in rounds of NT * U, a round being U runs of NT consecutive
// senders spread evenly over the cloud. Scale: a power of two chosen from the largest
// |term| of the first round's senders times 8 (those terms are in registers by then,
// so the choice costs no pass of its own); a term above that bound raises a flag and
// the workgroup repeats with the bound over all senders. Non-finite input takes the
// floating-point path.
// The own terms are fetched first, while the accumulators are cleared and the first
// match indices arrive, and meet the sums at the end.
template <int R, int NT>
__global__ __launch_bounds__(NT) void chamfer_backward_fixed_kernel(
    const float *__restrict__ gd1, const float *__restrict__ gd2,
    const float *__restrict__ xyz1, const float *__restrict__ xyz2,
    const int64_t *__restrict__ idx1, const int64_t *__restrict__ idx2, int n1, int n2,
    int ranges1, int ranges2, float *__restrict__ gx1, float *__restrict__ gx2)
{
    extern __shared__ __align__(16) unsigned long long acc[];  // [R * 3], then the range
    float *sx = reinterpret_cast<float *>(acc + R * 3);        // of X itself: [R * 3] floats
    __shared__ unsigned s_max;
    __shared__ int s_exceeded;
    const double MAGIC = 6755399441055744.0;  // 1.5 * 2^52
    constexpr int U = 8;           // senders per lane and round
    constexpr int F = R / NT;      // points of the range per lane
    static_assert(R % NT == 0 && R * 3 % (2 * NT) == 0, "whole steps of the workgroup");

    // Decode: a batch's ranges1 + ranges2 workgroups are consecutive logical workgroups
    // (first those that produce grad_xyz1), and each XCD takes a contiguous run of logical
    // workgroups (blockIdx goes round-robin over the 8 XCDs): every workgroup of a batch
    // reads both clouds, both gradients and both index arrays of that batch, which then
    // come from HBM once and from the XCD's L2 afterwards.
    int lb = blockIdx.x;
    {
        const int per = (int)gridDim.x >> 3, full = per << 3;
        if (lb < full)
            lb = (lb & 7) * per + (lb >> 3);
    }
    const int tid = threadIdx.x;
    const int b = lb / (ranges1 + ranges2);
    const int r = lb - b * (ranges1 + ranges2);
    const bool second = r >= ranges1;
    const int j0 = (second ? r - ranges1 : r) * R;
    const int nx = second ? n2 : n1, ny = second ? n1 : n2;
    const float *__restrict__ X = (second ? xyz2 : xyz1) + (int64_t)b * nx * 3;
    // An empty opposite cloud has no storage (its base may be NULL) and sends nothing; the
    // loads below that fetch a placeholder element before testing the match index then
    // read this cloud's own first point instead.
    const float *__restrict__ Y =
        ny > 0 ? (second ? xyz1 : xyz2) + (int64_t)b * ny * 3 : X;
    const float *__restrict__ gX = (second ? gd2 : gd1) + (int64_t)b * nx;
    const float *__restrict__ gY = (second ? gd1 : gd2) + (int64_t)b * ny;
    const int64_t *__restrict__ iX = (second ? idx2 : idx1) + (int64_t)b * nx;
    const int64_t *__restrict__ iY = (second ? idx1 : idx2) + (int64_t)b * ny;
    float *__restrict__ out = (second ? gx2 : gx1) + (int64_t)b * nx * 3;
    const int j1 = (j0 + R < nx) ? j0 + R : nx;
    const int rounds = (ny + NT * U - 1) / (NT * U);

    // Everything is fetched through buffer descriptors: a 32-bit offset per element against
    // a base in scalar registers, where 64-bit addresses for the gathers of a round would
    // not fit the register file beside the data (the host sends clouds whose byte offsets
    // pass 2^31 to the other kernels).
    auto rsrc = [](const void *p, int64_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t rX = rsrc(X, (int64_t)nx * 12);
    const __amdgpu_buffer_rsrc_t rY = rsrc(Y, (int64_t)(ny > 0 ? ny : 1) * 12);
    const __amdgpu_buffer_rsrc_t rgX = rsrc(gX, (int64_t)nx * 4);
    const __amdgpu_buffer_rsrc_t rgY = rsrc(gY, (int64_t)ny * 4);
    const __amdgpu_buffer_rsrc_t riX = rsrc(iX, (int64_t)nx * 8);
    const __amdgpu_buffer_rsrc_t riY = rsrc(iY, (int64_t)ny * 8);
    typedef float f3 __attribute__((ext_vector_type(3)));
    auto load_f = [](__amdgpu_buffer_rsrc_t rs, int at) {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, at, 0, 0));
    };
    auto load_f3 = [](__amdgpu_buffer_rsrc_t rs, int at) {
        return __builtin_bit_cast(f3, __builtin_amdgcn_raw_buffer_load_b96(rs, at, 0, 0));
    };
    auto load_i64 = [](__amdgpu_buffer_rsrc_t rs, int at) {
        return __builtin_bit_cast(int64_t, __builtin_amdgcn_raw_buffer_load_b64(rs, at, 0, 0));
    };

    // Sender u of a lane in round `round`: runs of NT consecutive senders, the rounds
    // interleaved so that each of them is spread over the whole cloud.
    auto sender = [&](int round, int u) { return tid + NT * (u * rounds + round); };
    // A sender's match as a position within the range, -1 when it lies outside.
    auto load_matches = [&](int round, int (&jj)[U]) {
        int64_t m64[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = sender(round, u);
            m64[u] = load_i64(riY, (i < ny ? i : 0) * 8);
            m64[u] = i < ny ? m64[u] : -1;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            jj[u] = (m64[u] >= j0 && m64[u] < j1) ? (int)(m64[u] - j0) : -1;
    };
    // The negated terms of a round's senders that match inside the range. Senders that
    // match outside it read one fixed element instead (a broadcast), so only the index
    // stream is paid for per range; everything is requested before anything is used. The
    // matched points come from the copy of the range in LDS: fetched from memory, each of
    // these 12-byte reads at a random place pulled a cache line of 128 bytes into the
    // compute unit, and that traffic was what the kernel waited for.
    auto load_terms = [&](int round, const int (&jj)[U], float (&v)[U][3]) {
        float g[U];
        f3 y[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int is = jj[u] >= 0 ? sender(round, u) : 0;
            g[u] = load_f(rgY, is * 4) * 2;
            y[u] = load_f3(rY, is * 12);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float *x = sx + (jj[u] >= 0 ? jj[u] : 0) * 3;  // the matched point, from LDS
            v[u][0] = -(g[u] * (y[u].x - x[0]));
            v[u][1] = -(g[u] * (y[u].y - x[1]));
            v[u][2] = -(g[u] * (y[u].z - x[2]));
        }
    };
    // Adds a round's terms to the accumulators; true when one of them is above the bound.
    auto accumulate = [&](const int (&jj)[U], const float (&v)[U][3], float bound,
                          double scale) {
        bool exceeded = false;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (jj[u] < 0)
                continue;
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                exceeded = exceeded || !(__builtin_fabsf(v[u][a]) <= bound);
                const double d = __builtin_fma((double)v[u][a], scale, MAGIC);
                atomicAdd(&acc[jj[u] * 3 + a],
                          __builtin_bit_cast(unsigned long long, d) -
                              __builtin_bit_cast(unsigned long long, MAGIC));
            }
        }
        return exceeded;
    };
    auto clear = [&]() {
        __syncthreads();
        for (int t = tid; t < R * 3 / 2; t += NT)
            reinterpret_cast<ulonglong2 *>(acc)[t] = make_ulonglong2(0ull, 0ull);
        if (tid == 0) {
            s_max = 0u;
            s_exceeded = 0;
        }
    };
    // one LDS atomic per wave: 64 lanes on one address would be served one by one
    auto workgroup_max = [&](unsigned m) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const unsigned t = (unsigned)__shfl_xor((int)m, o);
            m = t > m ? t : m;
        }
        if ((tid & 63) == 0 && m != 0u)
            atomicMax(&s_max, m);
        __syncthreads();
        return s_max;
    };
    // The power of two that places a term at the bound below 2^50 and leaves room for up to
    // 2^12 of them (more senders than that on one point lower the scale further).
    auto scale_exponent = [&](float bound) {
        int e = 0;
        (void)__builtin_frexpf(bound, &e);
        int log2_count = 1;
        while ((1 << log2_count) < ny + 1)
            ++log2_count;
        return (62 - log2_count < 50 ? 62 - log2_count : 50) - e;
    };

    // ---- the own terms: F points per lane --------------------------------------------------
    float own[F][3];
    int jj[U];
    {
        int mj[F];  // the point's own match, -1 when it has none
        f3 xs[F];
        {
            int64_t m64[F];
#pragma unroll
            for (int f = 0; f < F; ++f) {
                const int j = j0 + tid + f * NT;
                m64[f] = load_i64(riX, (j < j1 ? j : j0) * 8);
                m64[f] = j < j1 ? m64[f] : -1;
            }
            // the lane's points of the range: for its own terms and into LDS for everyone
#pragma unroll
            for (int f = 0; f < F; ++f) {
                const int j = j0 + tid + f * NT;
                xs[f] = load_f3(rX, (j < j1 ? j : j0) * 12);
            }
            if (rounds > 0)
                load_matches(0, jj);
            clear();
#pragma unroll
            for (int f = 0; f < F; ++f) {
                mj[f] = (m64[f] >= 0 && m64[f] < ny) ? (int)m64[f] : -1;
                float *at = sx + (tid + f * NT) * 3;
                at[0] = xs[f].x;
                at[1] = xs[f].y;
                at[2] = xs[f].z;
            }
        }
        __syncthreads();
        float gg[F];
        f3 ys[F];
#pragma unroll
        for (int f = 0; f < F; ++f) {
            const int j = j0 + tid + f * NT;
            gg[f] = load_f(rgX, (j < j1 ? j : j0) * 4);
            ys[f] = load_f3(rY, (mj[f] >= 0 ? mj[f] : 0) * 12);
        }
#pragma unroll
        for (int f = 0; f < F; ++f) {
            own[f][0] = mj[f] >= 0 ? (gg[f] * 2) * (xs[f].x - ys[f].x) : 0.0f;
            own[f][1] = mj[f] >= 0 ? (gg[f] * 2) * (xs[f].y - ys[f].y) : 0.0f;
            own[f][2] = mj[f] >= 0 ? (gg[f] * 2) * (xs[f].z - ys[f].z) : 0.0f;
        }
    }
    // Own term and the exact sum of the sent terms meet in double: the gradient is rounded
    // once. A lane stores the 12 bytes of a point at once, so a wave's store covers 768
    // consecutive bytes.
    auto finish = [&](int kexp) {
        const __amdgpu_buffer_rsrc_t rout = rsrc(out, (int64_t)nx * 12);
#pragma unroll
        for (int f = 0; f < F; ++f) {
            const int p = tid + f * NT;
            if (j0 + p >= j1)
                continue;
            // (kept as three floats until here: converted where they were computed, they
            // would occupy twice the registers through the whole scan)
            asm volatile("" : "+v"(own[f][0]), "+v"(own[f][1]), "+v"(own[f][2]));
            f3 o;
            o.x = (float)((double)own[f][0] +
                          __builtin_ldexp((double)(long long)acc[p * 3 + 0], -kexp));
            o.y = (float)((double)own[f][1] +
                          __builtin_ldexp((double)(long long)acc[p * 3 + 1], -kexp));
            o.z = (float)((double)own[f][2] +
                          __builtin_ldexp((double)(long long)acc[p * 3 + 2], -kexp));
            typedef unsigned u3 __attribute__((ext_vector_type(3)));
            __builtin_amdgcn_raw_buffer_store_b96(__builtin_bit_cast(u3, o), rout, (j0 + p) * 12, 0,
                                                  0);
        }
    };

    // ---- first attempt: the bound comes from the first round ------------------------------
    {
        float v[U][3];
        int jn[U];
        unsigned m = 0u;
        if (rounds > 0) {
            load_terms(0, jj, v);
            if (rounds > 1)
                load_matches(1, jn);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (jj[u] < 0)
                    continue;
#pragma unroll
                for (int a = 0; a < 3; ++a) {
                    const unsigned bits = __builtin_bit_cast(unsigned, v[u][a]) & 0x7fffffffu;
                    m = bits > m ? bits : m;
                }
            }
        }
        const float bound = __builtin_bit_cast(float, workgroup_max(m)) * 8.0f;
        if (bound < 3.0e38f) {  // (else NaN or inf: floating point below)
            const int kexp = scale_exponent(bound);
            const double scale = __builtin_ldexp(1.0, kexp);
            bool exceeded = false;
            for (int round = 0; round < rounds; ++round) {
                exceeded = accumulate(jj, v, bound, scale) || exceeded;
                if (round + 1 < rounds) {
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        jj[u] = jn[u];
                    load_terms(round + 1, jj, v);
                    if (round + 2 < rounds)
                        load_matches(round + 2, jn);
                }
            }
            if (exceeded)
                s_exceeded = 1;
            __syncthreads();
            if (!s_exceeded) {
                finish(kexp);
                return;
            }
        }
    }
    // ---- second attempt: the bound over all senders ---------------------------------------
    {
        clear();
        __syncthreads();
        unsigned m = 0u;
        float v[U][3];
        for (int round = 0; round < rounds; ++round) {
            load_matches(round, jj);
            load_terms(round, jj, v);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (jj[u] < 0)
                    continue;
#pragma unroll
                for (int a = 0; a < 3; ++a) {
                    const unsigned bits = __builtin_bit_cast(unsigned, v[u][a]) & 0x7fffffffu;
                    m = bits > m ? bits : m;
                }
            }
        }
        const float bound = __builtin_bit_cast(float, workgroup_max(m)) * 1.000001f;
        if (bound < 3.0e38f) {
            const int kexp = scale_exponent(bound);
            const double scale = __builtin_ldexp(1.0, kexp);
            bool exceeded = false;
            for (int round = 0; round < rounds; ++round) {
                load_matches(round, jj);
                load_terms(round, jj, v);
                exceeded = accumulate(jj, v, bound, scale) || exceeded;
            }
            if (exceeded)
                s_exceeded = 1;
            __syncthreads();
            if (!s_exceeded) {
                finish(kexp);
                return;
            }
        }
    }

    // Non-finite gradients or coordinates: floating-point LDS accumulation.
    float *facc = reinterpret_cast<float *>(acc);
    __syncthreads();
    for (int t = tid; t < R * 3; t += NT)
        facc[t] = 0.0f;
    __syncthreads();
    for (int i = tid; i < ny; i += NT) {
        const int64_t j = iY[i];
        if (j < j0 || j >= j1)
            continue;
        const float g = gY[i] * 2;
#pragma unroll
        for (int a = 0; a < 3; ++a)
            atomicAdd(&facc[(j - j0) * 3 + a], -(g * (Y[(int64_t)i * 3 + a] - X[j * 3 + a])));
    }
    __syncthreads();
    for (int t = tid; t < (j1 - j0) * 3; t += NT) {
        const int j = j0 + t / 3, a = t - (t / 3) * 3;
        const int64_t jm = iX[j];
        float o = 0.0f;
        if (jm >= 0 && jm < ny)
            o = (gX[j] * 2) * (X[(int64_t)j * 3 + a] - Y[jm * 3 + a]);
        out[(int64_t)j * 3 + a] = o + facc[t];
    }
}

// Split sweeps: the index outputs start as packed (+inf, -1) words ...
__global__ __launch_bounds__(256) void chamfer_split_init_kernel(ChamferFwdArgs<float> args,
                                                                 int64_t total0, int64_t total1)
{
    const unsigned long long word = (0x7f800000ull << 32) | 0xffffffffull;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < total0) {
        if (args.dir[0].slices > 1)
            reinterpret_cast<unsigned long long *>(args.dir[0].idx)[i] = word;
    } else if (i - total0 < total1) {
        if (args.dir[1].slices > 1)
            reinterpret_cast<unsigned long long *>(args.dir[1].idx)[i - total0] = word;
    }
}

// ... and are unpacked into distance and index once every slice has been merged.
__global__ __launch_bounds__(256) void chamfer_split_finish_kernel(ChamferFwdArgs<float> args,
                                                                   int64_t total0, int64_t total1)
{
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int which = i >= total0;
    if (which)
        i -= total0;
    if (i >= (which ? total1 : total0))
        return;
    const ChamferDir<float> &d = args.dir[which];
    if (d.slices <= 1)
        return;
    const unsigned long long word = reinterpret_cast<const unsigned long long *>(d.idx)[i];
    d.dist[i] = __builtin_bit_cast(float, (unsigned)(word >> 32));
    d.idx[i] = (int64_t)(int)(unsigned)word;
}

// A key cloud of `nk` points cut into about `want` slices of whole tiles: returns the
// number of slices and their length.
inline int64_t chamfer_slices(int64_t nk, int64_t want, int tile, int64_t &len)
{
    len = nk;
    if (want <= 1 || nk <= tile)
        return 1;
    len = (nk + want - 1) / want;
    len = (len + tile - 1) / tile * tile;
    return (nk + len - 1) / len;
}

// Fills the launch description. `want_slices` > 1 asks for that many key slices per
// query (fp32 only); each direction gets as many as its key cloud has whole tiles for.
template <typename T, int QB, int TILE>
int chamfer_fill_args(ChamferFwdArgs<T> &a, const T *xyz1, const T *xyz2, int64_t B, int64_t N1,
                      int64_t N2, T *dist1, int64_t *idx1, T *dist2, int64_t *idx2,
                      int want_slices, int64_t &nblocks, int want_slices_dir1 = -1)
{
    // (one count for both directions unless the second is given)
    const int want[2] = {want_slices, want_slices_dir1 < 0 ? want_slices : want_slices_dir1};
    const T *q[2] = {xyz1, xyz2}, *k[2] = {xyz2, xyz1};
    T *dist[2] = {dist1, dist2};
    int64_t *idx[2] = {idx1, idx2};
    const int64_t nq[2] = {N1, N2}, nk[2] = {N2, N1};
    int64_t nb[2];
    for (int w = 0; w < 2; ++w) {
        int64_t len;
        const int64_t slices = chamfer_slices(nk[w], sizeof(T) == 4 ? want[w] : 1, TILE, len);
        const int64_t qblocks = (nq[w] + QB - 1) / QB;
        a.dir[w] = {q[w], k[w], dist[w], idx[w], (int)nq[w], (int)nk[w],
                    (int)(qblocks * slices), (int)slices, (int)(len > 0 ? len : 1)};
        nb[w] = B * qblocks * slices;
    }
    nblocks = nb[0] + nb[1];
    if (nblocks > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    a.nblocks0 = (int)nb[0];
    a.only_if = nullptr;
    a.nbatch = (int)B;
    return TK3D_OK;
}

// Launches `kernel` on the filled description, bracketed by the init / finish kernels
// when any direction is split.
template <typename T, typename Kernel>
int chamfer_forward_run(Kernel kernel, int block, const ChamferFwdArgs<T> &a, int64_t nblocks,
                        int64_t B, hipStream_t stream)
{
    if (nblocks == 0)
        return TK3D_OK;
    bool split = false;
    if constexpr (sizeof(T) == 4) {
        split = a.dir[0].slices > 1 || a.dir[1].slices > 1;
        if (split) {
            const int64_t t0 = B * a.dir[0].nq, t1 = B * a.dir[1].nq;
            if ((t0 + t1 + 255) / 256 > TK_MAX_I32)
                return TK3D_ERR_UNSUPPORTED;
            const unsigned grid = (unsigned)((t0 + t1 + 255) / 256);
            hipLaunchKernelGGL(chamfer_split_init_kernel, dim3(grid), dim3(256), 0, stream, a, t0,
                               t1);
            hipLaunchKernelGGL(kernel, dim3((unsigned)nblocks), dim3(block), 0, stream, a);
            hipLaunchKernelGGL(chamfer_split_finish_kernel, dim3(grid), dim3(256), 0, stream, a,
                               t0, t1);
            return tk_launch_status();
        }
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)nblocks), dim3(block), 0, stream, a);
    return tk_launch_status();
}

template <typename T, int QPL, int BLOCK = 256, int TILE = 32, int STAGE = 1024, bool SOA = false>
int chamfer_forward_launch(const T *xyz1, const T *xyz2, int64_t B, int64_t N1,
                           int64_t N2, T *dist1, int64_t *idx1, T *dist2,
                           int64_t *idx2, hipStream_t stream, int slices = 1)
{
    ChamferFwdArgs<T> a;
    int64_t nblocks;
    const int rc = chamfer_fill_args<T, QPL * BLOCK, TILE>(a, xyz1, xyz2, B, N1, N2, dist1, idx1,
                                                           dist2, idx2, slices, nblocks);
    if (rc != TK3D_OK)
        return rc;
    return chamfer_forward_run<T>(chamfer_forward_kernel<T, QPL, BLOCK, TILE, STAGE, SOA>, BLOCK, a,
                                  nblocks, B, stream);
}

template <int QPL, int BLOCK = 256, int TILE = 64, int STAGE = 1024>
int chamfer_forward_filter_launch(const float *xyz1, const float *xyz2, int64_t B, int64_t N1,
                                  int64_t N2, float *dist1, int64_t *idx1, float *dist2,
                                  int64_t *idx2, hipStream_t stream, int slices = 1)
{
    ChamferFwdArgs<float> a;
    int64_t nblocks;
    const int rc = chamfer_fill_args<float, QPL * BLOCK, TILE>(
        a, xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, slices, nblocks);
    if (rc != TK3D_OK)
        return rc;
    return chamfer_forward_run<float>(chamfer_forward_filter_kernel<QPL, BLOCK, TILE, STAGE>,
                                      BLOCK, a, nblocks, B, stream);
}

// The matrix pre-filter on the clouds flagged in `only_if` ([2, B]), unsplit.
template <int NQB, bool SOA = false, int BLOCK = 256, int STAGE = 512>
int chamfer_forward_mfma_flagged_launch(const float *xyz1, const float *xyz2, int64_t B,
                                        int64_t N1, int64_t N2, float *dist1, int64_t *idx1,
                                        float *dist2, int64_t *idx2, hipStream_t stream,
                                        const int *only_if)
{
    ChamferFwdArgs<float> a;
    int64_t nblocks;
    const int rc = chamfer_fill_args<float, (BLOCK / TK_WAVE) * NQB * 32, 128>(
        a, xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, 1, nblocks, 1);
    if (rc != TK3D_OK)
        return rc;
    a.only_if = only_if;
    const int64_t grid = nblocks < 4 * tk_cu_count() ? nblocks : 4 * tk_cu_count();
    if (grid == 0)
        return TK3D_OK;
    hipLaunchKernelGGL((chamfer_forward_mfma_flagged_kernel<NQB, BLOCK, STAGE, SOA>),
                       dim3((unsigned)grid), dim3(BLOCK), 0, stream, a, (int)nblocks);
    return tk_launch_status();
}

template <int NQB, bool SOA = false, int BLOCK = 256, int STAGE = 512>
int chamfer_forward_mfma_launch(const float *xyz1, const float *xyz2, int64_t B, int64_t N1,
                                int64_t N2, float *dist1, int64_t *idx1, float *dist2,
                                int64_t *idx2, hipStream_t stream, int slices0 = 1, int slices1 = 1)
{
    ChamferFwdArgs<float> a;
    int64_t nblocks;
    const int rc = chamfer_fill_args<float, (BLOCK / TK_WAVE) * NQB * 32, 128>(
        a, xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, slices0, nblocks, slices1);
    if (rc != TK3D_OK)
        return rc;
    return chamfer_forward_run<float>(chamfer_forward_mfma_kernel<NQB, BLOCK, STAGE, SOA>, BLOCK, a,
                                      nblocks, B, stream);
}

// Estimated duration in microseconds of the pre-filtered sweep launched as `qpl`
// queries per lane, `block` lanes per workgroup and `want_slices` key slices; used only
// to rank launch shapes. A wave issues qpl * ipp vector instructions per key (ipp per
// pair: 3.76 measured with 4 queries per lane, 4.5 with 2, which reads LDS and keeps tile
// minima twice as often), plus a prologue and epilogue worth `overhead_keys` keys per
// slice (about 250 for 256-lane workgroups, 500 for 512-lane ones).
// A SIMD with n resident waves finishes them in max(2.4 n, 5.5) cycles per instruction
// of one wave: 2.4 is the issue cost of the instruction mix, 5.5 what a lone wave
// achieves between dependent instructions. Workgroups spread over 256 CUs, so n steps
// with ceil(workgroups / 256). 12 us cover launch and fixed latencies, 20 us with the
// two extra launches of a split sweep. Within 8 % of the best shape (1 % on average) on
// 54 timed shapes from B=1, N=512 to B=32, N=16384 and B=4, N=65536.
inline double chamfer_sweep_cost(int64_t B, int64_t N1, int64_t N2, int qpl, int block,
                                 double ipp, double overhead_keys, int want_slices)
{
    const int64_t nq[2] = {N1, N2}, nk[2] = {N2, N1};
    const int64_t qb = (int64_t)qpl * block;
    double groups = 0.0, instructions = 0.0;
    for (int w = 0; w < 2; ++w) {
        int64_t len;
        const int64_t slices = chamfer_slices(nk[w], want_slices, 64, len);
        const double g = (double)B * (double)((nq[w] + qb - 1) / qb) * (double)slices;
        groups += g;
        instructions += g * qpl * ((double)len + overhead_keys) * ipp;
    }
    if (groups == 0.0)
        return 0.0;
    const double per_wave = instructions / groups;
    const double rounds = (double)(((int64_t)groups + 255) / 256);
    const double resident = rounds * (block / 64) / 4.0;  // waves per SIMD
    const double cycles = per_wave * (2.4 * resident > 5.5 ? 2.4 * resident : 5.5);
    return (want_slices > 1 ? 20.0 : 12.0) + cycles / 2100.0;
}

template <typename T, bool SOA = false>
int chamfer_forward(const T *xyz1, const T *xyz2, int64_t B, int64_t N1, int64_t N2,
                    T *dist1, int64_t *idx1, T *dist2, int64_t *idx2, void *stream)
{
    if (B < 0 || N1 < 0 || N2 < 0)
        return TK3D_ERR_BAD_SIZE;
    if (N1 > TK_MAX_I32 / 4 || N2 > TK_MAX_I32 / 4 || !tk_fits(TK_MAX_ELEMS, B, N1, 3) ||
        !tk_fits(TK_MAX_ELEMS, B, N2, 3))
        return TK3D_ERR_UNSUPPORTED;
    if (B * N1 > 0 && (!xyz1 || !dist1 || !idx1))
        return TK3D_ERR_NULL_POINTER;
    if (B * N2 > 0 && (!xyz2 || !dist2 || !idx2))
        return TK3D_ERR_NULL_POINTER;
    hipStream_t s = (hipStream_t)stream;
    // Fewer queries per lane when the clouds are small, so the launch still
    // spreads over the chip.
    const int64_t work = B * (N1 > N2 ? N1 : N2);
    if constexpr (sizeof(T) == 4) {
        // The pre-filter pays off once the key clouds are a few hundred points long
        // (its prologue passes over the keys twice per workgroup).
        const int64_t nkmin = N1 < N2 ? N1 : N2;
        // Matrix-core pre-filter, 512 queries per workgroup: the fastest sweep from about a
        // hundred workgroups on key clouds of 1024 points or more (1.3-2.2x over the
        // vector pre-filter). A workgroup sweeps its direction's whole key cloud unless
        // that leaves fewer than 256 workgroups or - clouds of very different lengths -
        // a few workgroups with most of the work: a direction's key cloud is then cut
        // into slices no longer than 1/256 of all the sweeping (and no shorter than 1024
        // keys), each direction on its own (B=1, 200000 x 2048: 1.99 -> 0.07 ms).
        if (nkmin >= 1 && (N1 > N2 ? N1 : N2) >= 1024) {
            const int64_t qb[2] = {B * ((N1 + 511) / 512), B * ((N2 + 511) / 512)};
            const int64_t nk[2] = {N2, N1};
            const double sweep = (double)qb[0] * (double)nk[0] + (double)qb[1] * (double)nk[1];
            double longest = sweep / 256.0;
            longest = longest < 1024.0 ? 1024.0 : longest;
            int want[2];
            double len[2];
            for (int w = 0; w < 2; ++w) {
                const double parts = (double)nk[w] / longest;
                want[w] = parts <= 1.0 ? 1 : parts >= 256.0 ? 256 : (int)(parts + 0.999);
                len[w] = (double)nk[w] / want[w];
            }
            // ... and no workgroup sweeps more than twice what the other direction's do
            // (the long ones would run on alone at the end)
            const double shorter = len[0] < len[1] ? len[0] : len[1];
            const double cap = 2.0 * shorter < 1024.0 ? 1024.0 : 2.0 * shorter;
            int64_t blocks = 0;
            for (int w = 0; w < 2; ++w) {
                if (len[w] > cap) {
                    const double parts = (double)nk[w] / cap;
                    want[w] = parts >= 256.0 ? 256 : (int)(parts + 0.999);
                }
                int64_t slice_len;
                blocks += qb[w] * chamfer_slices(nk[w], want[w], 128, slice_len);
            }
            // Launches of up to one and a half workgroups per CU (two and a half on key
            // clouds of up to 4096 points) run with two query blocks per wave instead of
            // four: twice the workgroups of half the queries, so the chip holds them all at
            // once with work for every SIMD (B=16, 4096 x 4096: 43 -> 37 us; B=24,
            // 2048 x 2048: 42 -> 32 us; B=48, 2500 x 3001: 107 -> 84 us). Larger launches
            // lose to the key terms every workgroup stages for itself (B=32, 16384 x 16384:
            // 0.59 -> 0.64 ms).
            const int64_t nkmax = N1 > N2 ? N1 : N2;
            // ([3,N] clouds: the vector pre-filter below reads [N,3] only, so the matrix
            // pre-filter also takes the launches of under 96 workgroups)
            if ((SOA || blocks >= 96) && (blocks <= 384 || (blocks <= 640 && nkmax <= 4096)))
                return chamfer_forward_mfma_launch<2, SOA>(xyz1, xyz2, B, N1, N2, dist1, idx1,
                                                           dist2, idx2, s, want[0], want[1]);
            if (blocks >= 96)
                return chamfer_forward_mfma_launch<4, SOA>(xyz1, xyz2, B, N1, N2, dist1, idx1,
                                                           dist2, idx2, s, want[0], want[1]);
        }
        if (!SOA && nkmin >= 512) {
            // Launch shapes: 4 queries per lane in 512-lane workgroups is the fastest
            // sweep once it fills the chip; below that 2 queries per lane in 256-lane
            // workgroups, with the key cloud cut into slices when even those are too few.
            double best = chamfer_sweep_cost(B, N1, N2, 4, 512, 3.76, 500.0, 1);
            int best_slices = 0;  // 0: the 4 x 512 shape
            for (int slices = 1; slices <= 16; slices *= 2) {
                const double c = chamfer_sweep_cost(B, N1, N2, 2, 256, 4.5, 250.0, slices);
                if (c < best) {
                    best = c;
                    best_slices = slices;
                }
            }
            if (best_slices == 0)
                return chamfer_forward_filter_launch<4, 512, 64, 512>(
                    xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, s);
            return chamfer_forward_filter_launch<2, 256, 64, 512>(
                xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, s, best_slices);
        }
    }
    if (sizeof(T) == 8 || work < (int64_t)256 * 1024)
        return chamfer_forward_launch<T, 2, 256, 32, 1024, SOA>(xyz1, xyz2, B, N1, N2, dist1, idx1,
                                                                dist2, idx2, s);
    return chamfer_forward_launch<T, 4, 512, 64, 1024, SOA>(xyz1, xyz2, B, N1, N2, dist1, idx1,
                                                            dist2, idx2, s);
}

// ---- fp32 forward on clouds sorted along a space-filling curve ---------------------
//
// The sweeps above evaluate every (query, key) pair. Points that are far apart cannot be
// nearest neighbours, and once both clouds are ordered along a space-filling curve that
// can be decided for 32 keys and a wave's queries at a time:
//
//   chamfer_cell_kernel (four workgroups per cloud): the cloud's frame - its bounding box,
//     trimmed so that a few points far from the rest do not decide it - with centre and
//     power-of-two scale as in the matrix pre-filter, and every point's cell in a 32^3
//     grid over the frame, numbered along the Hilbert curve.
//   chamfer_sort_kernel (one workgroup per cloud): counting sort of the points by cell.
//     The sorted points carry their original index.
//   chamfer_tile_kernel (one lane per point): per tile of 32 sorted points the 16 fp16
//     terms of every key (the layout the matrix kernel stages in LDS) and the tile's
//     bounding box in centred, scaled coordinates; keys far outside the frame go on a
//     short list instead.
//   chamfer_pruned_kernel (waves work alone, no LDS): a wave takes NQB x 32 consecutive
//     sorted queries - a compact patch - and sweeps a key tile only if the squared gap
//     between the patch's box and the tile's box does not exceed T, an upper bound of
//     every query's distance to the nearest key met so far: first the tiles that overlap
//     the patch, then (if those were few) the tiles within T/4, then those within T,
//     with T taken anew each time. The
//     sweep, the three smallest tile minima per lane and the exact re-evaluation of the
//     candidate tiles are those of the matrix kernel; ties between equal distances go to
//     the lower original index, compared explicitly because sorted order is not index
//     order. Queries with three or more candidate tiles are scanned exactly over the
//     swept tiles only.
//
// Why a skipped tile cannot matter. With the notation of the matrix kernel (k', q' the
// centred, scaled points as rounded, u = 2^-24, R = (max|k'| + |q'|)^2): the score of a
// swept key satisfies |s + |q'|^2 - d2| <= 52.3 u R for its canonical distance d2 (in
// scaled units), so ub = min s + |q'|^2 + 128 u R (the sum in fp32: 4 u R more) is at
// least the canonical distance of some swept key. For a key of a skipped tile,
// d2 >= |q' - k'|^2 - 7.1 u R >= gap^2 - 7.1 u R, where gap^2, evaluated in fp32 from box
// corners that are themselves coordinates of rounded points, is within a factor 1 - 8u of
// the exact squared gap. A tile is skipped only if gap^2 > (T + 128 u R) * 1.001 with
// T >= ub of every query of the wave, so each of its keys is strictly farther from every
// query than a key already met: it can neither be the minimum nor tie with it. T only
// shrinks as tiles are swept, so a tile skipped under an earlier T stays skipped rightly.
//
// Input the bound does not cover (non-finite coordinates, extents outside 2^+-40, a query
// cloud whose frame reaches further than 8000 extents from the key cloud or holds many
// stray queries that far out), a key cloud under a quarter of the query
// cloud's extent (boxes cannot prune for queries far from all keys) and waves whose exact
// scans would take long (heavy ties on many swept tiles) raise a flag for their cloud and
// direction; the matrix pre-filter runs behind this one and serves exactly the flagged
// ones.
constexpr int CHAMFER_FAR_KEYS = 64;  // keys far outside the frame that a cloud may have

struct ChamferSortedHdr {  // 64 bytes per cloud and batch element
    float c[3];            // centre of the frame (the trimmed bounding box)
    float scale;           // 2^-(exponent of the frame's largest half extent)
    int kmax2_bits;        // largest |k'|^2 of the keys inside 4 units (bit pattern)
    int unsafe;            // the bound does not cover this cloud
    float lo[3], hi[3];    // bounding box of all points, caller's units
    float extent;          // largest extent of the frame, caller's units
    int far_keys;          // keys beyond 4 units of the frame, kept on a list of their own
    int occupied;          // cells of the 32^3 grid that hold a point
    int pad;
};

struct ChamferSortArgs {
    const float *xyz[2];
    float4 *sorted[2];  // [B, npad]: x, y, z, original index (bits); padding: NaN, -1
    uint4 *terms[2];    // [B, npad / 32][2][32]
    uint4 *boxes[2];    // [B, npad / 32]: lo and hi corner in centred, scaled coordinates,
                        // six fp16 values rounded outwards
    float4 *far_keys[2];  // [B, CHAMFER_FAR_KEYS]: x, y, z, original index
    ChamferSortedHdr *hdr;  // [2, B]
    int *flags;             // [2, B], then one word that is set when any of them is
    int n[2], npad[2];
    int B;
    int three_launches[2];  // this cloud is prepared by the cell, sort and tile kernels
                            // (beyond 16384 points); else by chamfer_prepare_kernel
    int channels_first;     // the clouds are [B,3,N] (chamfer_prepare_kernel only)
};

__host__ __device__ constexpr int chamfer_morton5(int v)
{
    v &= 0x1f;
    v = (v | (v << 8)) & 0x100f;
    v = (v | (v << 4)) & 0x10c3;
    v = (v | (v << 2)) & 0x1249;
    return v;
}

// Position of cell (x, y, z), each below 32, along the 3-D Hilbert curve of order 5
// (Skilling's transposed form, then the bits interleaved): consecutive positions are
// neighbouring cells, so a run of consecutive sorted points is a compact patch, which a
// run along the Morton curve, with its jumps, often is not.
__host__ __device__ constexpr int chamfer_hilbert15(unsigned x, unsigned y, unsigned z)
{
    unsigned X[3] = {x, y, z};
#pragma unroll
    for (unsigned Q = 16; Q > 1; Q >>= 1) {
        const unsigned P = Q - 1;
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const bool set = (X[i] & Q) != 0;
            const unsigned t = (X[0] ^ X[i]) & P;
            X[0] ^= set ? P : t;
            if (i != 0)
                X[i] ^= set ? 0u : t;
        }
    }
    X[1] ^= X[0];
    X[2] ^= X[1];
    unsigned t = 0;
#pragma unroll
    for (unsigned Q = 16; Q > 1; Q >>= 1)
        t ^= (X[2] & Q) ? Q - 1 : 0u;
    X[0] ^= t;
    X[1] ^= t;
    X[2] ^= t;
    return (chamfer_morton5((int)X[0]) << 2) | (chamfer_morton5((int)X[1]) << 1) |
           chamfer_morton5((int)X[2]);
}

// A pilot centre that a few stray points cannot move: per axis the median of three medians
// of three, over nine points spread through the cloud; and `cap`, 16 times the typical
// deviation of the nine from it (none, i.e. the nine coincide: no cap).
__device__ __forceinline__ void chamfer_pilot(const float *__restrict__ P, int n, float (&pilot)[3],
                                              float (&cap)[3], bool channels_first = false)
{
    const float INF = __builtin_huge_valf();
    TkPoint3<float> q[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) {
        const int j = (int)(((int64_t)n * (2 * i + 1)) / 19);
        q[i] = channels_first ? chamfer_point<true, float>(P, n, j)
                              : chamfer_point<false, float>(P, n, j);
    }
    auto ninther = [](float v0, float v1, float v2, float v3, float v4, float v5, float v6,
                      float v7, float v8) {
        return __builtin_amdgcn_fmed3f(__builtin_amdgcn_fmed3f(v0, v1, v2),
                                       __builtin_amdgcn_fmed3f(v3, v4, v5),
                                       __builtin_amdgcn_fmed3f(v6, v7, v8));
    };
    pilot[0] = ninther(q[0].x, q[1].x, q[2].x, q[3].x, q[4].x, q[5].x, q[6].x, q[7].x, q[8].x);
    pilot[1] = ninther(q[0].y, q[1].y, q[2].y, q[3].y, q[4].y, q[5].y, q[6].y, q[7].y, q[8].y);
    pilot[2] = ninther(q[0].z, q[1].z, q[2].z, q[3].z, q[4].z, q[5].z, q[6].z, q[7].z, q[8].z);
    float d[9][3];
#pragma unroll
    for (int i = 0; i < 9; ++i) {
        d[i][0] = __builtin_fabsf(q[i].x - pilot[0]);
        d[i][1] = __builtin_fabsf(q[i].y - pilot[1]);
        d[i][2] = __builtin_fabsf(q[i].z - pilot[2]);
    }
#pragma unroll
    for (int ax = 0; ax < 3; ++ax) {
        const float typical = ninther(d[0][ax], d[1][ax], d[2][ax], d[3][ax], d[4][ax],
                                      d[5][ax], d[6][ax], d[7][ax], d[8][ax]);
        cap[ax] = typical > 0.0f ? 16.0f * typical : INF;
    }
}

// The frame of a cloud from the waves' partial results (sred: lo and hi per axis, sdev: sums
// of capped deviations): the bounding box, trimmed to three mean deviations around the pilot
// centre. A uniform or a Gaussian cloud keeps (nearly) its bounding box - three mean
// deviations are 1.5 half extents of the first and 2.4 sigma of the second, and keys up to
// twice as far out as the frame are still swept like any other; a few points far away no
// longer decide the cells and the scale of everything else - they go on a list of their own.
// Returns the bounding box (lo, hi), the frame's centre cc, lower corner flo and largest half
// extent ext.
template <int NW>
__device__ __forceinline__ void chamfer_frame(const float (*sred)[8], const float (*sdev)[4],
                                              const float (&pilot)[3], int n, float (&lo)[3],
                                              float (&hi)[3], float (&cc)[3], float (&flo)[3],
                                              float &ext)
{
    ext = 0.0f;
#pragma unroll
    for (int ax = 0; ax < 3; ++ax) {
        float l = sred[0][ax], h = sred[0][3 + ax], dsum = sdev[0][ax];
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            l = __builtin_fminf(l, sred[w][ax]);
            h = __builtin_fmaxf(h, sred[w][3 + ax]);
            dsum += sdev[w][ax];
        }
        lo[ax] = l;
        hi[ax] = h;
        const float reach = 3.0f * (dsum / (float)n);
        const float fl = __builtin_fmaxf(l, pilot[ax] - reach);
        const float fh = __builtin_fminf(h, pilot[ax] + reach);
        flo[ax] = fl;
        cc[ax] = 0.5f * fl + 0.5f * fh;
        ext = __builtin_fmaxf(ext, 0.5f * fh - 0.5f * fl);
    }
    if (ext == 0.0f) {
        // Nearly all points in one place: a frame of no extent would leave the others at
        // scale 1, possibly far below it, where the fp16 terms have no precision left
        // (the error bound counts on max|k'| of order 1). The bounding box, then.
#pragma unroll
        for (int ax = 0; ax < 3; ++ax) {
            flo[ax] = lo[ax];
            cc[ax] = 0.5f * lo[ax] + 0.5f * hi[ax];
            ext = __builtin_fmaxf(ext, 0.5f * hi[ax] - 0.5f * lo[ax]);
        }
    }
}

// A tile's box as six fp16 corners, moved outwards by more than the rounding to nearest can
// bring them back (2^-11 relative, 2^-25 in the subnormal range); an empty box stays
// (+inf, -inf).
__device__ __forceinline__ uint4 chamfer_box_bits(const float (&bl)[3], const float (&bh)[3])
{
    unsigned h[6];
#pragma unroll
    for (int ax = 0; ax < 3; ++ax) {
        const float wl = __builtin_fabsf(bl[ax]) * 9.765625e-4f + 1.1920929e-7f;
        const float wh = __builtin_fabsf(bh[ax]) * 9.765625e-4f + 1.1920929e-7f;
        h[ax] = bl[ax] > 3.0e38f ? 0x7c00u : tk_f16_bits(bl[ax] - wl);
        h[3 + ax] = bh[ax] < -3.0e38f ? 0xfc00u : tk_f16_bits(bh[ax] + wh);
    }
    return make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), 0u);
}

constexpr int CHAMFER_SORT_CELLS = 32768;

// Bounding box of a cloud and the cell of every point. CHAMFER_CELL_PARTS workgroups per
// cloud: each finds the bounding box of the whole cloud for itself (a pass over memory)
// and then computes the cells of its share of the points (the arithmetic of the launch),
// kept where the key terms will go. Points are loaded U at a time per lane so that a pass
// over the cloud is a few round trips to memory.
constexpr int CHAMFER_CELL_PARTS = 4;

__global__ __launch_bounds__(1024) void chamfer_cell_kernel(ChamferSortArgs a)
{
    constexpr int NT = 1024, NW = NT / TK_WAVE, U = 16, PARTS = CHAMFER_CELL_PARTS;
    __shared__ float sred[NW][8];
    __shared__ float sdev[NW][4];
    __shared__ int sbad;
    const int tid = threadIdx.x, lane = tid & (TK_WAVE - 1), wave = tid / TK_WAVE;
    const int cloud = (int)blockIdx.x / PARTS, part = (int)blockIdx.x - cloud * PARTS;
    const int which = cloud >= a.B;
    if (!a.three_launches[which])  // uniform over the workgroup
        return;
    const int b = cloud - which * a.B;
    const int n = a.n[which], npad = a.npad[which];
    const float *__restrict__ P = a.xyz[which] + (int64_t)b * n * 3;
    unsigned short *__restrict__ cells =
        reinterpret_cast<unsigned short *>(a.terms[which] + (int64_t)b * npad * 2);
    ChamferSortedHdr *hdr = a.hdr + which * a.B + b;
    const float INF = __builtin_huge_valf();

    // A pilot centre that a few stray points cannot move: per axis the median of three
    // medians of three, over nine points spread through the cloud.
    float pilot[3] = {0.0f, 0.0f, 0.0f};
    float cap[3] = {INF, INF, INF};  // a deviation counts up to 16 typical ones
    float lo[3] = {INF, INF, INF}, hi[3] = {-INF, -INF, -INF};
    float dev[3] = {0.0f, 0.0f, 0.0f};  // sum of |x - pilot|
    bool bad = false;
    for (int base = 0; base < n; base += NT * U) {
        TkPoint3<float> p[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = base + u * NT + tid;
            p[u] = tk_load3<float>(P + (int64_t)(j < n ? j : n - 1) * 3);
        }
        if (base == 0)  // (requested together with the first points: one round trip)
            chamfer_pilot(P, n, pilot, cap);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float v[3] = {p[u].x, p[u].y, p[u].z};
            const bool counts = base + u * NT + tid < n;
#pragma unroll
            for (int ax = 0; ax < 3; ++ax) {
                bad |= !(v[ax] - v[ax] == 0.0f);
                lo[ax] = __builtin_fminf(lo[ax], counts ? v[ax] : INF);
                hi[ax] = __builtin_fmaxf(hi[ax], counts ? v[ax] : -INF);
                dev[ax] += counts ? __builtin_fminf(__builtin_fabsf(v[ax] - pilot[ax]), cap[ax]) : 0.0f;
            }
        }
    }
#pragma unroll
    for (int ax = 0; ax < 3; ++ax) {
        lo[ax] = wave_reduce_min(lo[ax]);
        hi[ax] = wave_reduce_max(hi[ax]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
            dev[ax] += __shfl_xor(dev[ax], o);
    }
    if (tid == 0)
        sbad = 0;
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int ax = 0; ax < 3; ++ax) {
            sred[wave][ax] = lo[ax];
            sred[wave][3 + ax] = hi[ax];
            sdev[wave][ax] = dev[ax];
        }
    }
    if (bad)
        sbad = 1;
    __syncthreads();
    float cc[3], ext, flo[3];
    chamfer_frame<NW>(sred, sdev, pilot, n, lo, hi, cc, flo, ext);
    const float c0 = cc[0], c1 = cc[1], c2 = cc[2];
    const int ebits = (int)((__builtin_bit_cast(unsigned, ext) >> 23) & 0xffu) - 127;
    const bool safe = n > 0 && sbad == 0 && (c0 - c0 == 0.0f) && (c1 - c1 == 0.0f) &&
                      (c2 - c2 == 0.0f) && (ext - ext == 0.0f) &&
                      (ext == 0.0f || (ebits >= -40 && ebits <= 40));
    if (tid == 0 && part == 0) {
        a.flags[which * a.B + b] = 0;
        if (cloud == 0)
            a.flags[2 * a.B] = 0;
        hdr->c[0] = c0;
        hdr->c[1] = c1;
        hdr->c[2] = c2;
        hdr->scale =
            ext == 0.0f ? 1.0f : __builtin_bit_cast(float, (unsigned)(127 - ebits) << 23);
        hdr->kmax2_bits = 0;
        hdr->unsafe = safe ? 0 : 1;
        hdr->extent = 2.0f * ext;
        hdr->far_keys = 0;
        hdr->occupied = 0x7fffffff;  // (not counted on this route: never "crowded")
#pragma unroll
        for (int ax = 0; ax < 3; ++ax) {
            hdr->lo[ax] = lo[ax];
            hdr->hi[ax] = hi[ax];
        }
    }
    if (!safe)  // uniform over the workgroup
        return;
    // cells: 32 per axis over the frame's largest extent (a point on the upper face, or
    // beyond the frame: the outermost cell)
    const float inv = ext > 0.0f ? (16.0f / ext) * 0.99999f : 0.0f;
    const int share = (n + PARTS - 1) / PARTS;
    const int first = part * share, last = first + share < n ? first + share : n;
    for (int j = first + tid; j < last; j += NT) {
        const TkPoint3<float> p = tk_load3<float>(P + (int64_t)j * 3);
        const float ux = __builtin_fminf(__builtin_fmaxf((p.x - flo[0]) * inv, 0.0f), 31.0f);
        const float uy = __builtin_fminf(__builtin_fmaxf((p.y - flo[1]) * inv, 0.0f), 31.0f);
        const float uz = __builtin_fminf(__builtin_fmaxf((p.z - flo[2]) * inv, 0.0f), 31.0f);
        const int ix = (int)ux, iy = (int)uy, iz = (int)uz;
        cells[j] = (unsigned short)chamfer_hilbert15((unsigned)ix, (unsigned)iy, (unsigned)iz);
    }
}

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ int wave_inclusive_sum(int v)
{
    // within rows of 16 lanes, then row 0 -> 1, 2 -> 3 and rows 0..1 -> 2..3
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31
    return v;
}

// One workgroup per cloud: counting sort of the points by cell.
__global__ __launch_bounds__(1024) void chamfer_sort_kernel(ChamferSortArgs a)
{
    constexpr int NT = 1024, NW = NT / TK_WAVE, CELLS = CHAMFER_SORT_CELLS, U = 16;
    extern __shared__ int hist[];  // CELLS counters
    __shared__ int swave[NW];
    __shared__ int sstart[NW];
    const int tid = threadIdx.x, lane = tid & (TK_WAVE - 1), wave = tid / TK_WAVE;
    const int which = (int)blockIdx.x >= a.B;
    const int b = (int)blockIdx.x - which * a.B;
    const int n = a.n[which], npad = a.npad[which];
    if (!a.three_launches[which] || a.hdr[which * a.B + b].unsafe != 0)  // uniform
        return;
    const float *__restrict__ P = a.xyz[which] + (int64_t)b * n * 3;
    float4 *__restrict__ sorted = a.sorted[which] + (int64_t)b * npad;
    const unsigned short *__restrict__ cells =
        reinterpret_cast<const unsigned short *>(a.terms[which] + (int64_t)b * npad * 2);
    for (int i = tid; i < CELLS; i += NT)
        hist[i] = 0;
    __syncthreads();
    for (int base = 0; base < n; base += NT * U) {
        int cell[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = base + u * NT + tid;
            cell[u] = cells[j < n ? j : n - 1];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (base + u * NT + tid < n)
                atomicAdd(&hist[cell[u]], 1);
        }
    }
    __syncthreads();
    // Every wave turns its 2048 counters into starting positions within its range, 64
    // at a time; the ranges' own starts are added when a position is taken.
    {
        constexpr int PER_WAVE = CELLS / NW;
        int carry = 0;
        for (int i = 0; i < PER_WAVE; i += TK_WAVE) {
            const int at = wave * PER_WAVE + i + lane;
            const int count = hist[at];
            const int incl = wave_inclusive_sum(count);
            hist[at] = carry + incl - count;
            carry += __builtin_amdgcn_readlane(incl, TK_WAVE - 1);
        }
        if (lane == 0)
            swave[wave] = carry;
    }
    __syncthreads();
    if (tid < NW) {  // the ranges' own starts, looked up by cell >> 11 below
        int run = 0;
        for (int w = 0; w < tid; ++w)
            run += swave[w];
        sstart[tid] = run;
    }
    __syncthreads();
    for (int base = 0; base < n; base += NT * U) {
        TkPoint3<float> p[U];
        int cell[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = base + u * NT + tid;
            const int jj = j < n ? j : n - 1;
            p[u] = tk_load3<float>(P + (int64_t)jj * 3);
            cell[u] = cells[jj];
        }
        int pos[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = base + u * NT + tid;
            pos[u] = j < n ? atomicAdd(&hist[cell[u]], 1) : 0;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = base + u * NT + tid;
            const int start = sstart[cell[u] >> 11];
            if (j < n)
                sorted[pos[u] + start] =
                    make_float4(p[u].x, p[u].y, p[u].z, __builtin_bit_cast(float, j));
        }
    }
}

// Key terms and bounding boxes of the sorted tiles, one lane per point; the padding up to
// a whole number of 128 points is written here too.
__global__ __launch_bounds__(256) void chamfer_tile_kernel(ChamferSortArgs a, int blocks0)
{
    const int tid = threadIdx.x;
    const int which = (int)blockIdx.x >= blocks0;
    const int lb = (int)blockIdx.x - which * blocks0;
    const int n = a.n[which], npad = a.npad[which];
    // (npad is a multiple of 128: a cloud's last block may be half empty)
    const int bpc = (npad + 255) / 256;
    const int b = lb / bpc;
    const int i = (lb - b * bpc) * 256 + tid;
    ChamferSortedHdr *hdr = a.hdr + which * a.B + b;
    if (!a.three_launches[which])
        return;
    if (hdr->unsafe != 0 || i >= npad)  // (uniform over each half wave: npad % 32 == 0)
        return;
    float4 *__restrict__ sorted = a.sorted[which] + (int64_t)b * npad;
    uint4 *__restrict__ terms = a.terms[which] + (int64_t)b * npad * 2;
    uint4 *__restrict__ boxes = a.boxes[which] + (int64_t)b * (npad / 32);
    const float INF = __builtin_huge_valf();
    const float c0 = hdr->c[0], c1 = hdr->c[1], c2 = hdr->c[2], scale = hdr->scale;
    const bool exists = i < n;
    const float qnan = __builtin_nanf("");
    float4 s = make_float4(qnan, qnan, qnan, __builtin_bit_cast(float, -1));
    if (exists)
        s = sorted[i];
    else
        sorted[i] = s;
    const float x = ((exists ? s.x : c0) - c0) * scale;
    const float y = ((exists ? s.y : c1) - c1) * scale;
    const float z = ((exists ? s.z : c2) - c2) * scale;
    const float nn = __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x));
    // A key beyond 4 units of the frame (the frame itself reaches 3.5) would widen the
    // error bound of every pair through max|k'|: the sweep sees it as padding, and every
    // wave compares its queries with the few such keys directly.
    const bool far = exists && !(nn <= 16.0f);
    if (far) {
        const int slot = atomicAdd(&hdr->far_keys, 1);
        if (slot < CHAMFER_FAR_KEYS)
            a.far_keys[which][(int64_t)b * CHAMFER_FAR_KEYS + slot] = s;
    }
    const bool swept = exists && !far;
    uint4 h0, h1;
    chamfer_key_terms(x, y, z, nn, swept, h0, h1);
    uint4 *tile = terms + (i >> 5) * 64 + (i & 31);
    tile[0] = h0;
    tile[32] = h1;
    float bl[3] = {swept ? x : INF, swept ? y : INF, swept ? z : INF};
    float bh[3] = {swept ? x : -INF, swept ? y : -INF, swept ? z : -INF};
    float kmax2 = swept ? nn : 0.0f;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
#pragma unroll
        for (int ax = 0; ax < 3; ++ax) {
            bl[ax] = __builtin_fminf(bl[ax], __shfl_xor(bl[ax], o));
            bh[ax] = __builtin_fmaxf(bh[ax], __shfl_xor(bh[ax], o));
        }
        kmax2 = __builtin_fmaxf(kmax2, __shfl_xor(kmax2, o));
    }
    if ((i & 31) == 0) {
        boxes[i >> 5] = chamfer_box_bits(bl, bh);
        // non-negative floats order as their bit patterns
        atomicMax(&hdr->kmax2_bits, __builtin_bit_cast(int, kmax2));
    }
}

// The Hilbert position of every cell of the 32^3 grid, worked out when the library is
// compiled: the kernel below copies the 64 KiB table into LDS and looks a cell up there
// instead of spending 135 instructions on it.
struct ChamferHilbertTable {
    unsigned short at[CHAMFER_SORT_CELLS];
};
constexpr ChamferHilbertTable chamfer_make_hilbert_table()
{
    ChamferHilbertTable t = {};
    for (unsigned x = 0; x < 32; ++x)
        for (unsigned y = 0; y < 32; ++y)
            for (unsigned z = 0; z < 32; ++z)
                t.at[(x << 10) | (y << 5) | z] = (unsigned short)chamfer_hilbert15(x, y, z);
    return t;
}
__device__ const ChamferHilbertTable chamfer_hilbert_table = chamfer_make_hilbert_table();

// Floats as signed integers that order the same way (an involution; -0 sorts below +0).
__device__ __forceinline__ int tk_float_order(float x)
{
    const int i = __builtin_bit_cast(int, x);
    return i ^ ((i >> 31) & 0x7fffffff);
}
__device__ __forceinline__ float tk_order_float(int i)
{
    return __builtin_bit_cast(float, i ^ ((i >> 31) & 0x7fffffff));
}

// Minimum (MAX: maximum) over each half of the wave, left in lanes 31 and 63: a scan along
// rows of 16 lanes with row shifts, then row 0's result carried into row 1 (2's into 3).
// On integers: a floating-point minimum quiets its operands first, one more instruction per
// step and operand (57 of the 271 instructions a sorted point cost went there).
template <bool MAX> __device__ __forceinline__ int half_wave_reduce_to_last(int v)
{
#define TK_HALF_WAVE_STEP(ctrl, rows)                                                  \
    {                                                                                  \
        const int o = __builtin_amdgcn_update_dpp(v, v, ctrl, rows, 0xf, false);       \
        v = MAX ? (o > v ? o : v) : (o < v ? o : v);                                   \
    }
    TK_HALF_WAVE_STEP(0x111, 0xf)  // row_shr:1
    TK_HALF_WAVE_STEP(0x112, 0xf)  // row_shr:2
    TK_HALF_WAVE_STEP(0x114, 0xf)  // row_shr:4
    TK_HALF_WAVE_STEP(0x118, 0xf)  // row_shr:8
    TK_HALF_WAVE_STEP(0x142, 0xa)  // row_bcast:15 into rows 1 and 3
#undef TK_HALF_WAVE_STEP
    return v;
}

// Everything the pruned sweep needs of one cloud of up to 16384 points, in one launch.
// `parts` workgroups of 1024 lanes (16 points per lane) serve a cloud. Each works out, for
// itself, what needs the whole cloud:
//   the frame (bounding box, trimmed as in chamfer_cell_kernel), the largest swept |k'|^2 and
//     the list of keys far outside the frame,
//   the cells (a table look-up), their histogram in LDS (two 16-bit counters per word:
//     64 KiB; the atomic that counts a point also hands it its rank within the cell) and the
//     prefix sums, hence every point's position in sorted order.
// The write-out is divided by cells: the sixteen ranges of 2048 cells are dealt to the parts
// in runs of about equal numbers of points, and a part writes the sorted positions of its own
// cells (the rank within a cell is whatever order the part's own atomics arrived in, so two
// parts must not share a cell). It takes its positions in windows of PREP_WINDOW - the lanes
// drop the points that belong to the window into LDS, and the workgroup then walks the window
// in sorted order, a lane per point, storing the sorted point, its 16 fp16 terms and, per 32
// points, the tile's box, all as runs of consecutive addresses. (Storing each point at its
// sorted position straight from the lane that holds it is one cache line per lane and store:
// it took 16 of the 23 us of the counting sort that three separate launches used to run.)
// A tile of 32 positions that two parts share gets its box from the part that owns its first
// position: exact for that part's points, and for the rest the box of every point of the
// later cells that begin inside the tile - a superset of the tile's points, which is all a
// box has to be. What every part repeats is about a third of the work of a cloud, and no
// workgroup waits for another.
constexpr int PREP_MAX_POINTS = 16384;
constexpr int PREP_WINDOW = 5600;  // 175 tiles; three windows cover 16384 points
constexpr size_t PREP_LDS_BYTES = (size_t)(CHAMFER_SORT_CELLS / 2) * sizeof(unsigned) +
                                  (size_t)(PREP_WINDOW + TK_WAVE) * sizeof(float4);

__global__ __launch_bounds__(1024) void chamfer_prepare_kernel(ChamferSortArgs a, int first_cloud,
                                                               int parts)
{
    constexpr int NT = 1024, NW = NT / TK_WAVE, U = PREP_MAX_POINTS / NT, W = PREP_WINDOW;
    constexpr int WORDS = CHAMFER_SORT_CELLS / 2;
    constexpr int ORDER_POS_INF = 0x7f800000, ORDER_NEG_INF = (int)0x807fffffu;
    extern __shared__ __align__(16) unsigned prep_lds[];
    unsigned *const hist = prep_lds;                                  // WORDS packed counters
    float4 *const win = reinterpret_cast<float4 *>(prep_lds + WORDS);  // W sorted points, then
                                                                       // a spare slot per lane
    __shared__ float sred[NW][8];
    __shared__ float sdev[NW][4];
    __shared__ int swave[NW];
    __shared__ int sstart[NW + 1];
    __shared__ float4 sfar_list[CHAMFER_FAR_KEYS];
    __shared__ int sbad, sfar;
    __shared__ int sextra[8];  // box of the later parts' points in this part's last tile
    const int tid = threadIdx.x, lane = tid & (TK_WAVE - 1), wave = tid / TK_WAVE;
    // (the parts of a cloud on one XCD, whose L2 then fetches the cloud once: consecutive
    // workgroup ids go to the eight XCDs in turn)
    int unit = (int)blockIdx.x;
    if ((int)gridDim.x % (8 * parts) == 0)
        unit = (unit & 7) * ((int)gridDim.x >> 3) + (unit >> 3);
    const int cloud = first_cloud + unit / parts;
    const int part = unit % parts;
    const int which = cloud >= a.B;
    const int b = cloud - which * a.B;
    const int n = a.n[which], npad = a.npad[which];
    const float *__restrict__ P = a.xyz[which] + (int64_t)b * n * 3;
    ChamferSortedHdr *hdr = a.hdr + which * a.B + b;
    const float INF = __builtin_huge_valf();

    // The lane's 16 points, all loads in flight together. Each pass below asks for them anew
    // (after the first they come from the L2) rather than holding 48 registers across the
    // kernel, and through a buffer descriptor: one 32-bit offset per point against a base in
    // scalar registers (a lane past the end of the cloud reads the last point again). With
    // sixteen 64-bit addresses, the same in every pass, the compiler kept the addresses alive
    // across the kernel and spilled them, and a spilled address is a round trip to memory in
    // front of its load.
    const __amdgpu_buffer_rsrc_t cloud_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P), 0, n * 12, 0x00020000);
    auto load_points = [&](TkPoint3<float>(&p)[U]) {
        // (the lane number is made opaque per pass, or the compiler merges the passes' loads
        // into one set of 48 registers that lives across the kernel)
        int t = tid;
        asm volatile("" : "+v"(t));
        if (a.channels_first) {  // (uniform) a [3,N] cloud: one load per coordinate
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = u * NT + t;
                const int at = (j < n ? j : n - 1) * 4;
                p[u].x = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(cloud_rsrc, at, 0, 0));
                p[u].y = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(cloud_rsrc, at, n * 4, 0));
                p[u].z = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(cloud_rsrc, at, n * 8, 0));
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            typedef float f3 __attribute__((ext_vector_type(3)));
            const int j = u * NT + t;
            const f3 v = __builtin_bit_cast(
                f3, __builtin_amdgcn_raw_buffer_load_b96(cloud_rsrc, (j < n ? j : n - 1) * 12, 0, 0));
            p[u].x = v.x;
            p[u].y = v.y;
            p[u].z = v.z;
        }
    };

    // ---- the pilot centre, the bounding box and the deviations ----
    float pilot[3], cap[3];
    chamfer_pilot(P, n, pilot, cap, a.channels_first != 0);
    for (int i = tid; i < WORDS / 4; i += NT)
        reinterpret_cast<uint4 *>(hist)[i] = make_uint4(0u, 0u, 0u, 0u);
    if (tid < 8)
        sextra[tid] = tid < 3 ? ORDER_POS_INF : ORDER_NEG_INF;
    __builtin_amdgcn_sched_barrier(0);  // (the pilot's nine points and the lane's sixteen at
                                        // once do not fit the registers)
    float lo[3] = {INF, INF, INF}, hi[3] = {-INF, -INF, -INF};
    float dev[3] = {0.0f, 0.0f, 0.0f};
    bool bad = false;
    // (the table of Hilbert positions comes along, into the LDS that the windows use later:
    // looked up in global memory, one cache line per lane, the look-ups took 8 us)
    unsigned short *const cell_of = reinterpret_cast<unsigned short *>(win);
    static_assert(sizeof(ChamferHilbertTable) <= (size_t)PREP_WINDOW * sizeof(float4), "table fits");
    {
        TkPoint3<float> p[U];
        load_points(p);
        constexpr int QUADS = (int)(sizeof(ChamferHilbertTable) / sizeof(uint4)) / NT;
        uint4 table[QUADS];
#pragma unroll
        for (int k = 0; k < QUADS; ++k)
            table[k] = reinterpret_cast<const uint4 *>(chamfer_hilbert_table.at)[k * NT + tid];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float v[3] = {p[u].x, p[u].y, p[u].z};
            const bool counts = u * NT + tid < n;
#pragma unroll
            for (int ax = 0; ax < 3; ++ax) {
                bad |= !(v[ax] - v[ax] == 0.0f);
                lo[ax] = __builtin_fminf(lo[ax], v[ax]);
                hi[ax] = __builtin_fmaxf(hi[ax], v[ax]);
                dev[ax] += counts ? __builtin_fminf(__builtin_fabsf(v[ax] - pilot[ax]), cap[ax]) : 0.0f;
            }
        }
#pragma unroll
        for (int k = 0; k < QUADS; ++k)
            reinterpret_cast<uint4 *>(win)[k * NT + tid] = table[k];
    }
#pragma unroll
    for (int ax = 0; ax < 3; ++ax) {
        lo[ax] = wave_reduce_min(lo[ax]);
        hi[ax] = wave_reduce_max(hi[ax]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
            dev[ax] += __shfl_xor(dev[ax], o);
    }
    if (tid == 0) {
        sbad = 0;
        sfar = 0;
    }
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int ax = 0; ax < 3; ++ax) {
            sred[wave][ax] = lo[ax];
            sred[wave][3 + ax] = hi[ax];
            sdev[wave][ax] = dev[ax];
        }
    }
    if (bad)
        sbad = 1;
    __syncthreads();
    float cc[3], flo[3], ext;
    chamfer_frame<NW>(sred, sdev, pilot, n, lo, hi, cc, flo, ext);
    const float c0 = cc[0], c1 = cc[1], c2 = cc[2];
    const int ebits = (int)((__builtin_bit_cast(unsigned, ext) >> 23) & 0xffu) - 127;
    const bool safe = n > 0 && sbad == 0 && (c0 - c0 == 0.0f) && (c1 - c1 == 0.0f) &&
                      (c2 - c2 == 0.0f) && (ext - ext == 0.0f) &&
                      (ext == 0.0f || (ebits >= -40 && ebits <= 40));
    const float scale =
        ext == 0.0f ? 1.0f : __builtin_bit_cast(float, (unsigned)(127 - ebits) << 23);
    if (tid == 0 && part == 0) {
        a.flags[which * a.B + b] = 0;
        if (cloud == 0)
            a.flags[2 * a.B] = 0;
        hdr->c[0] = c0;
        hdr->c[1] = c1;
        hdr->c[2] = c2;
        hdr->scale = scale;
        hdr->unsafe = safe ? 0 : 1;
        hdr->extent = 2.0f * ext;
#pragma unroll
        for (int ax = 0; ax < 3; ++ax) {
            hdr->lo[ax] = lo[ax];
            hdr->hi[ax] = hi[ax];
        }
        if (!safe) {
            hdr->kmax2_bits = 0;
            hdr->far_keys = 0;
        }
    }
    if (!safe)  // uniform over the workgroup
        return;

    // ---- cells, their histogram and the points' ranks within their cells; the far keys
    //      and the largest swept |k'|^2 ----
    const float inv = ext > 0.0f ? (16.0f / ext) * 0.99999f : 0.0f;
    int where[U];  // cell | rank << 15; later the position in sorted order; -1: no point
    float kmax2 = 0.0f;
    {
        TkPoint3<float> p[U];
        load_points(p);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float ux = __builtin_fminf(__builtin_fmaxf((p[u].x - flo[0]) * inv, 0.0f), 31.0f);
            const float uy = __builtin_fminf(__builtin_fmaxf((p[u].y - flo[1]) * inv, 0.0f), 31.0f);
            const float uz = __builtin_fminf(__builtin_fmaxf((p[u].z - flo[2]) * inv, 0.0f), 31.0f);
            where[u] = cell_of[((int)ux << 10) | ((int)uy << 5) | (int)uz];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = u * NT + tid;
            const float x = (p[u].x - c0) * scale, y = (p[u].y - c1) * scale,
                        z = (p[u].z - c2) * scale;
            const float nn = __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x));
            // (a key beyond 4 units of the frame: see chamfer_tile_kernel)
            const bool far = j < n && !(nn <= 16.0f);
            if (far) {
                const int slot = atomicAdd(&sfar, 1);
                if (slot < CHAMFER_FAR_KEYS)
                    sfar_list[slot] =
                        make_float4(p[u].x, p[u].y, p[u].z, __builtin_bit_cast(float, j));
            }
            kmax2 = __builtin_fmaxf(kmax2, (j < n && !far) ? nn : 0.0f);
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int cell = where[u], shift = (cell & 1) * 16;
        int packed = -1;
        if (u * NT + tid < n)
            packed = cell | (int)(((atomicAdd(&hist[cell >> 1], 1u << shift) >> shift) & 0xffffu) << 15);
        where[u] = packed;
    }
    kmax2 = wave_reduce_max(kmax2);
    __syncthreads();
    if (lane == 0)
        sred[wave][0] = kmax2;
    // Every wave turns the 2048 counters of its range into starting positions within the
    // range (at most 16384: they fit the 16 bits); the ranges' own starts are added when a
    // position is looked up.
    {
        constexpr int PER_WAVE = WORDS / NW;
        int carry = 0, occupied = 0;
        for (int i = 0; i < PER_WAVE; i += TK_WAVE) {
            const int at = wave * PER_WAVE + i + lane;
            const unsigned both = hist[at];
            const int even = (int)(both & 0xffffu), odd = (int)(both >> 16);
            occupied += (even != 0) + (odd != 0);
            const int incl = wave_inclusive_sum(even + odd);
            const int start = carry + incl - (even + odd);
            hist[at] = (unsigned)start | ((unsigned)(start + even) << 16);
            carry += __builtin_amdgcn_readlane(incl, TK_WAVE - 1);
        }
        occupied = __builtin_amdgcn_readlane(wave_inclusive_sum(occupied), TK_WAVE - 1);
        if (lane == 0) {
            swave[wave] = carry;
            sred[wave][1] = (float)occupied;  // (at most 2048: exact)
        }
    }
    __syncthreads();
    if (tid <= NW) {
        int run = 0;
        for (int w = 0; w < tid; ++w)
            run += swave[w];
        sstart[tid] = run;  // (sstart[NW] = n)
    }
    if (part == 0) {  // what belongs to the cloud as a whole leaves with its first workgroup
        const int nfar = sfar;
        if (tid == 0) {
            float m = 0.0f, cells = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                m = __builtin_fmaxf(m, sred[w][0]);
                cells += sred[w][1];
            }
            hdr->kmax2_bits = __builtin_bit_cast(int, m);
            hdr->far_keys = nfar;
            hdr->occupied = (int)cells;
        }
        if (tid < nfar && tid < CHAMFER_FAR_KEYS)
            a.far_keys[which][(int64_t)b * CHAMFER_FAR_KEYS + tid] = sfar_list[tid];
    }
    __syncthreads();
    // This part's run of cell ranges [r_lo, r_hi) and of sorted positions [s_lo, s_hi): range
    // boundary q is the first range that starts at or beyond q / parts of the points.
    int r_lo = 0, r_hi = NW;
    if (part > 0 || part + 1 < parts) {
        const int want_lo = (int)(((int64_t)n * part) / parts);
        const int want_hi = (int)(((int64_t)n * (part + 1)) / parts);
        int first_lo = NW, first_hi = NW;
        for (int w = NW - 1; w >= 0; --w) {
            const int at = sstart[w];
            first_lo = at >= want_lo ? w : first_lo;
            first_hi = at >= want_hi ? w : first_hi;
        }
        r_lo = part > 0 ? first_lo : 0;
        r_hi = part + 1 < parts ? first_hi : NW;
    }
    const bool last = part + 1 == parts;
    const int s_lo = sstart[r_lo], s_hi = sstart[r_hi];
    // the part's last tile is shared with later parts when its positions end inside a tile
    const int shared_end = (!last && (s_hi & 31) != 0 && s_hi > s_lo) ? ((s_hi + 31) & ~31) : -1;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int cell = where[u] & 0x7fff, rank = where[u] >> 15;
        const unsigned both = hist[cell >> 1];
        const int start = (int)((cell & 1) ? both >> 16 : both & 0xffffu) + sstart[cell >> 11];
        // bit 20: a point of a later part whose cell begins inside this part's last tile
        const int later = ((cell >> 11) >= r_hi && start < shared_end) ? 1 << 20 : 0;
        where[u] = where[u] < 0 ? -1 : ((start + rank) | later);
    }

    // ---- write-out of the part's positions, in windows ----
    float4 *__restrict__ sorted = a.sorted[which] + (int64_t)b * npad;
    uint4 *__restrict__ terms = a.terms[which] + (int64_t)b * npad * 2;
    uint4 *__restrict__ boxes = a.boxes[which] + (int64_t)b * (npad / 32);
    const float qnan = __builtin_nanf("");
    const int t_lo = s_lo & ~31, t_hi = last ? npad : ((s_hi + 31) & ~31);
    for (int base = t_lo; base < t_hi; base += W) {
        const int width = t_hi - base < W ? t_hi - base : W;
        {
            TkPoint3<float> p[U];
            load_points(p);
            if (base > t_lo)
                __syncthreads();  // the window's previous contents have been read
            int marked = 0;  // bit u: a later part's point whose cell begins in the last tile
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int pos = where[u] & 0xfffff;
                const bool mine = where[u] >= 0 && pos >= s_lo && pos < s_hi;
                const unsigned at = (unsigned)(pos - base);
                // (a point of another window or another part goes to the lane's spare slot:
                // a store that is skipped costs a branch per point)
                win[(mine && at < (unsigned)width) ? at : (unsigned)(W + lane)] =
                    make_float4(p[u].x, p[u].y, p[u].z, __builtin_bit_cast(float, u * NT + tid));
                marked |= (where[u] >= 0 && (where[u] & (1 << 20)) != 0) ? 1 << u : 0;
            }
            if (base == t_lo && marked != 0) {  // (a handful of lanes, if any)
                int extra_lo[3] = {ORDER_POS_INF, ORDER_POS_INF, ORDER_POS_INF};
                int extra_hi[3] = {ORDER_NEG_INF, ORDER_NEG_INF, ORDER_NEG_INF};
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const float x = (p[u].x - c0) * scale, y = (p[u].y - c1) * scale,
                                z = (p[u].z - c2) * scale;
                    if (((marked >> u) & 1) != 0 &&
                        __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x)) <= 16.0f) {
                        const int o[3] = {tk_float_order(x), tk_float_order(y), tk_float_order(z)};
#pragma unroll
                        for (int ax = 0; ax < 3; ++ax) {
                            extra_lo[ax] = o[ax] < extra_lo[ax] ? o[ax] : extra_lo[ax];
                            extra_hi[ax] = o[ax] > extra_hi[ax] ? o[ax] : extra_hi[ax];
                        }
                    }
                }
#pragma unroll
                for (int ax = 0; ax < 3; ++ax) {
                    atomicMin(&sextra[ax], extra_lo[ax]);
                    atomicMax(&sextra[3 + ax], extra_hi[ax]);
                }
            }
        }
        __syncthreads();
        for (int s0 = 0; s0 < width; s0 += NT) {
            const int i = base + s0 + tid;
            if (s0 + tid >= width)  // (uniform over each half wave: width is a multiple of 32)
                continue;
            const bool owned = (i >= s_lo && i < s_hi) || (last && i >= n);
            const bool exists = owned && i < n;
            float4 s = make_float4(qnan, qnan, qnan, __builtin_bit_cast(float, -1));
            if (exists)
                s = win[s0 + tid];
            const float x = ((exists ? s.x : c0) - c0) * scale;
            const float y = ((exists ? s.y : c1) - c1) * scale;
            const float z = ((exists ? s.z : c2) - c2) * scale;
            const float nn = __builtin_fmaf(z, z, __builtin_fmaf(y, y, x * x));
            const bool swept = exists && nn <= 16.0f;
            if (owned) {
                sorted[i] = s;
                uint4 h0, h1;
                chamfer_key_terms(x, y, z, nn, swept, h0, h1);
                uint4 *tile = terms + (i >> 5) * 64 + (i & 31);
                tile[0] = h0;
                tile[32] = h1;
            }
            int bl[3], bh[3];
            bl[0] = half_wave_reduce_to_last<false>(swept ? tk_float_order(x) : ORDER_POS_INF);
            bl[1] = half_wave_reduce_to_last<false>(swept ? tk_float_order(y) : ORDER_POS_INF);
            bl[2] = half_wave_reduce_to_last<false>(swept ? tk_float_order(z) : ORDER_POS_INF);
            bh[0] = half_wave_reduce_to_last<true>(swept ? tk_float_order(x) : ORDER_NEG_INF);
            bh[1] = half_wave_reduce_to_last<true>(swept ? tk_float_order(y) : ORDER_NEG_INF);
            bh[2] = half_wave_reduce_to_last<true>(swept ? tk_float_order(z) : ORDER_NEG_INF);
            // the tile's box comes from the part that owns the tile's first position
            if ((i & 31) == 31 && i - 31 >= s_lo) {
                if (i + 1 == shared_end) {
#pragma unroll
                    for (int ax = 0; ax < 3; ++ax) {
                        bl[ax] = sextra[ax] < bl[ax] ? sextra[ax] : bl[ax];
                        bh[ax] = sextra[3 + ax] > bh[ax] ? sextra[3 + ax] : bh[ax];
                    }
                }
                const float fl[3] = {tk_order_float(bl[0]), tk_order_float(bl[1]), tk_order_float(bl[2])};
                const float fh[3] = {tk_order_float(bh[0]), tk_order_float(bh[1]), tk_order_float(bh[2])};
                boxes[i >> 5] = chamfer_box_bits(fl, fh);
            }
        }
    }
}

struct ChamferPrunedArgs {
    const float4 *sorted[2];
    const uint4 *terms[2];
    const uint4 *boxes[2];
    const float4 *far_keys[2];
    const ChamferSortedHdr *hdr;
    int *flags;
    float *dist[2];
    int64_t *idx[2];
    int n[2], npad[2];
    int B;
    int waves_per_cloud[2];
    int waves0;  // waves of direction 0 (queries: cloud 0); the rest belong to direction 1
    unsigned long long *counters;  // COUNT builds only: executed work, four words
};

__device__ __forceinline__ int wave_reduce_min_int(int v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const int other = __shfl_xor(v, o);
        v = other < v ? other : v;
    }
    return v;
}

// Whether at least three quarters of a key cloud's tiles may hold a key as near to some point
// of the box (flo, fhi) as that point's nearest key is at most: first an upper bound of any
// such point's distance to its nearest key (the least, over the tiles, of the distance
// between farthest corners), then the tiles whose boxes come that near. The bound is a
// tile's diameter too loose, which only clouds of a few hundred tiles can afford. Called by
// a whole wave with the same arguments in every lane; coordinates are the key cloud's
// centred, scaled ones. (Keeping its arguments and registers few matters: a version that
// also read the nearest tile's keys raised the calling kernel from 112 to 122 registers, and
// ordinary clouds lost 7 %.)
__device__ __attribute__((noinline)) bool chamfer_most_tiles_within_reach(
    const uint4 *__restrict__ BX, int ntiles, float flo0, float flo1, float flo2, float fhi0,
    float fhi1, float fhi2)
{
    const float INF = __builtin_huge_valf();
    const int lane = threadIdx.x & (TK_WAVE - 1);
    const int rounds = (ntiles + TK_WAVE - 1) / TK_WAVE;
    float ub = INF;
    int within_reach = 0;
#pragma unroll 1
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll 1
        for (int r = 0; r < rounds; ++r) {
            const int t = r * TK_WAVE + lane;
            const uint4 box = BX[t < ntiles ? t : 0];
            const float lx = tk_f16_value(box.x & 0xffffu), ly = tk_f16_value(box.x >> 16);
            const float lz = tk_f16_value(box.y & 0xffffu), hx = tk_f16_value(box.y >> 16);
            const float hy = tk_f16_value(box.z & 0xffffu), hz = tk_f16_value(box.z >> 16);
            if (pass == 0) {  // an empty box (lo = +inf, hi = -inf): +inf
                const float mx = __builtin_fmaxf(hx - flo0, fhi0 - lx);
                const float my = __builtin_fmaxf(hy - flo1, fhi1 - ly);
                const float mz = __builtin_fmaxf(hz - flo2, fhi2 - lz);
                const float m2 = __builtin_fmaf(mz, mz, __builtin_fmaf(my, my, mx * mx));
                ub = t < ntiles ? __builtin_fminf(ub, m2) : ub;
            } else {
                const float gx = __builtin_fmaxf(0.0f, __builtin_fmaxf(lx - fhi0, flo0 - hx));
                const float gy = __builtin_fmaxf(0.0f, __builtin_fmaxf(ly - fhi1, flo1 - hy));
                const float gz = __builtin_fmaxf(0.0f, __builtin_fmaxf(lz - fhi2, flo2 - hz));
                const float gap2 = __builtin_fmaf(gz, gz, __builtin_fmaf(gy, gy, gx * gx));
                within_reach +=
                    __builtin_popcountll(__builtin_amdgcn_ballot_w64(t < ntiles && gap2 <= ub));
            }
        }
        if (pass == 0)
            ub = wave_reduce_min(ub);
    }
    return within_reach * 4 >= ntiles * 3;
}

// (Launched one wave per workgroup - waves share nothing, and a finished wave frees its
// slot at once: 2-3 % over four waves per workgroup. The bound of 256 lanes only caps the
// registers at four waves per SIMD.)
template <int NQB, int RMAX, bool COUNT = false>
__global__ __launch_bounds__(256) void chamfer_pruned_kernel(ChamferPrunedArgs a)
{
    const int tid = threadIdx.x;
    const int lane = tid & (TK_WAVE - 1);
    const int col = lane & 31, half = lane >> 5;
    const float INF = __builtin_huge_valf();
    // the workgroups of a cloud on one XCD, as in chamfer_decode_block
    int lb = blockIdx.x;
    {
        const int nb = gridDim.x, per = nb >> 3, full = per << 3;
        if (lb < full)
            lb = (lb & 7) * per + (lb >> 3);
    }
    // A batch element's two directions follow each other, so that the XCD whose L2 holds its
    // two sorted clouds serves both.
    const int wid = __builtin_amdgcn_readfirstlane(lb + tid / TK_WAVE);
    const int wpb = a.waves_per_cloud[0] + a.waves_per_cloud[1];
    const int b = wid / wpb;
    if (b >= a.B)
        return;
    const int within = wid - b * wpb;
    const int which = within >= a.waves_per_cloud[0];
    const int qw = within - (which ? a.waves_per_cloud[0] : 0);
    const int nq = a.n[which], npq = a.npad[which], npk = a.npad[1 - which];
    const ChamferSortedHdr *hq = a.hdr + which * a.B + b;
    const ChamferSortedHdr *hk = a.hdr + (1 - which) * a.B + b;
    int *flag = a.flags + which * a.B + b;
    // this cloud and direction goes to the sweep of all pairs (one word says that any does)
    auto hand_over = [&]() {
        atomicOr(flag, 1);
        atomicOr(a.flags + 2 * a.B, 1);
    };
    const float4 *__restrict__ SQ = a.sorted[which] + (int64_t)b * npq;
    const float4 *__restrict__ SK = a.sorted[1 - which] + (int64_t)b * npk;
    const uint4 *__restrict__ TK = a.terms[1 - which] + (int64_t)b * npk * 2;
    const uint4 *__restrict__ BX = a.boxes[1 - which] + (int64_t)b * (npk / 32);
    const float4 *__restrict__ FK = a.far_keys[1 - which] + (int64_t)b * CHAMFER_FAR_KEYS;
    const int ntiles = npk / 32;
    const int rounds = (ntiles + TK_WAVE - 1) / TK_WAVE;  // <= RMAX
    // The wave's queries and the first boxes are requested before anything is known about
    // the clouds (the addresses are inside the workspace whatever it holds): one round
    // trip to memory instead of three in a row.
    float4 squery[NQB];
    uint4 box0[8];
#pragma unroll
    for (int g = 0; g < NQB; ++g)
        squery[g] = SQ[(qw * NQB + g) * 32 + col];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const int t = r * TK_WAVE + lane;
        box0[r] = BX[t < ntiles ? t : 0];
    }
    const int handed_over = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_sched_barrier(0);
    const float c0 = hk->c[0], c1 = hk->c[1], c2 = hk->c[2], scale = hk->scale;
    // the farthest corner of the query cloud's frame from the key cloud's centre, in key
    // extents (stray queries beyond the frame are looked at one by one below)
    float far2 = 0.0f;
    {
        const float cc[3] = {c0, c1, c2};
#pragma unroll
        for (int ax = 0; ax < 3; ++ax) {
            const float m =
                (__builtin_fabsf(hq->c[ax] - cc[ax]) + 0.5f * hq->extent) * scale;
            far2 = __builtin_fmaf(m, m, far2);
        }
    }
    // A key cloud much smaller than the query cloud (by their frames): most queries are far
    // from it compared with its size, every one of its tiles is within their reach, and
    // this kernel would sweep all pairs at four times the matrix kernel's cost per tile.
    const bool dwarfed = ntiles >= 16 && hk->extent < 0.25f * hq->extent;
    const int nfar = hk->far_keys;  // keys kept out of the sweep (far outside the frame)
    // (What follows from the headers alone is the same for every wave of the cloud: its
    // first wave raises the flag, the others just leave - thousands of atomics on one word
    // took 50 us.)
    if (hq->unsafe != 0 || hk->unsafe != 0) {  // uniform over the wave
        if (lane == 0 && qw == 0)
            hand_over();
        return;
    }
    if (hk->lo[0] == hk->hi[0] && hk->lo[1] == hk->hi[1] && hk->lo[2] == hk->hi[2]) {
        // Every key is the same point (uniform over the wave): each query's nearest key is
        // key 0 at that point - or none, if the distance overflows (strict '<' from +inf).
#pragma unroll
        for (int g = 0; g < NQB; ++g) {
            const int id = __builtin_bit_cast(int, squery[g].w);
            const float dd = tk_dist2<float>(hk->lo[0], hk->lo[1], hk->lo[2], squery[g].x,
                                             squery[g].y, squery[g].z);
            if (half == 0 && id >= 0) {
                const int64_t o = (int64_t)b * nq + id;
                a.dist[which][o] = dd < INF ? dd : INF;
                a.idx[which][o] = dd < INF ? 0 : -1;
            }
        }
        return;
    }
    // The error bound of the scores counts on a swept key with |k'| >= 1/4 (the fp16 pieces
    // have an absolute floor): a frame that outliers stretched far beyond the bulk of the
    // keys does not give one.
    const bool flat_terms = hk->kmax2_bits < 0x3d800000;  // |k'|^2 < 1/16 for every swept key
    // Keys crowded into few cells - over a hundred per occupied cell: points on a line, or a
    // few hundred distinct points repeated - put several tiles of equal or nearly equal keys
    // in front of every query; the exact scans that follow cost more than all pairs do.
    const bool crowded = ntiles >= 16 && (int64_t)hk->occupied * 128 < a.n[1 - which];
    if (!(far2 <= 6.4e7f) || dwarfed || flat_terms || crowded ||
        nfar > CHAMFER_FAR_KEYS) {  // uniform over the wave
        if (lane == 0 && qw == 0)
            hand_over();
        return;
    }
    if (handed_over != 0)
        return;  // the cloud goes to the other kernel anyway
    // A query cloud much smaller than the key cloud (by their frames) with most key tiles about
    // as far from it as the nearest one - a cluster of queries inside a shell of keys: every
    // wave would find nearly every tile within reach (B=8, 16384 points: 0.91 ms where all
    // pairs take 0.72). From 256 tiles on, where the boxes are small enough to tell. (A call,
    // not inlined: the test is rare and its code inside this kernel cost ordinary clouds
    // 2-5 %.)
    if (ntiles >= 256 && hq->extent < 0.25f * hk->extent) {  // uniform over the wave
        const float h = 0.5f * hq->extent * scale;
        const float m0 = (hq->c[0] - c0) * scale, m1 = (hq->c[1] - c1) * scale,
                    m2 = (hq->c[2] - c2) * scale;
        if (chamfer_most_tiles_within_reach(BX, ntiles, m0 - h, m1 - h, m2 - h, m0 + h, m1 + h,
                                            m2 + h)) {
            if (lane == 0 && qw == 0)
                hand_over();
            return;
        }
    }
    const float kmax =
        __builtin_sqrtf(__builtin_bit_cast(float, hk->kmax2_bits)) * 1.000001f;
    const float guard = 1e-36f * scale * scale;

    // ---- queries ----
    tk_f16x8 qterm[NQB];
    float qnorm[NQB], qn2[NQB], rx[NQB], ry[NQB], rz[NQB];
    int qid[NQB];
    // live: a query the sweep serves; stray: a query too far from the key cloud for the
    // fp16 terms (beyond 8000 key extents), served by an exact scan of all keys instead
    bool live[NQB], stray[NQB];
    float v0[NQB], v1[NQB], v2[NQB];
    int id0[NQB], id1[NQB];
    float blo[3] = {INF, INF, INF}, bhi[3] = {-INF, -INF, -INF};
    float qnmax = 0.0f;
    int nstray = 0;
#pragma unroll
    for (int g = 0; g < NQB; ++g) {
        const float4 s = squery[g];
        qid[g] = __builtin_bit_cast(int, s.w);
        const bool ok = qid[g] >= 0;
        rx[g] = s.x;
        ry[g] = s.y;
        rz[g] = s.z;
        float px = ((ok ? s.x : c0) - c0) * scale;
        float py = ((ok ? s.y : c1) - c1) * scale;
        float pz = ((ok ? s.z : c2) - c2) * scale;
        const bool near = __builtin_fmaf(pz, pz, __builtin_fmaf(py, py, px * px)) <= 6.4e7f;
        live[g] = ok && near;
        stray[g] = ok && !near;
        nstray += __builtin_popcountll(__builtin_amdgcn_ballot_w64(stray[g] && half == 0));
        px = near ? px : 0.0f;
        py = near ? py : 0.0f;
        pz = near ? pz : 0.0f;
        qn2[g] = __builtin_fmaf(pz, pz, __builtin_fmaf(py, py, px * px));
        qnorm[g] = 1.000001f * __builtin_sqrtf(qn2[g]);
        qterm[g] = __builtin_bit_cast(tk_f16x8, chamfer_query_terms(px, py, pz, half));
        v0[g] = v1[g] = v2[g] = INF;
        id0[g] = id1[g] = -1;
        if (live[g]) {
            blo[0] = __builtin_fminf(blo[0], px);
            blo[1] = __builtin_fminf(blo[1], py);
            blo[2] = __builtin_fminf(blo[2], pz);
            bhi[0] = __builtin_fmaxf(bhi[0], px);
            bhi[1] = __builtin_fmaxf(bhi[1], py);
            bhi[2] = __builtin_fmaxf(bhi[2], pz);
            qnmax = __builtin_fmaxf(qnmax, qnorm[g]);
        }
    }
#pragma unroll
    for (int ax = 0; ax < 3; ++ax) {
        blo[ax] = wave_reduce_min(blo[ax]);
        bhi[ax] = wave_reduce_max(bhi[ax]);
    }
    const bool nothing_to_sweep = !(blo[0] <= bhi[0]);  // padding and strays only (uniform)
    if (nothing_to_sweep && nstray == 0)
        return;
    // An exact scan of all keys costs what scanning every tile costs: more than 16384
    // (query, tile) pairs of it per wave and the cloud is handed over.
    if ((int64_t)nstray * ntiles > 16384) {
        if (lane == 0)
            hand_over();
        return;
    }
#pragma unroll
    for (int ax = 0; ax < 3; ++ax) {  // (the same in every lane: scalar registers)
        blo[ax] = __builtin_bit_cast(
            float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, blo[ax])));
        bhi[ax] = __builtin_bit_cast(
            float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, bhi[ax])));
    }
    qnmax = wave_reduce_max(qnmax);
    const float rw = kmax + qnmax;
    const float slackw = rw * rw * 7.6293945e-06f + guard;  // 2^-17 R of the wave

    // squared gap between the wave's patch and the box of each of this lane's tiles (tile
    // r * 64 + lane in g2[r]; an empty box or no tile: +inf)
    float g2[RMAX];
#pragma unroll
    for (int r0 = 0; r0 < RMAX; r0 += 8) {  // eight boxes in flight at a time
        if (r0 >= rounds) {  // uniform over the wave: no tiles left
#pragma unroll
            for (int r = 0; r < 8; ++r)
                g2[r0 + r] = INF;
            continue;
        }
        uint4 box[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int t = (r0 + r) * TK_WAVE + lane;
            box[r] = r0 == 0 ? box0[r] : BX[t < ntiles ? t : 0];
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const float lx = tk_f16_value(box[r].x & 0xffffu), ly = tk_f16_value(box[r].x >> 16);
            const float lz = tk_f16_value(box[r].y & 0xffffu), hx = tk_f16_value(box[r].y >> 16);
            const float hy = tk_f16_value(box[r].z & 0xffffu), hz = tk_f16_value(box[r].z >> 16);
            const float gx = __builtin_fmaxf(0.0f, __builtin_fmaxf(lx - bhi[0], blo[0] - hx));
            const float gy = __builtin_fmaxf(0.0f, __builtin_fmaxf(ly - bhi[1], blo[1] - hy));
            const float gz = __builtin_fmaxf(0.0f, __builtin_fmaxf(lz - bhi[2], blo[2] - hz));
            g2[r0 + r] = (r0 + r) * TK_WAVE + lane < ntiles
                             ? __builtin_fmaf(gz, gz, __builtin_fmaf(gy, gy, gx * gx))
                             : INF;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    const tk_f32x16 zero = {};
    auto sweep_tile = [&](const tk_f16x8 &ka, int t) {
#pragma unroll
        for (int g = 0; g < NQB; ++g) {
            const tk_f32x16 acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qterm[g], zero, 0, 0, 0);
            const float x = chamfer_fold16(INF, acc);
            const bool lt0 = x < v0[g];
            const bool lt1 = x < v1[g];
            id1[g] = lt1 ? t : id1[g];
            id1[g] = lt0 ? id0[g] : id1[g];
            id0[g] = lt0 ? t : id0[g];
            v2[g] = __builtin_amdgcn_fmed3f(v1[g], v2[g], x);
            v1[g] = __builtin_amdgcn_fmed3f(v0[g], v1[g], x);
            v0[g] = __builtin_amdgcn_fmed3f(-INF, v0[g], x);
        }
    };
    unsigned swept = 0;  // bit r: tile r * 64 + lane has been swept
    int nswept = 0;
    // an upper bound of every query's squared distance to its nearest key so far
    auto bound = [&]() {
        float ub = -INF;
#pragma unroll
        for (int g = 0; g < NQB; ++g) {
            const float best = __builtin_fminf(v0[g], __shfl_xor(v0[g], 32));
            ub = live[g] ? __builtin_fmaxf(ub, best + qn2[g]) : ub;
        }
        return wave_reduce_max(ub);
    };
    // Up to three passes (one copy of the code): the tiles that overlap the patch - without
    // any, the nearest tile -, then everything within reach at T. When the first pass met
    // fewer than four tiles T is still loose, and a pass at T/4 tightens it first.
#pragma unroll 1
    for (int phase = 0; phase < (nothing_to_sweep ? 0 : 3); ++phase) {
        float thr = 0.0f;
        if (phase == 1 && nswept >= 4)  // uniform over the wave
            continue;
        if (phase > 0) {
            if (nswept == 0) {  // (phase 1 only) uniform over the wave
                float best = INF;
                int at = -1;
#pragma unroll
                for (int r = 0; r < RMAX; ++r) {
                    if (g2[r] < best) {
                        best = g2[r];
                        at = r * TK_WAVE + lane;
                    }
                }
                const float least = wave_reduce_min(best);
                const unsigned long long m =
                    __builtin_amdgcn_ballot_w64(best == least && at >= 0);
                if (m == 0) {  // no key tile holds a point (cannot happen with nk >= 1)
                    if (lane == 0)
                        hand_over();
                    return;
                }
                const int t = __builtin_amdgcn_readlane(at, (int)__builtin_ctzll(m));
                if (lane == (t & (TK_WAVE - 1)))
                    swept |= 1u << (t / TK_WAVE);
                sweep_tile(__builtin_bit_cast(tk_f16x8, TK[(int64_t)t * 64 + lane]), t);
                ++nswept;
            }
            const float reach = phase == 1 ? 0.25f : 1.001f;
            // (finite, so that the +inf of a tile that does not exist never passes)
            thr = __builtin_fminf((bound() + slackw) * reach, 3.0e38f);
        }
        unsigned takes = 0;
#pragma unroll
        for (int r = 0; r < RMAX; ++r)
            takes |= g2[r] <= thr ? 1u << r : 0u;
        takes &= ~swept;
        swept |= takes;
#pragma unroll 1
        for (int r = 0; r < rounds; ++r) {
            unsigned long long m = __builtin_amdgcn_ballot_w64(((takes >> r) & 1u) != 0);
            while (m != 0) {  // four tiles in flight at a time
                int t[4];
                uint4 ka[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    t[u] = -1;
                    if (m != 0) {
                        t[u] = r * TK_WAVE + (int)__builtin_ctzll(m);
                        m &= m - 1;
                        ka[u] = TK[(int64_t)t[u] * 64 + lane];
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (t[u] >= 0) {
                        sweep_tile(__builtin_bit_cast(tk_f16x8, ka[u]), t[u]);
                        ++nswept;
                    }
                }
            }
        }
    }

    if constexpr (COUNT) {  // matrix instructions issued and waves that swept
        if (lane == 0 && nswept > 0) {
            atomicAdd(a.counters + 0, (unsigned long long)nswept * NQB);
            atomicAdd(a.counters + 1, 1ull);
        }
    }
    // ---- exact evaluation of each half's candidate tiles, then the merge ----
    unsigned over_mask[NQB], stray_mask[NQB];
    int nover = 0;
#pragma unroll
    for (int g = 0; g < NQB; ++g) {
        const bool ok = live[g];
        stray_mask[g] = (unsigned)__builtin_amdgcn_ballot_w64(stray[g] && half == 0);
        const float best_score = __builtin_fminf(v0[g], __shfl_xor(v0[g], 32));
        const float r = kmax + qnorm[g];
        const float thr = best_score + (r * r * 7.6293945e-06f + guard);  // 2^-17 R
        const bool crowded = v2[g] <= thr;  // three or more candidate tiles in this half
        const bool over =
            ok && ((__builtin_amdgcn_ballot_w64(crowded) >> col & 0x100000001ull) != 0);
        float bestd = INF;
        int bestj = -1;
        // (distance bits << 32 | original index): distances are non-negative, so the words
        // order as (distance, index) pairs; a NaN (padding) is above +inf and never taken
        unsigned long long best = (0x7f800000ull << 32) | 0xffffffffull;
        if (ok && !over) {
            const int ta = v0[g] <= thr ? id0[g] : -1, tb = v1[g] <= thr ? id1[g] : -1;
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                const int tile = pass == 0 ? ta : tb;
                if (tile < 0)
                    continue;
                // this half's keys of the tile: runs of 4 keys, 8 keys apart
                const float4 *p = SK + (int64_t)tile * 32 + half * 4;
                float4 f[16];
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    f[e] = p[(e >> 2) * 8 + (e & 3)];
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float dd = tk_dist2<float>(f[e].x, f[e].y, f[e].z, rx[g], ry[g], rz[g]);
                    const unsigned long long word =
                        ((unsigned long long)__builtin_bit_cast(unsigned, dd) << 32) |
                        __builtin_bit_cast(unsigned, f[e].w);
                    best = word < best ? word : best;
                }
            }
            // (a distance that overflowed is no match: strict '<' from +inf)
            const float d = __builtin_bit_cast(float, (unsigned)(best >> 32));
            bestd = d < INF ? d : INF;
            bestj = d < INF ? (int)(unsigned)best : -1;
        }
        // the other half's result: smaller distance, then lower key index
        const float od = __shfl_xor(bestd, 32);
        const int oj = __shfl_xor(bestj, 32);
        if (oj >= 0 && (bestj < 0 || od < bestd || (od == bestd && oj < bestj))) {
            bestd = od;
            bestj = oj;
        }
        for (int e = 0; e < nfar; ++e) {  // (uniform; usually none)
            const float4 f = FK[e];
            const float dd = tk_dist2<float>(f.x, f.y, f.z, rx[g], ry[g], rz[g]);
            const int fj = __builtin_bit_cast(int, f.w);
            if (dd < bestd || (dd == bestd && fj < bestj)) {
                bestd = dd;
                bestj = fj;
            }
        }
        if (half == 0 && ok && !over) {
            const int64_t o = (int64_t)b * nq + qid[g];
            a.dist[which][o] = bestd;
            a.idx[which][o] = (int64_t)bestj;
        }
        over_mask[g] = (unsigned)__builtin_amdgcn_ballot_w64(over && half == 0);
        nover += __builtin_popcount(over_mask[g]);
    }
    if (nover == 0 && nstray == 0)
        return;
    if constexpr (COUNT) {  // queries that take an exact scan
        if (lane == 0)
            atomicAdd(a.counters + 2, (unsigned long long)(nover + nstray));
    }
    // An exact scan costs about 13 instructions per two swept tiles and query, a normal wave
    // issues 2100 in all: beyond 2048 (query, tile) pairs - six times a wave's usual work - the
    // cloud is handed to the other kernel (heavy ties: quantised or duplicated points; clouds
    // of duplicated collinear points spent 0.9 ms here before the limit came down from 8192),
    // and a wave whose cloud another wave has handed over meanwhile does not scan either.
    if ((int64_t)nover * nswept > 2048) {
        if (lane == 0)
            hand_over();
        return;
    }
    if (nover > 8 && __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)
        return;
    // ---- queries with three or more candidate tiles: exact scan of the swept tiles;
    //      stray queries: exact scan of all tiles ----
#pragma unroll
    for (int g = 0; g < NQB; ++g) {
        unsigned m = over_mask[g] | stray_mask[g];
        while (m != 0) {
            const int src = __builtin_ctz(m);
            m &= m - 1;
            const bool all_tiles = ((stray_mask[g] >> src) & 1u) != 0;  // uniform
            const float qx = __builtin_bit_cast(
                float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, rx[g]), src));
            const float qy = __builtin_bit_cast(
                float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ry[g]), src));
            const float qz = __builtin_bit_cast(
                float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, rz[g]), src));
            const int out = __builtin_amdgcn_readlane(qid[g], src);
            float bestd = INF;
            int bestj = -1;
            // two swept tiles at a time, lane l taking key l % 32 of the tile of its half
#pragma unroll 1
            for (int r = 0; r < rounds; ++r) {
                unsigned long long mm = __builtin_amdgcn_ballot_w64(
                    all_tiles ? r * TK_WAVE + lane < ntiles : ((swept >> r) & 1u) != 0);
                while (mm != 0) {
                    const int t0 = r * TK_WAVE + (int)__builtin_ctzll(mm);
                    mm &= mm - 1;
                    int t1 = -1;
                    if (mm != 0) {
                        t1 = r * TK_WAVE + (int)__builtin_ctzll(mm);
                        mm &= mm - 1;
                    }
                    const int mine = half == 0 ? t0 : t1;
                    if (mine >= 0) {
                        const float4 f = SK[(int64_t)mine * 32 + col];
                        const float dd = tk_dist2<float>(f.x, f.y, f.z, qx, qy, qz);
                        const int oj = __builtin_bit_cast(int, f.w);
                        if (dd < bestd || (dd == bestd && oj < bestj)) {
                            bestd = dd;
                            bestj = oj;
                        }
                    }
                }
            }
            if (lane < nfar) {  // the keys kept out of the sweep, one per lane
                const float4 f = FK[lane];
                const float dd = tk_dist2<float>(f.x, f.y, f.z, qx, qy, qz);
                const int fj = __builtin_bit_cast(int, f.w);
                if (dd < bestd || (dd == bestd && fj < bestj)) {
                    bestd = dd;
                    bestj = fj;
                }
            }
            const float least = wave_reduce_min(bestd);
            const int cand = (bestd == least && bestj >= 0) ? bestj : 0x7fffffff;
            const int first = wave_reduce_min_int(cand);
            if (lane == 0) {
                const int64_t o = (int64_t)b * nq + out;
                a.dist[which][o] = first == 0x7fffffff ? INF : least;
                a.idx[which][o] = first == 0x7fffffff ? -1 : (int64_t)first;
            }
        }
    }
}

// The sorted path can serve clouds of 1 to 65536 points each (a lane's 32-bit mask of
// swept tiles covers 2048 tiles of 32 keys) ...
constexpr int64_t CHAMFER_SORTED_MIN = 1, CHAMFER_SORTED_MAX = 65536;

inline bool chamfer_sorted_can_serve(int64_t B, int64_t N1, int64_t N2)
{
    return B >= 1 && B <= (1 << 20) && N1 >= CHAMFER_SORTED_MIN && N2 >= CHAMFER_SORTED_MIN &&
           N1 <= CHAMFER_SORTED_MAX && N2 <= CHAMFER_SORTED_MAX;
}

// ... and pays where the sweeps it saves outweigh its five launches and the sort: from
// half a billion pairs per direction on clouds of 4096 points and more whose lengths are
// within a factor of four (30 timed shapes: B=32, 4096 x 4096 1.08 times faster than the
// full sweep, B=8, 8192 x 8192 1.16, B=4, 16384 x 16384 1.7, B=32, 16384 x 16384 4.0,
// B=1, 65536 x 65536 2.4; B=16, 4096 x 4096 0.84 and B=4, 65536 x 2048 0.39 stay with the
// full sweep).
inline bool chamfer_sorted_serves(int64_t B, int64_t N1, int64_t N2)
{
    const int64_t lo = N1 < N2 ? N1 : N2, hi = N1 < N2 ? N2 : N1;
    return chamfer_sorted_can_serve(B, N1, N2) && lo >= 4096 && hi <= 4 * lo &&
           (double)B * (double)N1 * (double)N2 >= 5.0e8;
}

struct ChamferSortedLayout {
    size_t hdr, flags, sorted[2], terms[2], boxes[2], far_keys[2], total;
    int64_t npad[2];
};

inline ChamferSortedLayout chamfer_sorted_layout(int64_t B, int64_t N1, int64_t N2)
{
    ChamferSortedLayout l;
    const int64_t n[2] = {N1, N2};
    size_t at = 0;
    auto take = [&](size_t bytes) {
        const size_t here = at;
        at += (bytes + 255) / 256 * 256;
        return here;
    };
    l.hdr = take((size_t)2 * B * sizeof(ChamferSortedHdr));
    l.flags = take((size_t)(2 * B + 1) * sizeof(int));
    for (int w = 0; w < 2; ++w) {
        l.npad[w] = (n[w] + 127) / 128 * 128;
        l.sorted[w] = take((size_t)B * l.npad[w] * sizeof(float4));
        l.terms[w] = take((size_t)B * l.npad[w] * 2 * sizeof(uint4));
        l.boxes[w] = take((size_t)B * (l.npad[w] / 32) * sizeof(uint4));
        l.far_keys[w] = take((size_t)B * CHAMFER_FAR_KEYS * sizeof(float4));
    }
    l.total = at;
    return l;
}

__global__ __launch_bounds__(256) void chamfer_count_clear_kernel(unsigned long long *counters)
{
    if (threadIdx.x < 4)
        counters[threadIdx.x] = 0ull;
}

__global__ __launch_bounds__(256) void chamfer_count_flags_kernel(const int *flags, int n,
                                                                 unsigned long long *counters)
{
    unsigned long long mine = 0;
    for (int i = threadIdx.x; i < n; i += 256)
        mine += flags[i] != 0 ? 1ull : 0ull;
    if (mine != 0)
        atomicAdd(counters + 3, mine);
}

int chamfer_forward_sorted(const float *xyz1, const float *xyz2, int64_t B, int64_t N1,
                           int64_t N2, float *dist1, int64_t *idx1, float *dist2, int64_t *idx2,
                           void *workspace, hipStream_t s, unsigned long long *counters = nullptr,
                           int stages = 7, bool channels_first = false)
{
    // ([3,N] clouds: read in place by chamfer_prepare_kernel and by the hand-over launch;
    // the callers keep clouds of more than 16384 points away)
    // stages (tests and the benchmark time them apart): 1 the preparing launches, 2 the
    // pruned sweep, 4 the hand-over check
    constexpr int NQB = 2;
    const ChamferSortedLayout l = chamfer_sorted_layout(B, N1, N2);
    char *ws = static_cast<char *>(workspace);
    ChamferSortArgs sa;
    ChamferPrunedArgs pa;
    const float *xyz[2] = {xyz1, xyz2};
    const int64_t n[2] = {N1, N2};
    for (int w = 0; w < 2; ++w) {
        sa.xyz[w] = xyz[w];
        sa.sorted[w] = reinterpret_cast<float4 *>(ws + l.sorted[w]);
        sa.terms[w] = reinterpret_cast<uint4 *>(ws + l.terms[w]);
        sa.boxes[w] = reinterpret_cast<uint4 *>(ws + l.boxes[w]);
        sa.far_keys[w] = reinterpret_cast<float4 *>(ws + l.far_keys[w]);
        sa.n[w] = (int)n[w];
        sa.npad[w] = (int)l.npad[w];
        pa.sorted[w] = sa.sorted[w];
        pa.terms[w] = sa.terms[w];
        pa.boxes[w] = sa.boxes[w];
        pa.far_keys[w] = sa.far_keys[w];
        pa.n[w] = sa.n[w];
        pa.npad[w] = sa.npad[w];
        pa.waves_per_cloud[w] = (int)((l.npad[w] + 32 * NQB - 1) / (32 * NQB));
    }
    sa.hdr = reinterpret_cast<ChamferSortedHdr *>(ws + l.hdr);
    sa.flags = reinterpret_cast<int *>(ws + l.flags);
    sa.B = (int)B;
    sa.channels_first = channels_first ? 1 : 0;
    pa.hdr = sa.hdr;
    pa.flags = sa.flags;
    pa.dist[0] = dist1;
    pa.dist[1] = dist2;
    pa.idx[0] = idx1;
    pa.idx[1] = idx2;
    pa.B = (int)B;
    const int64_t waves0 = B * pa.waves_per_cloud[0], waves1 = B * pa.waves_per_cloud[1];
    if (waves0 + waves1 > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    pa.waves0 = (int)waves0;
    pa.counters = counters;
    if (counters != nullptr)
        hipLaunchKernelGGL(chamfer_count_clear_kernel, dim3(1), dim3(256), 0, s, counters);
    constexpr size_t lds = (size_t)CHAMFER_SORT_CELLS * sizeof(int);
    const int allowed = tk_allow_dynamic_lds<chamfer_sort_kernel>((int)lds);
    if (allowed != TK3D_OK)
        return allowed;
    if (stages & 1) {
        // clouds of up to 16384 points: one launch; longer ones: cell, sort and tile kernels
        int first = 2 * (int)B, count = 0;
        for (int w = 1; w >= 0; --w) {
            sa.three_launches[w] = n[w] > PREP_MAX_POINTS;
            if (!sa.three_launches[w]) {
                first = w * (int)B;
                count += (int)B;
            }
        }
        // (both clouds short: first = 0, count = 2 B; one: its own B clouds)
        if (count > 0) {
            const int ok = tk_allow_dynamic_lds<chamfer_prepare_kernel>((int)PREP_LDS_BYTES);
            if (ok != TK3D_OK)
                return ok;
            // workgroups per cloud: as many (4, 2 or 1) as one round over the chip's compute
            // units allows, each with about 2048 sorted positions or more to write out
            const int64_t shortest = sa.three_launches[0] ? n[1] : sa.three_launches[1] ? n[0]
                                     : (n[0] < n[1] ? n[0] : n[1]);
            int parts = 1;
            while (parts < 4 && (int64_t)count * parts * 2 <= tk_cu_count() + tk_cu_count() / 4 &&
                   shortest >= 2048 * parts * 2)
                parts *= 2;
            hipLaunchKernelGGL(chamfer_prepare_kernel, dim3((unsigned)(count * parts)), dim3(1024),
                               PREP_LDS_BYTES, s, sa, first, parts);
        }
        if (sa.three_launches[0] || sa.three_launches[1]) {
            hipLaunchKernelGGL(chamfer_cell_kernel, dim3((unsigned)(2 * B * CHAMFER_CELL_PARTS)),
                               dim3(1024), 0, s, sa);
            hipLaunchKernelGGL(chamfer_sort_kernel, dim3((unsigned)(2 * B)), dim3(1024), lds, s, sa);
            const int64_t tb0 = B * ((l.npad[0] + 255) / 256), tb1 = B * ((l.npad[1] + 255) / 256);
            hipLaunchKernelGGL(chamfer_tile_kernel, dim3((unsigned)(tb0 + tb1)), dim3(256), 0, s,
                               sa, (int)tb0);
        }
    }
    const dim3 grid((unsigned)((waves0 + waves1)));
    const bool small = l.npad[0] <= 16384 && l.npad[1] <= 16384;
    if (!(stages & 2)) {
    } else if (counters != nullptr) {  // (the counting build: tests and the benchmark's untimed repeat)
        if (small)
            hipLaunchKernelGGL((chamfer_pruned_kernel<NQB, 8, true>), grid, dim3(64), 0, s, pa);
        else
            hipLaunchKernelGGL((chamfer_pruned_kernel<NQB, 32, true>), grid, dim3(64), 0, s, pa);
        hipLaunchKernelGGL(chamfer_count_flags_kernel, dim3(1), dim3(256), 0, s, sa.flags,
                           (int)(2 * B), counters);
    } else if (small) {
        hipLaunchKernelGGL((chamfer_pruned_kernel<NQB, 8>), grid, dim3(64), 0, s, pa);
    } else {
        hipLaunchKernelGGL((chamfer_pruned_kernel<NQB, 32>), grid, dim3(64), 0, s, pa);
    }
    const int rc = tk_launch_status();
    if (rc != TK3D_OK)
        return rc;
    if (!(stages & 4))
        return TK3D_OK;
    // whatever the waves above handed over (none on ordinary input: its workgroups leave
    // at once)
    if (channels_first)
        return chamfer_forward_mfma_flagged_launch<4, true>(xyz1, xyz2, B, N1, N2, dist1, idx1,
                                                            dist2, idx2, s, sa.flags);
    return chamfer_forward_mfma_flagged_launch<4>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2,
                                                  idx2, s, sa.flags);
}

template <typename T>
int chamfer_backward(const T *gd1, const T *gd2, const T *xyz1, const T *xyz2,
                     const int64_t *idx1, const int64_t *idx2, int64_t B, int64_t N1,
                     int64_t N2, T *gx1, T *gx2, void *stream)
{
    if (B < 0 || N1 < 0 || N2 < 0)
        return TK3D_ERR_BAD_SIZE;
    if (N1 > TK_MAX_I32 || N2 > TK_MAX_I32 || !tk_fits(TK_MAX_ELEMS, B, N1, 3) ||
        !tk_fits(TK_MAX_ELEMS, B, N2, 3))
        return TK3D_ERR_UNSUPPORTED;
    const int64_t t1 = B * N1, t2 = B * N2;
    if (t1 > 0 && (!gd1 || !xyz1 || !idx1 || !gx1))
        return TK3D_ERR_NULL_POINTER;
    if (t2 > 0 && (!gd2 || !xyz2 || !idx2 || !gx2))
        return TK3D_ERR_NULL_POINTER;
    if (t1 + t2 == 0)
        return TK3D_OK;
    hipStream_t s = (hipStream_t)stream;
    if constexpr (sizeof(T) == 4) {
        // Every range scans all senders of its batch, so ranges are as long as LDS
        // allows: 4096 points x 3 x (8 bytes of accumulator + 4 of the point) = 144 KiB.
        constexpr int R = 4096, NT = 1024;
        const int64_t r1 = (N1 + R - 1) / R, r2 = (N2 + R - 1) / R;
        // (the kernel addresses a cloud with 32-bit byte offsets: 12 bytes a point)
        if (B * (r1 + r2) <= TK_MAX_I32 && N1 <= (1 << 27) && N2 <= (1 << 27)) {
            constexpr auto kernel = chamfer_backward_fixed_kernel<R, NT>;
            constexpr size_t lds = (size_t)R * 3 * (sizeof(unsigned long long) + sizeof(float));
            const int allowed = tk_allow_dynamic_lds<kernel>((int)lds);
            if (allowed != TK3D_OK)
                return allowed;
            hipLaunchKernelGGL(kernel, dim3((unsigned)(B * (r1 + r2))), dim3(NT), lds, s, gd1,
                               gd2, xyz1, xyz2, idx1, idx2, (int)N1, (int)N2, (int)r1, (int)r2,
                               gx1, gx2);
            return tk_launch_status();
        }
    }
    int64_t blocks = (t1 + t2 + 255) / 256;
    if (blocks > 65536)
        blocks = 65536;
    hipLaunchKernelGGL((chamfer_backward_own_kernel<T>), dim3((unsigned)blocks), dim3(256),
                       0, s, gd1, gd2, xyz1, xyz2, idx1, idx2, t1, t2, (int)N1, (int)N2,
                       gx1, gx2);
    hipLaunchKernelGGL((chamfer_backward_scatter_kernel<T>), dim3((unsigned)blocks),
                       dim3(256), 0, s, gd1, gd2, xyz1, xyz2, idx1, idx2, t1, t2, (int)N1,
                       (int)N2, gx1, gx2);
    return tk_launch_status();
}

// ---- entry points for the tests and the benchmark (tk3d_debug.h) ----------------------

// One matrix instruction per tile on caller-supplied fp16 terms. Lane l supplies terms
// 8 (l / 32) .. + 7 of key l % 32 as the first operand and of query l % 32 as the second;
// in the result, register r of lane l is key 8 (r / 4) + 4 (l / 32) + r % 4, query l % 32.
__global__ __launch_bounds__(64) void debug_mfma_dot16_kernel(const uint4 *__restrict__ key_terms,
                                                              const uint4 *__restrict__ query_terms,
                                                              float *__restrict__ scores)
{
    const int lane = threadIdx.x, col = lane & 31, half = lane >> 5;
    const int64_t t = blockIdx.x;
    const uint4 ka = key_terms[(t * 32 + col) * 2 + half];
    const uint4 qb = query_terms[(t * 32 + col) * 2 + half];
    const tk_f32x16 zero = {};
    const tk_f32x16 acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(tk_f16x8, ka), __builtin_bit_cast(tk_f16x8, qb), zero, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 16; ++r)
        scores[(t * 32 + 8 * (r / 4) + 4 * half + r % 4) * 32 + col] = acc[r];
}

// The chamfer pre-filter's score for centred, scaled points, terms staged as the kernels do.
__global__ __launch_bounds__(64) void debug_chamfer_scores_kernel(const float *__restrict__ keys,
                                                                  const float *__restrict__ queries,
                                                                  float *__restrict__ scores)
{
    const int lane = threadIdx.x, col = lane & 31, half = lane >> 5;
    const int64_t t = blockIdx.x;
    const float *k = keys + (t * 32 + col) * 3, *q = queries + (t * 32 + col) * 3;
    const float nn = __builtin_fmaf(k[2], k[2], __builtin_fmaf(k[1], k[1], k[0] * k[0]));
    uint4 h0, h1;
    chamfer_key_terms(k[0], k[1], k[2], nn, true, h0, h1);
    const uint4 ka = half == 0 ? h0 : h1;
    const uint4 qb = chamfer_query_terms(q[0], q[1], q[2], half);
    const tk_f32x16 zero = {};
    const tk_f32x16 acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(tk_f16x8, ka), __builtin_bit_cast(tk_f16x8, qb), zero, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 16; ++r)
        scores[(t * 32 + 8 * (r / 4) + 4 * half + r % 4) * 32 + col] = acc[r];
}

int chamfer_forward_route(const float *xyz1, const float *xyz2, int64_t B, int64_t N1, int64_t N2,
                          float *dist1, int64_t *idx1, float *dist2, int64_t *idx2, int route,
                          hipStream_t s)
{
    if (B < 0 || N1 < 0 || N2 < 0)
        return TK3D_ERR_BAD_SIZE;
    if (N1 > TK_MAX_I32 / 4 || N2 > TK_MAX_I32 / 4 || !tk_fits(TK_MAX_ELEMS, B, N1, 3) ||
        !tk_fits(TK_MAX_ELEMS, B, N2, 3))
        return TK3D_ERR_UNSUPPORTED;
    if (B * N1 > 0 && (!xyz1 || !dist1 || !idx1))
        return TK3D_ERR_NULL_POINTER;
    if (B * N2 > 0 && (!xyz2 || !dist2 || !idx2))
        return TK3D_ERR_NULL_POINTER;
    const int64_t lo = N1 < N2 ? N1 : N2, hi = N1 < N2 ? N2 : N1;
    switch (route) {
    case TK3D_CHAMFER_ROUTE_EXACT:
        return chamfer_forward_launch<float, 4, 512, 64>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2,
                                                         idx2, s);
    case TK3D_CHAMFER_ROUTE_VECTOR:
        if (lo < 512)
            return TK3D_ERR_UNSUPPORTED;
        return chamfer_forward_filter_launch<4, 512, 64, 512>(xyz1, xyz2, B, N1, N2, dist1, idx1,
                                                              dist2, idx2, s);
    case TK3D_CHAMFER_ROUTE_MATRIX4:
    case TK3D_CHAMFER_ROUTE_MATRIX2:
    case TK3D_CHAMFER_ROUTE_MATRIX_SLICED: {
        if (lo < 1 || hi < 1024)
            return TK3D_ERR_UNSUPPORTED;
        if (route == TK3D_CHAMFER_ROUTE_MATRIX2)
            return chamfer_forward_mfma_launch<2>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2,
                                                  s);
        if (route == TK3D_CHAMFER_ROUTE_MATRIX4)
            return chamfer_forward_mfma_launch<4>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2,
                                                  s);
        const int64_t w0 = (N2 + 1023) / 1024, w1 = (N1 + 1023) / 1024;
        return chamfer_forward_mfma_launch<2>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, s,
                                              (int)(w0 > 256 ? 256 : w0), (int)(w1 > 256 ? 256 : w1));
    }
    default:
        return TK3D_ERR_UNSUPPORTED;
    }
}

}  // namespace

extern "C" {

int tk3d_chamfer_distance_forward_f32(const float *xyz1, const float *xyz2, int64_t B,
                                      int64_t N1, int64_t N2, float *dist1,
                                      int64_t *idx1, float *dist2, int64_t *idx2,
                                      void *stream)
{
    return chamfer_forward<float>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, stream);
}

size_t tk3d_chamfer_distance_forward_workspace_bytes(int64_t B, int64_t N1, int64_t N2,
                                                     int always)
{
    const bool wanted =
        always ? chamfer_sorted_can_serve(B, N1, N2) : chamfer_sorted_serves(B, N1, N2);
    return wanted ? chamfer_sorted_layout(B, N1, N2).total : 0;
}

int tk3d_chamfer_distance_forward_ws_f32(const float *xyz1, const float *xyz2, int64_t B,
                                         int64_t N1, int64_t N2, float *dist1, int64_t *idx1,
                                         float *dist2, int64_t *idx2, void *workspace,
                                         size_t workspace_bytes, void *stream)
{
    if (workspace == nullptr || !chamfer_sorted_can_serve(B, N1, N2) ||
        (reinterpret_cast<uintptr_t>(workspace) & 255) != 0 ||
        workspace_bytes < chamfer_sorted_layout(B, N1, N2).total)
        return chamfer_forward<float>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, stream);
    if (!xyz1 || !xyz2 || !dist1 || !idx1 || !dist2 || !idx2)
        return TK3D_ERR_NULL_POINTER;
    return chamfer_forward_sorted(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, workspace,
                                  (hipStream_t)stream);
}

int tk3d_chamfer_distance_forward_f64(const double *xyz1, const double *xyz2, int64_t B,
                                      int64_t N1, int64_t N2, double *dist1,
                                      int64_t *idx1, double *dist2, int64_t *idx2,
                                      void *stream)
{
    return chamfer_forward<double>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2,
                                   stream);
}

int tk3d_chamfer_distance_forward_bcn_f32(const float *xyz1, const float *xyz2, int64_t B,
                                          int64_t N1, int64_t N2, float *dist1, int64_t *idx1,
                                          float *dist2, int64_t *idx2, void *workspace,
                                          size_t workspace_bytes, void *stream)
{
    // the sorted path where it serves and a workspace was lent, else the sweep of all pairs
    if (workspace != nullptr && chamfer_sorted_can_serve(B, N1, N2) && N1 <= PREP_MAX_POINTS &&
        N2 <= PREP_MAX_POINTS && (reinterpret_cast<uintptr_t>(workspace) & 255) == 0 &&
        workspace_bytes >= chamfer_sorted_layout(B, N1, N2).total) {
        if (!xyz1 || !xyz2 || !dist1 || !idx1 || !dist2 || !idx2)
            return TK3D_ERR_NULL_POINTER;
        return chamfer_forward_sorted(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, workspace,
                                      (hipStream_t)stream, nullptr, 7, true);
    }
    return chamfer_forward<float, true>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, stream);
}

int tk3d_chamfer_distance_forward_bcn_f64(const double *xyz1, const double *xyz2, int64_t B,
                                          int64_t N1, int64_t N2, double *dist1, int64_t *idx1,
                                          double *dist2, int64_t *idx2, void *stream)
{
    return chamfer_forward<double, true>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, stream);
}

int tk3d_chamfer_distance_backward_f32(const float *grad_dist1, const float *grad_dist2,
                                       const float *xyz1, const float *xyz2,
                                       const int64_t *idx1, const int64_t *idx2,
                                       int64_t B, int64_t N1, int64_t N2,
                                       float *grad_xyz1, float *grad_xyz2, void *stream)
{
    return chamfer_backward<float>(grad_dist1, grad_dist2, xyz1, xyz2, idx1, idx2, B, N1,
                                   N2, grad_xyz1, grad_xyz2, stream);
}

int tk3d_chamfer_distance_backward_f64(const double *grad_dist1,
                                       const double *grad_dist2, const double *xyz1,
                                       const double *xyz2, const int64_t *idx1,
                                       const int64_t *idx2, int64_t B, int64_t N1,
                                       int64_t N2, double *grad_xyz1,
                                       double *grad_xyz2, void *stream)
{
    return chamfer_backward<double>(grad_dist1, grad_dist2, xyz1, xyz2, idx1, idx2, B, N1,
                                    N2, grad_xyz1, grad_xyz2, stream);
}

int tk3d_debug_chamfer_forward_route_f32(const float *xyz1, const float *xyz2, int64_t B,
                                         int64_t N1, int64_t N2, float *dist1, int64_t *idx1,
                                         float *dist2, int64_t *idx2, int route, void *stream)
{
    return chamfer_forward_route(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, route,
                                 (hipStream_t)stream);
}

int tk3d_debug_chamfer_forward_sorted_counted_f32(const float *xyz1, const float *xyz2,
                                                  int64_t B, int64_t N1, int64_t N2,
                                                  float *dist1, int64_t *idx1, float *dist2,
                                                  int64_t *idx2, void *workspace,
                                                  size_t workspace_bytes,
                                                  unsigned long long *counters, int stages,
                                                  void *stream)
{
    if (!workspace || !xyz1 || !xyz2 || !dist1 || !idx1 || !dist2 || !idx2)
        return TK3D_ERR_NULL_POINTER;
    if (!chamfer_sorted_can_serve(B, N1, N2))
        return TK3D_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0 ||
        workspace_bytes < chamfer_sorted_layout(B, N1, N2).total)
        return TK3D_ERR_WORKSPACE;
    return chamfer_forward_sorted(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, workspace,
                                  (hipStream_t)stream, counters, stages);
}

int tk3d_debug_mfma_dot16_f16(const uint16_t *key_terms, const uint16_t *query_terms, int64_t T,
                              float *scores, void *stream)
{
    if (T < 0 || T > TK_MAX_I32)
        return TK3D_ERR_BAD_SIZE;
    if (T == 0)
        return TK3D_OK;
    if (!key_terms || !query_terms || !scores)
        return TK3D_ERR_NULL_POINTER;
    if (((reinterpret_cast<uintptr_t>(key_terms) | reinterpret_cast<uintptr_t>(query_terms)) & 15) != 0)
        return TK3D_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(debug_mfma_dot16_kernel, dim3((unsigned)T), dim3(64), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint4 *>(key_terms),
                       reinterpret_cast<const uint4 *>(query_terms), scores);
    return tk_launch_status();
}

int tk3d_debug_chamfer_scores_f32(const float *keys, const float *queries, int64_t T,
                                  float *scores, void *stream)
{
    if (T < 0 || T > TK_MAX_I32)
        return TK3D_ERR_BAD_SIZE;
    if (T == 0)
        return TK3D_OK;
    if (!keys || !queries || !scores)
        return TK3D_ERR_NULL_POINTER;
    hipLaunchKernelGGL(debug_chamfer_scores_kernel, dim3((unsigned)T), dim3(64), 0,
                       (hipStream_t)stream, keys, queries, scores);
    return tk_launch_status();
}

}  // extern "C"

// Ball query for gfx950.
//
// A wave serves QW query points. The 64 lanes walk the key cloud together, UNROLL
// coalesced chunks of 64 keys at a time; for each query the lanes test their keys,
// a ballot turns the hits into a mask, and the popcount prefix of that mask gives
// every hit its output slot, so hits land in ascending key order exactly as the
// reference's serial scan records them (ball_query_kernel.cu:66-88). A wave stops
// as soon as all of its queries hold `k` neighbours - with typical radii that is a
// fraction of the cloud - whereas the reference always scans to the end.
// Remaining slots repeat the first hit; a query with no hit gets -1 everywhere
// (ball_query_kernel.cu:94-101, :123).
#include "tk3d_common.h"

namespace {

// SOA: clouds are [B,3,N] (coordinate planes) instead of [B,N,3].
template <typename T, int QW, int UNROLL, bool SOA>
__global__ __launch_bounds__(256) void ball_query_kernel(const T *__restrict__ query,
                                                         const T *__restrict__ key,
                                                         int64_t *__restrict__ index,
                                                         int64_t total_waves,
                                                         int waves_per_batch, int n1,
                                                         int n2, T r2, int k)
{
    const int lane = threadIdx.x & (TK_WAVE - 1);
    // readfirstlane tells the compiler that the wave index is uniform: the queries'
    // coordinates, hit counters and output rows then live in scalar registers and the
    // "query is full" tests are scalar branches.
    const int wave_in_block = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / TK_WAVE));
    const int64_t gw = (int64_t)blockIdx.x * (256 / TK_WAVE) + wave_in_block;
    if (gw >= total_waves)
        return;
    const int b = (int)(gw / waves_per_batch);
    const int q0 = (int)(gw - (int64_t)b * waves_per_batch) * QW;
    const T *__restrict__ Q = query + (int64_t)b * n1 * 3 + (SOA ? q0 : q0 * 3);
    const T *__restrict__ K = key + (int64_t)b * n2 * 3;
    const int qps = SOA ? 1 : 3, qcs = SOA ? n1 : 1;  // point / coordinate strides
    const int kps = SOA ? 1 : 3, kcs = SOA ? n2 : 1;
    int64_t *__restrict__ out = index + ((int64_t)b * n1 + q0) * k;

    T qx[QW], qy[QW], qz[QW];
    int cnt[QW], first[QW];
    int nq = n1 - q0;
    nq = nq < QW ? nq : QW;
#pragma unroll
    for (int q = 0; q < QW; ++q) {
        const bool ok = q < nq;
        qx[q] = ok ? Q[q * qps] : (T)0;
        qy[q] = ok ? Q[q * qps + qcs] : (T)0;
        qz[q] = ok ? Q[q * qps + 2 * qcs] : (T)0;
        cnt[q] = ok ? 0 : k;  // absent queries count as finished
        first[q] = -1;
    }

    for (int j0 = 0; j0 < n2; j0 += TK_WAVE * UNROLL) {
        T kx[UNROLL], ky[UNROLL], kz[UNROLL];
        if (j0 + TK_WAVE * UNROLL <= n2) {
            // full chunk: unconditional loads at constant offsets from one lane address
            const T *__restrict__ kl = K + (int64_t)(j0 + lane) * kps;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                kx[u] = kl[u * TK_WAVE * kps];
                ky[u] = kl[u * TK_WAVE * kps + kcs];
                kz[u] = kl[u * TK_WAVE * kps + 2 * kcs];
            }
        } else {
            // last chunk: keys that do not exist become NaN, which is never within reach
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int j = j0 + u * TK_WAVE + lane;
                const int jc = j < n2 ? j : n2 - 1;
                const T nan = (T)__builtin_nanf("");
                kx[u] = j < n2 ? K[(int64_t)jc * kps] : nan;
                ky[u] = K[(int64_t)jc * kps + kcs];
                kz[u] = K[(int64_t)jc * kps + 2 * kcs];
            }
        }
        bool all_done = true;
#pragma unroll
        for (int q = 0; q < QW; ++q) {
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (cnt[q] >= k)  // wave-uniform
                    continue;
                const int j = j0 + u * TK_WAVE + lane;
                const T d = tk_dist2<T>(kx[u], ky[u], kz[u], qx[q], qy[q], qz[q]);
                const bool hit = d < r2;  // false for the NaN of a key that does not exist
                const unsigned long long mask = __builtin_amdgcn_ballot_w64(hit);
                if (mask == 0)
                    continue;
                const int below = __builtin_amdgcn_mbcnt_hi(
                    (unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0));
                const int slot = cnt[q] + below;
                if (hit && slot < k)
                    out[(int64_t)q * k + slot] = (int64_t)j;
                if (cnt[q] == 0)
                    first[q] = j0 + u * TK_WAVE + __builtin_ctzll(mask);
                cnt[q] += __builtin_popcountll(mask);
            }
            all_done = all_done && (cnt[q] >= k);
        }
        if (all_done)
            break;
    }

#pragma unroll
    for (int q = 0; q < QW; ++q) {
        if (q >= nq)
            continue;
        for (int s = cnt[q] + lane; s < k; s += TK_WAVE)
            out[(int64_t)q * k + s] = (int64_t)first[q];
    }
}

template <typename T, int QW>
int ball_query_launch(const T *query, const T *key, bool channels_first, int64_t B, int64_t N1,
                      int64_t N2, T r2, int64_t k, int64_t *index, void *stream)
{
    constexpr int UNROLL = 8;  // 512 keys per trip
    const int64_t wpb = (N1 + QW - 1) / QW;
    const int64_t waves = B * wpb;
    const int64_t blocks = (waves + 3) / 4;
    if (blocks > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    if (channels_first)
        hipLaunchKernelGGL((ball_query_kernel<T, QW, UNROLL, true>), dim3((unsigned)blocks),
                           dim3(256), 0, (hipStream_t)stream, query, key, index, waves, (int)wpb,
                           (int)N1, (int)N2, r2, (int)k);
    else
        hipLaunchKernelGGL((ball_query_kernel<T, QW, UNROLL, false>), dim3((unsigned)blocks),
                           dim3(256), 0, (hipStream_t)stream, query, key, index, waves, (int)wpb,
                           (int)N1, (int)N2, r2, (int)k);
    return tk_launch_status();
}

template <typename T>
int ball_query(const T *query, const T *key, bool channels_first, int64_t B, int64_t N1,
               int64_t N2, float radius, int64_t k, int64_t *index, void *stream)
{
    if (B < 0 || N1 < 0 || N2 < 0)
        return TK3D_ERR_BAD_SIZE;
    if (k < 0)
        return TK3D_ERR_BAD_K;
    if (N1 > TK_MAX_I32 / 4 || N2 > TK_MAX_I32 / 4 || k > TK_MAX_I32 / 4 ||
        !tk_fits(TK_MAX_ELEMS, B, N1, k > 3 ? k : 3) || !tk_fits(TK_MAX_ELEMS, B, N2, 3))
        return TK3D_ERR_UNSUPPORTED;
    if (B * N1 * k == 0)
        return TK3D_OK;
    if (!query || !index || (N2 > 0 && !key))
        return TK3D_ERR_NULL_POINTER;
    // r2 = r*r in the data type, r being the float the caller passed
    // (ball_query.h:9, ball_query_kernel.cu:19,26).
    const T r = (T)radius;
    const T r2 = r * r;
    // Queries per wave: 4 share every key load when there are enough queries to fill the
    // GPU with waves anyway; fewer per wave otherwise.
    const int64_t total = B * N1;
    if (total >= 16384)
        return ball_query_launch<T, 4>(query, key, channels_first, B, N1, N2, r2, k, index,
                                       stream);
    if (total >= 4096)
        return ball_query_launch<T, 2>(query, key, channels_first, B, N1, N2, r2, k, index,
                                       stream);
    return ball_query_launch<T, 1>(query, key, channels_first, B, N1, N2, r2, k, index, stream);
}

}  // namespace

extern "C" {

int tk3d_ball_query_f32(const float *query, const float *key, int64_t B, int64_t N1,
                        int64_t N2, float radius, int64_t max_neighbors, int64_t *index,
                        void *stream)
{
    return ball_query<float>(query, key, false, B, N1, N2, radius, max_neighbors, index,
                             stream);
}

int tk3d_ball_query_f64(const double *query, const double *key, int64_t B, int64_t N1,
                        int64_t N2, float radius, int64_t max_neighbors, int64_t *index,
                        void *stream)
{
    return ball_query<double>(query, key, false, B, N1, N2, radius, max_neighbors, index,
                              stream);
}

int tk3d_ball_query_bcn_f32(const float *query, const float *key, int64_t B, int64_t N1,
                            int64_t N2, float radius, int64_t max_neighbors,
                            int64_t *index, void *stream)
{
    return ball_query<float>(query, key, true, B, N1, N2, radius, max_neighbors, index,
                             stream);
}

int tk3d_ball_query_bcn_f64(const double *query, const double *key, int64_t B, int64_t N1,
                            int64_t N2, float radius, int64_t max_neighbors,
                            int64_t *index, void *stream)
{
    return ball_query<double>(query, key, true, B, N1, N2, radius, max_neighbors, index,
                              stream);
}

}  // extern "C"

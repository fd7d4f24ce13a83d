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
#include "tk3d_common.h"

namespace {

constexpr int KNN_BLOCK = 256;
constexpr int KNN_STAGE = 1024;

template <typename T, int KMAX>
__global__ __launch_bounds__(KNN_BLOCK) void knn_register_kernel(
    const T *__restrict__ query, const T *__restrict__ key, T *__restrict__ distance,
    int64_t *__restrict__ index, int blocks_per_batch, int n1, int n2, int k)
{
    __shared__ T skey[KNN_STAGE * 4];
    const int tid = threadIdx.x;
    const int b = blockIdx.x / blocks_per_batch;
    const int qi = (blockIdx.x - b * blocks_per_batch) * KNN_BLOCK + tid;
    const bool active = qi < n1;
    const T *__restrict__ K = key + (int64_t)b * n2 * 3;
    T qx = 0, qy = 0, qz = 0;
    if (active) {
        const T *q = query + ((int64_t)b * n1 + qi) * 3;
        qx = q[0];
        qy = q[1];
        qz = q[2];
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
            const T d = tk_dist2<T>(K[s * 3 + 0], K[s * 3 + 1], K[s * 3 + 2], qx, qy, qz);
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
template <int KMAX>
__global__ __launch_bounds__(KNN_BLOCK) void knn_batched_kernel_f32(
    const float *__restrict__ query, const float *__restrict__ key,
    float *__restrict__ distance, int64_t *__restrict__ index, int blocks_per_batch, int n1,
    int n2, int k)
{
    constexpr int CHUNK = 32;
    __shared__ __align__(16) float skey[KNN_STAGE * 4];
    const int tid = threadIdx.x;
    const int b = blockIdx.x / blocks_per_batch;
    const int qi = (blockIdx.x - b * blocks_per_batch) * KNN_BLOCK + tid;
    const bool active = qi < n1;
    const float *__restrict__ K = key + (int64_t)b * n2 * 3;
    float qx = 0, qy = 0, qz = 0;
    if (active) {
        const float *q = query + ((int64_t)b * n1 + qi) * 3;
        qx = q[0];
        qy = q[1];
        qz = q[2];
    }

    float kd[KMAX];
    int ki[KMAX];
    float max_key = 0.0f;
    int max_idx = 0;
    // Fill phase: keys 0..k-1 go to slots 0..k-1 (mink.cuh:63-72); unused slots stay at
    // -inf so the rescan never selects them.
#pragma unroll
    for (int s = 0; s < KMAX; ++s) {
        kd[s] = -__builtin_huge_valf();
        ki[s] = 0;
        if (s < k) {  // uniform
            const float d = tk_dist2<float>(K[s * 3 + 0], K[s * 3 + 1], K[s * 3 + 2], qx, qy, qz);
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
            float4 e = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (kj < n2) {
                e.x = K[(int64_t)kj * 3 + 0];
                e.y = K[(int64_t)kj * 3 + 1];
                e.z = K[(int64_t)kj * 3 + 2];
            }
            reinterpret_cast<float4 *>(skey)[j] = e;
        }
        __syncthreads();
        const int left = n2 - stage0;
        const int cnt = left < KNN_STAGE ? left : KNN_STAGE;
        for (int c0 = 0; c0 < cnt; c0 += CHUNK) {
            // ---- sweep: bit (31 - i) of `mask` <=> key c0+i is below the maximum ----
            const int maxbits = __builtin_bit_cast(int, max_key);
            unsigned mask = 0u;
            const float4 *ck = reinterpret_cast<const float4 *>(skey) + c0;
#pragma unroll
            for (int i = 0; i < CHUNK; ++i) {
                const float4 e = ck[i];
                const float d = tk_dist2<float>(e.x, e.y, e.z, qx, qy, qz);
                const unsigned diff = (unsigned)(__builtin_bit_cast(int, d) - maxbits);
                mask = __builtin_amdgcn_alignbit(mask, diff, 31);  // (mask << 1) | (diff >> 31)
            }
            // Keys that do not exist, or that the fill phase already took, are no candidates.
            const int first = stage0 + c0;               // global index of bit 31
            int lo = k - first;                          // keys below k were used for filling
            lo = lo < 0 ? 0 : (lo > CHUNK ? CHUNK : lo);
            int hi = cnt - c0;                           // keys at or beyond hi are padding
            hi = hi > CHUNK ? CHUNK : hi;
            unsigned valid = (lo >= CHUNK) ? 0u : (0xffffffffu >> lo);
            valid &= (hi >= CHUNK) ? 0xffffffffu : ~(0xffffffffu >> hi);
            mask &= valid;

            // ---- insertion rounds ----
            while (__builtin_amdgcn_ballot_w64(mask != 0u)) {  // wave-uniform
                const bool has = mask != 0u;
                const int i = has ? __builtin_clz(mask) : 0;
                mask &= ~(0x80000000u >> i);
                const float4 e = ck[i];
                const float d = tk_dist2<float>(e.x, e.y, e.z, qx, qy, qz);
                if (has && d < max_key) {
                    const int kj = first + i;
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
    }
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

template <typename T, int KMAX>
void knn_launch(const T *query, const T *key, T *distance, int64_t *index, int64_t B,
                int bpb, int n1, int n2, int k, hipStream_t s)
{
    if constexpr (sizeof(T) == 4)
        hipLaunchKernelGGL((knn_batched_kernel_f32<KMAX>), dim3((unsigned)(B * bpb)),
                           dim3(KNN_BLOCK), 0, s, query, key, distance, index, bpb, n1, n2, k);
    else
        hipLaunchKernelGGL((knn_register_kernel<T, KMAX>), dim3((unsigned)(B * bpb)),
                           dim3(KNN_BLOCK), 0, s, query, key, distance, index, bpb, n1, n2, k);
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
    if (k <= 4)
        knn_launch<T, 4>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
    else if (k <= 8)
        knn_launch<T, 8>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
    else if (k <= 16)
        knn_launch<T, 16>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
    else if (k <= 32)
        knn_launch<T, 32>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
    else if (k <= 64)
        knn_launch<T, 64>(query, key, distance, index, B, (int)bpb, n1, n2, kk, s);
    else
        hipLaunchKernelGGL((knn_global_kernel<T>), dim3((unsigned)(B * bpb)), dim3(KNN_BLOCK),
                           0, s, query, key, distance, index, (int)bpb, n1, n2, kk);
    return tk_launch_status();
}

}  // namespace

extern "C" {

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

}  // extern "C"

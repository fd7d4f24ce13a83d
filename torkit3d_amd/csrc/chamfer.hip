// Chamfer / nearest-neighbour distance for gfx950: forward (all-pairs minimum with
// argmin) and backward (closed-form gradient).
//
// Forward design
// --------------
// One workgroup owns QPL*BLOCK query points of one cloud and sweeps the whole
// opposite cloud. Key points are staged through LDS as (x,y,z,pad) quads; every
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

namespace {

template <typename T> struct ChamferDir {
    const T *query;   // [B, nq, 3]
    const T *key;     // [B, nk, 3]
    T *dist;          // [B, nq]
    int64_t *idx;     // [B, nq]
    int nq;
    int nk;
    int blocks_per_batch;
};

template <typename T> struct ChamferFwdArgs {
    ChamferDir<T> dir[2];
    int nblocks0;  // workgroups of direction 0; the rest belong to direction 1
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

template <typename T, int QPL, int BLOCK, int TILE, int STAGE>
__global__ __launch_bounds__(BLOCK) void chamfer_forward_kernel(ChamferFwdArgs<T> args)
{
    static_assert(STAGE % TILE == 0 && TILE % 2 == 0, "tile shapes");
    __shared__ T skey[STAGE * 4];

    const int tid = threadIdx.x;
    // Workgroups are handed to the 8 XCDs round-robin by blockIdx. Remap so that each
    // XCD works on a contiguous range of logical workgroups: the workgroups that
    // sweep the same key cloud then share one L2 instead of fetching it 8 times.
    int lb = blockIdx.x;
    {
        const int nb = gridDim.x, per = nb >> 3, full = per << 3;
        if (lb < full)
            lb = (lb & 7) * per + (lb >> 3);
    }
    const int which = lb >= args.nblocks0;
    if (which)
        lb -= args.nblocks0;
    const ChamferDir<T> &d = args.dir[which];
    const int nq = d.nq, nk = d.nk;
    const int b = lb / d.blocks_per_batch;
    const int qblock = lb - b * d.blocks_per_batch;
    const T *__restrict__ Q = d.query + (int64_t)b * nq * 3;
    const T *__restrict__ K = d.key + (int64_t)b * nk * 3;

    T qx[QPL], qy[QPL], qz[QPL], best[QPL];
    int btile[QPL];
#pragma unroll
    for (int i = 0; i < QPL; ++i) {
        const int qi = (qblock * QPL + i) * BLOCK + tid;
        const bool ok = qi < nq;
        qx[i] = ok ? Q[(int64_t)qi * 3 + 0] : (T)0;
        qy[i] = ok ? Q[(int64_t)qi * 3 + 1] : (T)0;
        qz[i] = ok ? Q[(int64_t)qi * 3 + 2] : (T)0;
        best[i] = chamfer_init_min<T>();
        btile[i] = -1;
    }

    for (int stage0 = 0; stage0 < nk; stage0 += STAGE) {
        __syncthreads();
        for (int j = tid; j < STAGE; j += BLOCK) {
            const int kj = stage0 + j;
            T x = tk_inf<T>(), y = tk_inf<T>(), z = tk_inf<T>();
            if (kj < nk) {
                x = K[(int64_t)kj * 3 + 0];
                y = K[(int64_t)kj * 3 + 1];
                z = K[(int64_t)kj * 3 + 2];
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
#pragma unroll
            for (int j = 0; j < TILE; j += 2) {
                const T ax = tk[j * 4 + 0], ay = tk[j * 4 + 1], az = tk[j * 4 + 2];
                const T bx = tk[j * 4 + 4], by = tk[j * 4 + 5], bz = tk[j * 4 + 6];
#pragma unroll
                for (int i = 0; i < QPL; ++i) {
                    const T da = tk_dist2<T>(ax, ay, az, qx[i], qy[i], qz[i]);
                    const T db = tk_dist2<T>(bx, by, bz, qx[i], qy[i], qz[i]);
                    tmin[i] = tk_min<T>(tk_min<T>(tmin[i], da), db);
                }
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
                const T kx = K[(int64_t)j * 3 + 0];
                const T ky = K[(int64_t)j * 3 + 1];
                const T kz = K[(int64_t)j * 3 + 2];
                const T dd = tk_dist2<T>(kx, ky, kz, qx[i], qy[i], qz[i]);
                found = (dd == best[i]) ? j : found;
            }
        }
        d.dist[(int64_t)b * nq + qi] = best[i];
        d.idx[(int64_t)b * nq + qi] = (int64_t)found;
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

template <typename T, int QPL, int BLOCK = 256, int TILE = 32, int STAGE = 1024>
int chamfer_forward_launch(const T *xyz1, const T *xyz2, int64_t B, int64_t N1,
                           int64_t N2, T *dist1, int64_t *idx1, T *dist2,
                           int64_t *idx2, hipStream_t stream)
{
    constexpr int QB = QPL * BLOCK;
    ChamferFwdArgs<T> a;
    a.dir[0] = {xyz1, xyz2, dist1, idx1, (int)N1, (int)N2, (int)((N1 + QB - 1) / QB)};
    a.dir[1] = {xyz2, xyz1, dist2, idx2, (int)N2, (int)N1, (int)((N2 + QB - 1) / QB)};
    const int64_t nb0 = B * a.dir[0].blocks_per_batch;
    const int64_t nb1 = B * a.dir[1].blocks_per_batch;
    if (nb0 + nb1 == 0)
        return TK3D_OK;
    if (nb0 + nb1 > TK_MAX_I32)
        return TK3D_ERR_UNSUPPORTED;
    a.nblocks0 = (int)nb0;
    hipLaunchKernelGGL((chamfer_forward_kernel<T, QPL, BLOCK, TILE, STAGE>),
                       dim3((unsigned)(nb0 + nb1)), dim3(BLOCK), 0, stream, a);
    return tk_launch_status();
}

template <typename T>
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
    if (sizeof(T) == 8 || work < (int64_t)256 * 1024)
        return chamfer_forward_launch<T, 2>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2,
                                            idx2, s);
    return chamfer_forward_launch<T, 4, 512, 64>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2,
                                                 idx2, s);
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

}  // namespace

extern "C" {

int tk3d_chamfer_distance_forward_f32(const float *xyz1, const float *xyz2, int64_t B,
                                      int64_t N1, int64_t N2, float *dist1,
                                      int64_t *idx1, float *dist2, int64_t *idx2,
                                      void *stream)
{
    return chamfer_forward<float>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2, stream);
}

int tk3d_chamfer_distance_forward_f64(const double *xyz1, const double *xyz2, int64_t B,
                                      int64_t N1, int64_t N2, double *dist1,
                                      int64_t *idx1, double *dist2, int64_t *idx2,
                                      void *stream)
{
    return chamfer_forward<double>(xyz1, xyz2, B, N1, N2, dist1, idx1, dist2, idx2,
                                   stream);
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

}  // extern "C"

// Farthest point sampling for gfx950.
//
// Clouds that fit in one workgroup's registers (16384 points in fp32, 8192 in fp64) are
// sampled by one workgroup each; larger ones by one launch of many workgroups per
// selection step (fps_wide_step_kernel, further down). The K-1 selection steps are
// strictly serial, so the one-workgroup kernels are built for latency per step, not
// throughput:
//   * every lane keeps P points and their running minimum distance in registers
//     for the whole kernel - the loop touches no global memory except the one
//     index it emits per step;
//   * per step a lane updates its P minima and finds its local maximum, the wave
//     reduces with DPP row shifts / row broadcasts (no LDS), ballot + find-first
//     pick the winning lane on the scalar unit;
//   * waves exchange (value, point index, xyz) through double-buffered LDS slots,
//     so a step costs a single s_barrier, and every wave redoes the tiny
//     cross-wave reduction itself instead of waiting for a broadcast.
//
// Ties. The reference resolves equal maxima by its thread layout: thread t scans
// j = t, t+BS, ... keeping the first maximum, then a shared-memory tree keeps the
// left operand (sample_farthest_points_kernel.cu:46-72, :75-95), i.e. the winner
// is the candidate with the smallest (bit-reversed t, j / BS). The points are
// laid out here in exactly that priority order ("positions"), lanes take
// consecutive positions, and every reduction keeps the lowest position among
// equal values, which reproduces the reference's choice.
#include "tk3d_common.h"

namespace {

template <typename T> struct Bits;
template <> struct Bits<float> { using type = int; };
template <> struct Bits<double> { using type = long long; };

template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_move(float v)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v),
                                           __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF,
                                           false));
}
template <int CTRL, int ROW_MASK> __device__ __forceinline__ double dpp_move(double v)
{
    const long long b = __builtin_bit_cast(long long, v);
    int lo = (int)b, hi = (int)(b >> 32);
    lo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xF, false);
    hi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xF, false);
    return __builtin_bit_cast(double,
                              ((long long)hi << 32) | (long long)(unsigned)lo);
}

__device__ __forceinline__ float read_lane(float v, int lane)
{
    return __builtin_bit_cast(float,
                              __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ int read_lane(int v, int lane)
{
    return __builtin_amdgcn_readlane(v, lane);
}
__device__ __forceinline__ double read_lane(double v, int lane)
{
    const long long b = __builtin_bit_cast(long long, v);
    const int lo = __builtin_amdgcn_readlane((int)b, lane);
    const int hi = __builtin_amdgcn_readlane((int)(b >> 32), lane);
    return __builtin_bit_cast(double, ((long long)hi << 32) | (long long)(unsigned)lo);
}

// Maximum over the 64 lanes, returned as a wave-uniform value. Inclusive scan
// inside each row of 16 (row_shr 1,2,4,8), then row_bcast15 / row_bcast31 carry
// the row totals up so that lane 63 holds the result.
template <typename T> __device__ __forceinline__ T wave_max(T v)
{
    v = tk_max<T>(v, dpp_move<0x111, 0xF>(v));
    v = tk_max<T>(v, dpp_move<0x112, 0xF>(v));
    v = tk_max<T>(v, dpp_move<0x114, 0xF>(v));
    v = tk_max<T>(v, dpp_move<0x118, 0xF>(v));
    v = tk_max<T>(v, dpp_move<0x142, 0xA>(v));
    v = tk_max<T>(v, dpp_move<0x143, 0xC>(v));
    return read_lane(v, 63);
}

// Coordinate `a` of point `j`: clouds are [n,3] rows, or with SOA three planes [3,n]
// (the layout the reference's models keep their clouds in).
template <bool SOA, typename T>
__device__ __forceinline__ T fps_coord(const T *__restrict__ pts, int n, int64_t j, int a)
{
    return SOA ? pts[(int64_t)a * n + j] : pts[j * 3 + a];
}

struct FpsLayout {
    int n;        // points per cloud
    int k;        // samples per cloud
    int bs;       // the reference's block size for this n (power of two, 32..512)
    int log2_bs;
    int c;        // ceil(n / bs): points per reference thread
    float inv_c;  // 1 / c
};

// Point index of a position in the priority order described at the top.
__device__ __forceinline__ int fps_point_of_position(int pos, const FpsLayout &L)
{
    int r = (int)(((float)pos + 0.5f) * L.inv_c);
    // One correction step makes the float estimate exact for every pos < 2^24.
    r += ((r + 1) * L.c <= pos) ? 1 : 0;
    r -= (r * L.c > pos) ? 1 : 0;
    const int cc = pos - r * L.c;
    const int t = (int)(__builtin_bitreverse32((unsigned)r) >> (32 - L.log2_bs));
    return t + cc * L.bs;
}

// One selection step per exchange between the waves, on points and minima held in
// registers (lane `tid` holds positions tid * P .. tid * P + P - 1). fmin keeps a
// minimum when a later distance is NaN, as the reference's '>' does. `md` arrives
// holding the distances to point 0 (see fps_first_minimum).
template <typename T, int P, int NT>
__device__ __forceinline__ void fps_one_step_loop(int64_t *__restrict__ out, const FpsLayout &L,
                                                  const T (&x)[P], const T (&y)[P],
                                                  const T (&z)[P], T (&md)[P], T cx, T cy, T cz)
{
    constexpr int NW = NT / TK_WAVE;
    __shared__ T s_val[2][NW], s_x[2][NW], s_y[2][NW], s_z[2][NW];
    __shared__ int s_j[2][NW];
    const int tid = threadIdx.x;
    const int lane = tid & (TK_WAVE - 1);
    const int wave = tid / TK_WAVE;
    int sel_j = 0;
    if (tid == 0)
        out[0] = 0;

    for (int it = 1; it < L.k; ++it) {
        // Lane-local update and first maximum above zero (strict '>' from zero, as
        // the reference thread does).
        T best = (T)0;
        int bp = 0;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const T d = tk_dist2<T>(x[p], y[p], z[p], cx, cy, cz);
            md[p] = tk_min<T>(md[p], d);
            const bool up = md[p] > best;
            best = up ? md[p] : best;
            bp = up ? p : bp;
        }
        const T wmax = wave_max<T>(best);
        const unsigned long long hit = __builtin_amdgcn_ballot_w64(best == wmax);
        const int wl = __builtin_ctzll(hit);  // lowest lane holding the maximum
        const int wp = read_lane(bp, wl);
        T sx = x[0], sy = y[0], sz = z[0];
#pragma unroll
        for (int p = 1; p < P; ++p) {
            if (wp == p) {  // wave-uniform: a scalar branch
                sx = x[p];
                sy = y[p];
                sz = z[p];
            }
        }
        // Cross-lane reads happen with the whole wave active: a lane switched off
        // by a branch has no defined value to hand over.
        const T wx = read_lane(sx, wl), wy = read_lane(sy, wl), wz = read_lane(sz, wl);
        const int wj = fps_point_of_position((wave * TK_WAVE + wl) * P + wp, L);
        const int buf = it & 1;
        if (lane == 0) {
            s_val[buf][wave] = wmax;
            s_j[buf][wave] = wj;
            s_x[buf][wave] = wx;
            s_y[buf][wave] = wy;
            s_z[buf][wave] = wz;
        }
        __syncthreads();
        // Every wave reduces the NW candidates itself. Lower waves hold lower
        // positions, so the lowest lane among equal values is the right winner.
        const bool has = lane < NW;
        const T cv = has ? s_val[buf][has ? lane : 0] : (T)-1;
        const T gmax = wave_max<T>(cv);
        if (gmax > (T)0) {
            const int gl = __builtin_ctzll(__builtin_amdgcn_ballot_w64(cv == gmax));
            sel_j = s_j[buf][gl];
            cx = s_x[buf][gl];
            cy = s_y[buf][gl];
            cz = s_z[buf][gl];
        }
        // gmax == 0: no point lies away from the chosen set; the previous choice
        // is emitted again, as the reference does.
        if (tid == 0)
            out[it] = (int64_t)sel_j;
    }
}

// The reference's minima start "unset" and take whatever the first step computes
// (sample_farthest_points_kernel.cu:59-64), a NaN included, which then never compares
// above anything. So a minimum starts at the distance to point 0, with -1 for a NaN and
// for unused slots: min() keeps -1 and it never exceeds 0.
template <typename T> __device__ __forceinline__ T fps_first_minimum(bool used, T d0)
{
    return (used && d0 == d0) ? d0 : (T)-1;
}

// The whole sampling of one cloud with the plain loop: loads the points into registers
// and runs fps_one_step_loop. With `only_odd` it does so only for a cloud that holds a NaN
// or an infinite coordinate, and returns at once for any other.
//
// The fp32 kernel below assumes finite coordinates (minima ordered as integers, a selected
// point's minimum dropping to zero) and is followed by this one with `only_odd`, which
// redoes the rare cloud it got wrong the way the reference treats it: a NaN point is never
// selected, an infinite one, once selected, is selected at every later step. The check
// lives here rather than in that kernel because anything added to it, even a test in
// its prologue, moved its loop's code and cost 4-7 % at 32 points per lane; the extra
// launch costs a few microseconds.
template <typename T, int P, int NT, bool SOA>
__global__ __launch_bounds__(NT) void fps_register_kernel(const T *__restrict__ points,
                                                          int64_t *__restrict__ index,
                                                          FpsLayout L, int only_odd)
{
    const T *__restrict__ pts = points + (int64_t)blockIdx.x * L.n * 3;
    int64_t *__restrict__ out = index + (int64_t)blockIdx.x * L.k;
    const int tid = threadIdx.x;
    if (only_odd) {
        // v - v is zero exactly for finite v; the 3n values are scanned in memory order
        bool odd = false;
#pragma unroll 8
        for (int i = tid; i < L.n * 3; i += NT) {
            const T v = pts[i];
            odd |= !(v - v == (T)0);
        }
        if (!__syncthreads_or(odd ? 1 : 0))  // uniform over the workgroup
            return;
    }
    T x[P], y[P], z[P], md[P];
    const int npos = L.bs * L.c;
    const T cx = fps_coord<SOA>(pts, L.n, 0, 0), cy = fps_coord<SOA>(pts, L.n, 0, 1),
            cz = fps_coord<SOA>(pts, L.n, 0, 2);
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int pos = tid * P + p;
        const int j = pos < npos ? fps_point_of_position(pos, L) : L.n;
        const bool ok = j < L.n;
        x[p] = ok ? fps_coord<SOA>(pts, L.n, j, 0) : (T)0;
        y[p] = ok ? fps_coord<SOA>(pts, L.n, j, 1) : (T)0;
        z[p] = ok ? fps_coord<SOA>(pts, L.n, j, 2) : (T)0;
        md[p] = fps_first_minimum<T>(ok, tk_dist2<T>(x[p], y[p], z[p], cx, cy, cz));
    }
    fps_one_step_loop<T, P, NT>(out, L, x, y, z, md, cx, cy, cz);
}

// ---- fp32 fast path ------------------------------------------------------------
// Same algorithm as fps_register_kernel, tuned for the serial step:
//   * running minima are kept as the bit patterns of non-negative floats, which
//     order like signed integers; integer min/max need no NaN canonicalisation
//     and the -1.0f marker of unused slots (a negative integer) stays put;
//   * a lane reduces its P minima through a binary tree of maxima kept in
//     registers; the wave's maximum is a scan with DPP row shifts and broadcasts, and
//     the runner-up (the largest value of the other lanes) a second such scan that runs
//     beside the walk below;
//   * the winning lane comes from one ballot + scalar find-first; its winning
//     point is found by walking the winner lane's tree with v_readlane and
//     scalar branches (left child first = lowest position), and the leaf reached
//     reads that point's coordinates from fixed registers - log2(P) steps, no
//     per-point compares or select chains in the loop;
//   * a wave publishes its candidate (xyz, value) and (runner-up, point) in LDS; after the
//     single barrier every wave loads all candidates and decides by itself how many of
//     them are winners (see fps_multistep_kernel_f32).

struct FpsPick {
    float x, y, z;
    int j;
};

// Largest of the 64 lanes' values (all >= 0), wave-uniform: a scan along rows of 16 lanes
// with row shifts, the rows' results carried on with row broadcasts, the total read from
// lane 63. A lane without a source lane in a step takes 0.
__device__ __forceinline__ int wave_max_i32(int v)
{
#define TK3D_MAX_STEP(ctrl, rows)                                                      \
    {                                                                                  \
        const int o = __builtin_amdgcn_update_dpp(0, v, ctrl, rows, 0xf, false);       \
        v = o > v ? o : v;                                                             \
    }
    TK3D_MAX_STEP(0x111, 0xf)  // row_shr:1
    TK3D_MAX_STEP(0x112, 0xf)  // row_shr:2
    TK3D_MAX_STEP(0x114, 0xf)  // row_shr:4
    TK3D_MAX_STEP(0x118, 0xf)  // row_shr:8
    TK3D_MAX_STEP(0x142, 0xa)  // row_bcast:15 into rows 1 and 3
    TK3D_MAX_STEP(0x143, 0xc)  // row_bcast:31 into rows 2 and 3
#undef TK3D_MAX_STEP
    return __builtin_amdgcn_readlane(v, 63);
}

// FpsWalk that also reports the largest value it passed by: the walk from the root to
// the first leaf equal to `wmax` sees the sibling of every node on its path, and the
// largest of those siblings is the lane's second-largest minimum (equal to `wmax` when
// the lane holds the maximum twice).
template <int P, int NODE> struct FpsWalk2 {
    static __device__ __forceinline__ void go(const int (&t)[2 * P], const float (&x)[P],
                                              const float (&y)[P], const float (&z)[P],
                                              const int (&jv)[P], int wl, int wmax,
                                              FpsPick &out, int &passed)
    {
        if constexpr (NODE >= P) {
            constexpr int p = NODE - P;
            out.x = read_lane(x[p], wl);
            out.y = read_lane(y[p], wl);
            out.z = read_lane(z[p], wl);
            out.j = read_lane(jv[p], wl);
            asm volatile("" ::"s"(out.j));
        } else {
            const int left = read_lane(t[2 * NODE], wl);
            const int right = read_lane(t[2 * NODE + 1], wl);
            if (left == wmax) {
                passed = right > passed ? right : passed;
                FpsWalk2<P, 2 * NODE>::go(t, x, y, z, jv, wl, wmax, out, passed);
            } else {
                passed = left > passed ? left : passed;
                FpsWalk2<P, 2 * NODE + 1>::go(t, x, y, z, jv, wl, wmax, out, passed);
            }
        }
    }
};

// FpsWalk2 for a caller that keeps the point indices elsewhere: reports the leaf reached.
template <int P, int NODE> struct FpsWalk3 {
    static __device__ __forceinline__ void go(const int (&t)[2 * P], const float (&x)[P],
                                              const float (&y)[P], const float (&z)[P], int wl,
                                              int wmax, FpsPick &out, int &passed)
    {
        if constexpr (NODE >= P) {
            constexpr int p = NODE - P;
            out.x = read_lane(x[p], wl);
            out.y = read_lane(y[p], wl);
            out.z = read_lane(z[p], wl);
            out.j = p;  // the leaf; the caller turns it into a point index
        } else {
            const int left = read_lane(t[2 * NODE], wl);
            const int right = read_lane(t[2 * NODE + 1], wl);
            if (left == wmax) {
                passed = right > passed ? right : passed;
                FpsWalk3<P, 2 * NODE>::go(t, x, y, z, wl, wmax, out, passed);
            } else {
                passed = left > passed ? left : passed;
                FpsWalk3<P, 2 * NODE + 1>::go(t, x, y, z, wl, wmax, out, passed);
            }
        }
    }
};

// fp32 kernel that takes up to MAXM selection steps per cross-wave exchange.
//
// A step's fixed cost (wave reduction, slot exchange, barrier: about 1000 clocks) is
// several times the cost of updating the minima for one more centre, so after the
// exchange every wave checks, redundantly, whether the next winners are already known.
// Let the waves' candidates be sorted by (value descending, wave ascending) - waves
// hold ascending position ranges, so this is the reference's order - and let w1 be the
// winner. The m-th candidate w_m (value V_m > 0) is the winner of the m-th following
// step exactly when
//   * no wave that already supplied a winner holds another point at or above V_m (each
//     wave publishes its second-largest minimum for this; ties are refused), and
//   * the canonical distance from w_m to every winner accepted so far is >= V_m, so the
//     coming updates leave its minimum at V_m;
// every other point is at or below V_m by the sort, minima only shrink, and the
// accepted winners drop to zero. The chain stops at the first candidate that fails;
// on uniform clouds about 2.7 steps are taken per exchange.
//
// The check is a chain of dependent instructions issued by one wave, so its length in
// instructions is its cost: conditions are single compares whose lane masks are combined
// in scalar registers, and the accepted candidates never go back to LDS - the coming
// update reads their coordinates with v_readlane from the lanes that already hold them.
template <int P, int NT, bool SOA, int MAXM, bool GATED = false>
__global__ __launch_bounds__(NT) void fps_multistep_kernel_f32(const float *__restrict__ points,
                                                               int64_t *__restrict__ index,
                                                               FpsLayout L)
{
    static_assert((P & (P - 1)) == 0, "P must be a power of two");
    if constexpr (GATED) {  // only the clouds the region kernel left (see its ORDER_PROBE)
        if (index[(int64_t)blockIdx.x * L.k + L.k - 1] != -1)  // uniform over the workgroup
            return;
    }
    constexpr int NW = NT / TK_WAVE;
    static_assert(NW <= 8, "the cross-wave step relates 8 x 8 candidates");
    constexpr int F32_INF = 0x7f800000;
    constexpr int F32_NEG1 = (int)0xbf800000;
    __shared__ float4 s_cand[2][8];  // a wave's candidate: x, y, z, running minimum (bits)
    __shared__ int2 s_aux[2][8];     // the wave's second-largest minimum, the candidate's index

    const int tid = threadIdx.x;
    const int lane = tid & (TK_WAVE - 1);
    const int wave = tid / TK_WAVE;
    const float *__restrict__ pts = points + (int64_t)blockIdx.x * L.n * 3;
    int64_t *__restrict__ out = index + (int64_t)blockIdx.x * L.k;

    float x[P], y[P], z[P];
    int jv[P];
    int t[2 * P];  // t[P + p]: running minimum of point p (bits); t[1..P-1]: maxima
    const int npos = L.bs * L.c;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int pos = tid * P + p;
        const int j = pos < npos ? fps_point_of_position(pos, L) : L.n;
        const bool ok = j < L.n;
        x[p] = ok ? fps_coord<SOA>(pts, L.n, j, 0) : 0.0f;
        y[p] = ok ? fps_coord<SOA>(pts, L.n, j, 1) : 0.0f;
        z[p] = ok ? fps_coord<SOA>(pts, L.n, j, 2) : 0.0f;
        jv[p] = j;
        t[P + p] = ok ? F32_INF : F32_NEG1;
    }
    t[0] = 0;

    // Lane (a, b) = (lane / 8, lane % 8) relates candidate a to candidate b after an
    // exchange. The centres of the coming update are the candidates of the lanes in
    // `centres` (lane 8 a stands for candidate a); the first update is point 0.
    const int ca = lane >> 3, cb = lane & 7;
    float ax = fps_coord<SOA>(pts, L.n, 0, 0);
    float ay = fps_coord<SOA>(pts, L.n, 0, 1);
    float az = fps_coord<SOA>(pts, L.n, 0, 2);
    unsigned long long centres = 1ull;
    // the last point emitted is the candidate of lane ctz(last_mask) / 8, whose index that
    // lane keeps in last_j; no mask: point 0
    unsigned long long last_mask = 0ull;
    int last_j = 0;
    constexpr unsigned long long FIRST_OF_EIGHT = 0x0101010101010101ull;  // lanes b == 0
    constexpr unsigned long long EARLIER = 0x7f3f1f0f07030100ull;         // lanes b < a
    int nc = 1;
    if (tid == 0)
        out[0] = 0;
    if (tid < 16 && (tid & 7) >= NW) {  // waves that do not exist never have a candidate
        s_cand[tid >> 3][tid & 7] = make_float4(0.0f, 0.0f, 0.0f, -1.0f);
        s_aux[tid >> 3][tid & 7] = make_int2(0, 0);
    }

    int round = 0;
    for (int it = 1; it < L.k; it += nc, ++round) {
        for (unsigned long long todo = centres; todo != 0ull; todo &= todo - 1) {  // uniform
            const int l = __builtin_ctzll(todo);
            const float sx = read_lane(ax, l), sy = read_lane(ay, l), sz = read_lane(az, l);
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const float d = tk_dist2<float>(x[p], y[p], z[p], sx, sy, sz);
                const int db = __builtin_bit_cast(int, d);
                t[P + p] = t[P + p] < db ? t[P + p] : db;
            }
        }
#pragma unroll
        for (int i = P - 1; i >= 1; --i)
            t[i] = t[2 * i] > t[2 * i + 1] ? t[2 * i] : t[2 * i + 1];
        // Only points strictly above zero are candidates (the reference starts its
        // scan from max_dist = 0 with strict '>').
        const int best = t[1] > 0 ? t[1] : 0;
        const int wmax = wave_max_i32(best);
        const int wl = __builtin_ctzll(__builtin_amdgcn_ballot_w64(best == wmax));
        int second = wave_max_i32(lane == wl ? 0 : best);  // over the other lanes
        FpsPick pick;
        FpsWalk2<P, 1>::go(t, x, y, z, jv, wl, wmax, pick, second);  // and inside lane wl
        const int buf = round & 1;
        if (lane == 0) {
            s_cand[buf][wave] = make_float4(pick.x, pick.y, pick.z, __builtin_bit_cast(float, wmax));
            s_aux[buf][wave] = make_int2(second, pick.j);
        }
        __syncthreads();
        // Every wave now works out, redundantly and without a serial chain, how many of
        // the candidates are certain winners of the coming steps. All 64 lanes are active,
        // so conditions are combined as lane masks in scalar registers.
        const float4 A = s_cand[buf][ca], Bc = s_cand[buf][cb];
        const int2 Bx = s_aux[buf][cb];  // the wave's second-largest minimum, its point
        ax = A.x;
        ay = A.y;
        az = A.z;
        const int va = __builtin_bit_cast(int, A.w), vb = __builtin_bit_cast(int, Bc.w);
        // b comes before a in the reference's order: larger value, then lower position
        // (waves hold ascending ranges of positions)
        const unsigned long long m_before =
            __builtin_amdgcn_ballot_w64(vb > va) | (__builtin_amdgcn_ballot_w64(vb == va) & EARLIER);
        const unsigned long long m_live = __builtin_amdgcn_ballot_w64(va > 0);
        const float dab = tk_dist2<float>(A.x, A.y, A.z, Bc.x, Bc.y, Bc.z);
        // a survives b's selection: b's update leaves a's minimum alone, and b's wave
        // holds nothing else at or above it
        const unsigned long long m_far =
            __builtin_amdgcn_ballot_w64(__builtin_bit_cast(int, dab) >= va);
        const unsigned long long m_alone = __builtin_amdgcn_ballot_w64(Bx.x < va);
        const unsigned long long m_fine = ~m_before | (m_far & m_alone);
        // byte a of a mask: candidate a against every b
        const unsigned before_a =
            __builtin_amdgcn_ubfe(lane < 32 ? (unsigned)m_before : (unsigned)(m_before >> 32),
                                  (unsigned)(lane & 24), 8u);
        const unsigned fine_a =
            __builtin_amdgcn_ubfe(lane < 32 ? (unsigned)m_fine : (unsigned)(m_fine >> 32),
                                  (unsigned)(lane & 24), 8u);
        const int rank = __builtin_popcount(before_a);  // a permutation of the candidates
        const unsigned long long fine = __builtin_amdgcn_ballot_w64(fine_a == 0xffu) & m_live;
        // Lane (a, b) asks whether candidate a has rank b and passed; folding the bytes of
        // that mask together gives, in bit b, whether the candidate of rank b passed.
        unsigned long long passed = __builtin_amdgcn_ballot_w64(rank == cb) & fine;
        passed |= passed >> 32;
        passed |= passed >> 16;
        passed |= passed >> 8;
        const int left = L.k - it;  // steps still wanted
        int good = __builtin_ctz(~(unsigned)passed | (1u << MAXM));  // ranks 0..good-1 passed
        good = good < left ? good : left;
        centres = __builtin_amdgcn_ballot_w64(rank < good) & FIRST_OF_EIGHT;
        if (good > 0) {  // uniform
            if (wave == 0) {  // uniform
                if (ca == cb && rank < good)
                    out[it + rank] = (int64_t)Bx.y;
            }
            // the last point emitted, should the cloud run out of distinct points
            last_mask = __builtin_amdgcn_ballot_w64(rank == good - 1);
            last_j = Bx.y;
            nc = good;
        } else {
            // No point lies away from the chosen set: the previous choice is emitted again,
            // as the reference does. Every minimum is zero already: nothing is updated.
            if (tid == 0)
                out[it] = last_mask != 0ull
                              ? (int64_t)read_lane(last_j, __builtin_ctzll(last_mask) >> 3)
                              : (int64_t)0;
            nc = 1;
        }
    }
}

// Position of point j in the reference's tie order: its thread's rank among the
// bit-reversed thread ids times the points per thread, plus its turn within the thread.
__device__ __forceinline__ int fps_position_of_point(int j, const FpsLayout &L)
{
    const int t = j & (L.bs - 1);
    const int r = (int)(__builtin_bitreverse32((unsigned)t) >> (32 - L.log2_bs));
    return r * L.c + (j >> L.log2_bs);
}

// fp32 kernel for clouds of 2049 to 16384 points: the multi-step kernel above with the
// points laid out by region, so that an update only visits the points a new centre can
// reach, and with sixteen waves, so that an exchange has sixteen candidates to accept from.
//
// At 16 or 32 points per lane a step is dominated by the update of the running minima
// (nine instructions per point and centre), and almost all of that work changes nothing:
// every running minimum is at most tau, the value of the last exchange's first winner (it
// was the largest of them all, and minima only shrink), so a centre can lower a point's
// minimum only if it lies within sqrt(tau) of it - a ball that shrinks as the sampling
// proceeds. Hence:
//   * the prologue sorts the points along a Morton curve (a counting sort by cell in LDS)
//     and cuts the sorted sequence into 64 regions; region R goes to wave R % 16 as block
//     R / 16 of the lanes' registers (P / 4 points per lane and block), so neighbouring
//     regions sit in different waves, on different SIMDs;
//   * every wave keeps the bounding boxes of its four blocks. Before an update, lane
//     (a, q) evaluates the canonical distance from candidate a to box q - the same rounded
//     operations as tk_dist2 on the per-axis gaps, each of which is monotone, so the
//     result is a lower bound of the canonical distance to every point of the box - and a
//     block is updated only if that bound is below tau. Skipping is therefore exact: a
//     skipped update would have changed no minimum.
//
// Sixteen waves of 16 points per lane instead of eight of 32: an exchange accepts 4.4
// candidates on uniform clouds where eight waves accepted 3.1, the walk to the winner's leaf
// is a level shorter and the regions are half the size. The price is what every wave repeats
// per exchange, now sixteen times on four SIMDs, so that part is kept short: four waves, one
// per SIMD, rank four candidates each (one ballot per condition) while the others work out
// how near the candidates come to their boxes, and ranks and verdicts meet in LDS behind a
// second barrier, as tables that one read and one ballot turn into the mask of certain
// winners; the wave's runner-up comes from a second plain maximum scan that runs beside the
// walk instead of a scan that carries pairs.
//
// Ties. With this layout the lane order is no longer the reference's priority order
// (see the top of the file), so equal maxima are resolved explicitly: a wave that holds
// its maximum more than once picks the point with the lowest reference position (the
// rare slow path below), the slots carry the point's sorted rank, and candidates with equal
// values are ranked by their positions. The acceptance rules are those of
// fps_multistep_kernel_f32.
template <int P, bool SOA, int MAXM>
__global__ __launch_bounds__(1024) void fps_region_kernel_f32(const float *__restrict__ points,
                                                             int64_t *__restrict__ index,
                                                             FpsLayout L)
{
    constexpr int NT = 1024, NW = 16, NB = 4, PB = P / NB, S = NT * P, RS = TK_WAVE * PB;
    constexpr int CELLS = 4096;  // 16^3 cells for the sort
    static_assert(P % NB == 0 && (P & (P - 1)) == 0 && MAXM <= NW && NW * NB == TK_WAVE, "shape");
    static_assert(CELLS % NT == 0 && S < (1 << 19), "sort");
    constexpr int F32_INF = 0x7f800000;
    constexpr int F32_NEG1 = (int)0xbf800000;
    extern __shared__ __align__(16) unsigned char fps_region_lds[];
    unsigned *const keys = reinterpret_cast<unsigned *>(fps_region_lds);  // [S] points, sorted
    unsigned *const cnt = keys + S;                                       // [CELLS + 1]
    __shared__ float4 s_cand[2][NW];  // a wave's candidate: x, y, z, running minimum (bits)
    __shared__ int2 s_aux[2][NW];     // the wave's second-largest minimum, the candidate's rank
    __shared__ int s_rank[2][NW];     // a candidate's rank among them, + 256: it passed
    __shared__ int s_byrank[2][NW];   // by rank: the exchange's number << 9, + 256: that one passed
    __shared__ float s_tau[2];        // the running minimum of the candidate of rank 0
    __shared__ float s_box[NW][NB][8];  // lo.xyz, hi.xyz of a wave's block
    __shared__ float s_red[NW][8];

    const int tid = threadIdx.x;
    const int lane = tid & (TK_WAVE - 1);
    const int wave = tid / TK_WAVE;
    const float *__restrict__ pts = points + (int64_t)blockIdx.x * L.n * 3;
    int64_t *__restrict__ out = index + (int64_t)blockIdx.x * L.k;
    const float INF = __builtin_huge_valf();

    // ---- bounding box of the cloud ----
    // (4 points per lane: also the point farthest from point 0, lowest index first - see
    // ORDER_PROBE below)
    constexpr bool ORDER_PROBE = P == 4;
    float lo[3] = {INF, INF, INF}, hi[3] = {-INF, -INF, -INF};
    float far_d = -1.0f;
    int far_j = 0;
    const float p0x = fps_coord<SOA>(pts, L.n, 0, 0), p0y = fps_coord<SOA>(pts, L.n, 0, 1),
                p0z = fps_coord<SOA>(pts, L.n, 0, 2);
    for (int j = tid; j < L.n; j += NT) {
        float v[3];
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            v[a] = fps_coord<SOA>(pts, L.n, j, a);
            lo[a] = __builtin_fminf(lo[a], v[a]);
            hi[a] = __builtin_fmaxf(hi[a], v[a]);
        }
        if constexpr (ORDER_PROBE) {
            const float d = tk_dist2<float>(v[0], v[1], v[2], p0x, p0y, p0z);
            if (d > far_d) {  // (j ascends within a lane)
                far_d = d;
                far_j = j;
            }
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
    if constexpr (ORDER_PROBE) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float od = __shfl_xor(far_d, o);
            const int oj = __shfl_xor(far_j, o);
            const bool take = od > far_d || (od == far_d && oj < far_j);
            far_d = take ? od : far_d;
            far_j = take ? oj : far_j;
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            s_red[wave][a] = lo[a];
            s_red[wave][3 + a] = hi[a];
        }
        s_red[wave][6] = far_d;
        s_red[wave][7] = __builtin_bit_cast(float, far_j);
    }
    __syncthreads();
    if constexpr (ORDER_PROBE) {
        // ORDER_PROBE. A cloud whose point 1 is the point farthest from point 0 is, in
        // practice, itself the output of a farthest point sampling, in sampling order (the
        // next level of a PointNet++ encoder): every stretch of such a cloud is spread over
        // all of it, which is what the multi-step kernel's waves want (their candidates get
        // in each other's way less: B=16, 4096 -> 1024 0.33 ms there against 0.44 on points
        // in random order) and this kernel, which sorts the points by cell anyway, cannot
        // use (0.39 either way). Such a cloud is left to the multi-step kernel, which is
        // launched behind this one and runs only where it finds the mark: -1 as the last
        // index. (A cloud in random order passes this test once in n.)
        float d = s_red[0][6];
        int j = __builtin_bit_cast(int, s_red[0][7]);
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            const float od = s_red[w][6];
            const int oj = __builtin_bit_cast(int, s_red[w][7]);
            const bool take = od > d || (od == d && oj < j);
            d = take ? od : d;
            j = take ? oj : j;
        }
        if (j == 1) {  // uniform over the workgroup
            if (tid == 0)
                out[L.k - 1] = -1;
            return;
        }
    }
    float origin[3], scale[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        float l = INF, h = -INF;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            l = __builtin_fminf(l, s_red[w][a]);
            h = __builtin_fmaxf(h, s_red[w][3 + a]);
        }
        origin[a] = l;
        const float extent = h - l;
        scale[a] = extent > 0.0f ? 15.99f / extent : 0.0f;  // also 0 for NaN / inf extents
    }

    // ---- the points in the order of their cells along a Morton curve; slots beyond the cloud
    // last. A counting sort: any order that keeps neighbours together is a valid layout, so 16
    // steps per axis are enough and the order within a cell is whatever the atomics give.
    // (A bitonic sort of (code, point) pairs took 105 passes with a barrier each: two thirds
    // of a prologue of 0.19 ms.) ----
    auto spread = [](unsigned v) {  // 4 bits -> every third bit
        v = (v | (v << 4)) & 0x0c3u;
        v = (v | (v << 2)) & 0x249u;
        return v;
    };
    for (int i = tid; i <= CELLS; i += NT)
        cnt[i] = 0u;
    __syncthreads();
    unsigned where[P];  // cell, and the point's turn within it from bit 13
    float own[P][3];    // point tid + k * NT, as read (coalesced) for its cell
#pragma unroll
    for (int k = 0; k < P; ++k) {
        const int e = tid + k * NT;
        unsigned cell = CELLS;
#pragma unroll
        for (int a = 0; a < 3; ++a)
            own[k][a] = e < L.n ? fps_coord<SOA>(pts, L.n, e, a) : 0.0f;
        if (e < L.n) {
            unsigned c3[3];
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                const float f = (own[k][a] - origin[a]) * scale[a];
                // (a NaN or an out-of-range value lands in cell 0 or 15)
                c3[a] = (unsigned)(int)__builtin_fminf(__builtin_fmaxf(f, 0.0f), 15.0f);
            }
            cell = spread(c3[0]) | (spread(c3[1]) << 1) | (spread(c3[2]) << 2);
        }
        where[k] = cell | (atomicAdd(&cnt[cell], 1u) << 13);
    }
    __syncthreads();
    {
        // counts -> first positions: a lane sums its run of counters, the waves scan the sums
        constexpr int RUN = CELLS / NT;
        unsigned c[RUN], mine = 0u;
#pragma unroll
        for (int i = 0; i < RUN; ++i) {
            c[i] = cnt[tid * RUN + i];
            mine += c[i];
        }
        unsigned incl = mine;
#pragma unroll
        for (int o = 1; o < TK_WAVE; o <<= 1) {
            const unsigned up = (unsigned)__shfl_up((int)incl, o);
            incl += lane >= o ? up : 0u;
        }
        if (lane == TK_WAVE - 1)
            s_red[wave][0] = __builtin_bit_cast(float, incl);
        __syncthreads();
        unsigned start = incl - mine;
        for (int w = 0; w < wave; ++w)
            start += __builtin_bit_cast(unsigned, s_red[w][0]);
#pragma unroll
        for (int i = 0; i < RUN; ++i) {
            cnt[tid * RUN + i] = start;
            start += c[i];
        }
        if (tid == 0)
            cnt[CELLS] = (unsigned)L.n;  // the slots beyond the cloud follow its points
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < P; ++k) {
        where[k] = cnt[where[k] & 0x1fffu] + (where[k] >> 13);  // the point's sorted rank
        keys[where[k]] = (unsigned)(tid + k * NT);
    }
    __syncthreads();

    // ---- this lane's points: block q, turn u <-> sorted rank (q*8 + wave) * RS + u*64 + lane.
    // The point indices stay in the sorted list in LDS (16 registers less). ----
    auto rank_of = [&](int in_lane, int p) {
        return ((p / PB) * NW + wave) * RS + (p % PB) * TK_WAVE + in_lane;
    };
    // The coordinates travel from the lanes that read them to the lanes that own them through
    // LDS, one coordinate at a time behind the counters (fetched from memory by sorted rank
    // they were 48 gathers of 64 cache lines per wave: 45 us).
    float x[P], y[P], z[P];
    int t[2 * P];  // t[P + p]: running minimum of point p (bits); t[1..P-1]: maxima
    {
        float *const plane = reinterpret_cast<float *>(cnt);  // [S]
#pragma unroll
        for (int a = 0; a < 3; ++a) {
#pragma unroll
            for (int k = 0; k < P; ++k)
                plane[where[k]] = own[k][a];
            __syncthreads();
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const float v = plane[rank_of(lane, p)];
                if (a == 0)
                    x[p] = v;
                else if (a == 1)
                    y[p] = v;
                else
                    z[p] = v;
            }
            __syncthreads();
        }
    }
#pragma unroll
    for (int p = 0; p < P; ++p)
        t[P + p] = (int)keys[rank_of(lane, p)] < L.n ? F32_INF : F32_NEG1;
    t[0] = 0;
    // boxes of the wave's blocks (an empty block gets an empty box: never reached)
#pragma unroll
    for (int q = 0; q < NB; ++q) {
        float bl[3] = {INF, INF, INF}, bh[3] = {-INF, -INF, -INF};
#pragma unroll
        for (int u = 0; u < PB; ++u) {
            const int p = q * PB + u;
            const bool ok = t[P + p] == F32_INF;
            const float v[3] = {x[p], y[p], z[p]};
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                bl[a] = __builtin_fminf(bl[a], ok ? v[a] : INF);
                bh[a] = __builtin_fmaxf(bh[a], ok ? v[a] : -INF);
            }
        }
#pragma unroll
        for (int a = 0; a < 3; ++a) {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                bl[a] = __builtin_fminf(bl[a], __shfl_xor(bl[a], o));
                bh[a] = __builtin_fmaxf(bh[a], __shfl_xor(bh[a], o));
            }
        }
        if (lane == 0) {
#pragma unroll
            for (int a = 0; a < 3; ++a) {
                s_box[wave][q][a] = bl[a];
                s_box[wave][q][3 + a] = bh[a];
            }
        }
    }
#pragma unroll
    for (int i = P - 1; i >= 1; --i)  // later only the touched blocks' maxima are redone
        t[i] = t[2 * i] > t[2 * i + 1] ? t[2 * i] : t[2 * i + 1];

    // From here on a point is named by its rank in the sorted list; the list is consulted
    // only where a point index is needed (output, ties).
    __syncthreads();  // the boxes are written
    // After an exchange lane (a, q) = (lane / 4, lane % 4) stands for candidate a and tests it
    // against the wave's block q, whose box it keeps in registers.
    const int ca = lane >> 2, cb = lane & 3;
    float box_lo[3], box_hi[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        box_lo[a] = s_box[wave][cb & (NB - 1)][a];
        box_hi[a] = s_box[wave][cb & (NB - 1)][3 + a];
    }
    // The centres of the coming update are the candidates of the lanes in `centres`
    // (lane 4 a stands for candidate a); bit 4 a + q of `reach` says whether candidate a
    // can lower a minimum in block q. The first update is point 0 against every block.
    float ax = fps_coord<SOA>(pts, L.n, 0, 0);
    float ay = fps_coord<SOA>(pts, L.n, 0, 1);
    float az = fps_coord<SOA>(pts, L.n, 0, 2);
    unsigned long long centres = 1ull, reach = (1ull << NB) - 1;
    // the last point emitted is the candidate of lane ctz(last_mask), whose sorted rank that
    // lane keeps in last_rank; no mask: point 0
    unsigned long long last_mask = 0ull;
    int last_rank = 0;
    int nc = 1;
    if (tid == 0)
        out[0] = 0;

    int round = 0;
    for (int it = 1; it < L.k; it += nc, ++round) {
        // ---- running minima: only the blocks a centre can reach ----
        unsigned touched = 0u;
        for (unsigned long long todo = centres; todo != 0ull; todo &= todo - 1) {  // uniform
            const int l = __builtin_ctzll(todo);
            const unsigned blocks = (unsigned)(reach >> l) & ((1u << NB) - 1);
            if (blocks == 0u)
                continue;
            const float sx = read_lane(ax, l), sy = read_lane(ay, l), sz = read_lane(az, l);
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                if ((blocks >> q) & 1u) {  // uniform
#pragma unroll
                    for (int u = 0; u < PB; ++u) {
                        const int p = q * PB + u;
                        const float d = tk_dist2<float>(x[p], y[p], z[p], sx, sy, sz);
                        const int db = __builtin_bit_cast(int, d);
                        t[P + p] = t[P + p] < db ? t[P + p] : db;
                    }
                }
            }
            touched |= blocks;
        }
        // maxima of the touched blocks (node 4 + q is the root of block q), then the top
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            if ((touched >> q) & 1u) {  // uniform
#pragma unroll
                for (int width = PB / 2; width >= 1; width /= 2) {
                    const int first = (NB + q) * width;
#pragma unroll
                    for (int i = first + width - 1; i >= first; --i)
                        t[i] = t[2 * i] > t[2 * i + 1] ? t[2 * i] : t[2 * i + 1];
                }
            }
        }
        t[2] = t[4] > t[5] ? t[4] : t[5];
        t[3] = t[6] > t[7] ? t[6] : t[7];
        t[1] = t[2] > t[3] ? t[2] : t[3];
        // Only points strictly above zero are candidates (the reference starts its
        // scan from max_dist = 0 with strict '>').
        const int best = t[1] > 0 ? t[1] : 0;
        // The wave's maximum and the first lane that holds it; the runner-up is the largest of
        // the other lanes' maxima (a second scan that does not wait for the walk) and of what
        // the walk through the winner lane's own tree passes by.
        const int wmax = wave_max_i32(best);
        int wl = __builtin_ctzll(__builtin_amdgcn_ballot_w64(best == wmax));
        int second = wave_max_i32(lane == wl ? 0 : best);
        FpsPick pick;
        FpsWalk3<P, 1>::go(t, x, y, z, wl, wmax, pick, second);  // and inside lane wl
        int pick_rank = rank_of(wl, pick.j);
        if (second == wmax && wmax > 0) {  // uniform
            // The wave holds its maximum more than once: the reference takes the point with
            // the lowest position in its own order.
            int lane_pos = 0x7fffffff, lane_p = 0;
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const int pos = fps_position_of_point((int)(unsigned)keys[rank_of(lane, p)], L);
                const bool take = t[P + p] == wmax && pos < lane_pos;
                lane_pos = take ? pos : lane_pos;
                lane_p = take ? p : lane_p;
            }
            int wave_pos = lane_pos;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const int other = __shfl_xor(wave_pos, o);
                wave_pos = other < wave_pos ? other : wave_pos;
            }
            wl = __builtin_ctzll(__builtin_amdgcn_ballot_w64(lane_pos == wave_pos));
            const int wp = read_lane(lane_p, wl);
            float sx = x[0], sy = y[0], sz = z[0];
#pragma unroll
            for (int p = 1; p < P; ++p) {
                if (wp == p) {  // uniform
                    sx = x[p];
                    sy = y[p];
                    sz = z[p];
                }
            }
            pick.x = read_lane(sx, wl);
            pick.y = read_lane(sy, wl);
            pick.z = read_lane(sz, wl);
            pick_rank = rank_of(wl, wp);
        }
        const int buf = round & 1;
        if (lane == 0) {
            s_cand[buf][wave] = make_float4(pick.x, pick.y, pick.z, __builtin_bit_cast(float, wmax));
            s_aux[buf][wave] = make_int2(second, pick_rank);
        }
        __syncthreads();
        // How many of the candidates are certain winners of the coming steps. All 64 lanes are
        // active, so conditions are combined as lane masks in scalar registers.
        {
            // Sixteen candidates, 256 relations between them. Four waves (one per SIMD) rank
            // four candidates each: lane (c, b) = (lane / 16, lane % 16) compares candidate
            // 4 wave + c with candidate b, a condition is one ballot whose sixteen-bit groups
            // belong to the four candidates, and rank and verdict go to LDS, where every wave
            // reads them after a second barrier. (Every wave ranking its own candidate in
            // sixteen of its lanes put four copies of the chain on every SIMD; all waves
            // working through all 256 relations, sixteen.)
            if (wave < NW / 4) {  // uniform
                const int mine = 4 * wave + (lane >> 4), other = lane & 15;
                const float4 W = s_cand[buf][mine];
                const int2 Wx = s_aux[buf][mine];
                const float4 Bc = s_cand[buf][other];
                const int2 Bx = s_aux[buf][other];
                const int vw = __builtin_bit_cast(int, W.w), vb = __builtin_bit_cast(int, Bc.w);
                // b comes before the candidate in the reference's order: larger value, then
                // lower position; positions are looked up only when two candidates really hold
                // the same value
                bool before = vb > vw;
                const bool equal = vb == vw && other != mine && vw > 0;
                if (__builtin_amdgcn_ballot_w64(equal) != 0ull) {  // uniform
                    const int pos_w = fps_position_of_point((int)(unsigned)keys[Wx.y], L);
                    const int pos_b = fps_position_of_point((int)(unsigned)keys[Bx.y], L);
                    before |= equal && pos_b < pos_w;
                }
                const float dwb = tk_dist2<float>(W.x, W.y, W.z, Bc.x, Bc.y, Bc.z);
                // the candidate survives b's selection: b's update leaves its minimum alone, and
                // b's wave holds nothing else at or above it
                const bool fine = !before || (__builtin_bit_cast(int, dwb) >= vw && Bx.x < vw);
                const unsigned long long m_before = __builtin_amdgcn_ballot_w64(before);
                const unsigned long long m_fine = __builtin_amdgcn_ballot_w64(fine);
                const unsigned mb = (unsigned)(m_before >> (lane & 48)) & 0xffffu;
                const unsigned mf = (unsigned)(m_fine >> (lane & 48)) & 0xffffu;
                const int verdict = __builtin_popcount(mb) | ((vw > 0 && mf == 0xffffu) ? 256 : 0);
                if (other == 0) {
                    // (The table by rank saves every wave the folding of sixteen verdicts into
                    // one mask, scalar work that sixteen waves repeated. Candidates without a
                    // point left share a rank: an entry counts only with this exchange's
                    // number on it.)
                    s_rank[buf][mine] = verdict;
                    s_byrank[buf][verdict & 15] = (round << 9) | (verdict & 256);
                    if ((verdict & 255) == 0)
                        s_tau[buf] = W.w;
                }
            }
            // Candidate a for lane (a, q) and how near it comes to the box of block q: known
            // since the first barrier. The twelve waves that have nothing to rank work that
            // out while they would wait, the four others behind the second barrier.
            float4 A;
            int2 Ax;  // its wave's second-largest minimum, its sorted rank
            float bound;
            auto approach = [&]() {
                A = s_cand[buf][ca];
                Ax = s_aux[buf][ca];
                const float gx = __builtin_fmaxf(__builtin_fmaxf(box_lo[0] - A.x, A.x - box_hi[0]), 0.0f);
                const float gy = __builtin_fmaxf(__builtin_fmaxf(box_lo[1] - A.y, A.y - box_hi[1]), 0.0f);
                const float gz = __builtin_fmaxf(__builtin_fmaxf(box_lo[2] - A.z, A.z - box_hi[2]), 0.0f);
                bound = __builtin_fmaf(gz, gz, __builtin_fmaf(gy, gy, gx * gx));
            };
            if (wave >= NW / 4)  // uniform
                approach();
            __syncthreads();
            if (wave < NW / 4)  // uniform
                approach();
            const int verdict = s_rank[buf][ca];
            ax = A.x;
            ay = A.y;
            az = A.z;
            const int rank = verdict & 255;  // a permutation of the live candidates
            // lane r (of the first sixteen): did the candidate of rank r pass
            const int by_rank = s_byrank[buf][lane & 15];
            const unsigned passed =
                (unsigned)__builtin_amdgcn_ballot_w64(by_rank == ((round << 9) | 256)) & 0xffffu;
            const int left = L.k - it;  // steps still wanted
            int good = __builtin_ctz(~passed | (1u << MAXM));  // ranks 0..good-1 passed
            good = good < left ? good : left;
            // tau and the reach of candidate a into block q: as with eight waves
            const float tau = s_tau[buf];  // (stale without a live candidate: unused then)
            reach = __builtin_amdgcn_ballot_w64(!(bound >= tau));
            centres = __builtin_amdgcn_ballot_w64(rank < good) & 0x1111111111111111ull;
            if (good > 0) {  // uniform
                if (wave == 0) {  // uniform
                    if (cb == 0 && rank < good)
                        out[it + rank] = (int64_t)(unsigned)keys[Ax.y];
                }
                // the last point emitted, should the cloud run out of distinct points
                last_mask = __builtin_amdgcn_ballot_w64(rank == good - 1);
                last_rank = Ax.y;
                nc = good;
            } else {
                // No point lies away from the chosen set: the previous choice is emitted again.
                if (tid == 0) {
                    int64_t j = 0;
                    if (last_mask != 0ull)
                        j = (int64_t)(unsigned)keys[read_lane(last_rank, __builtin_ctzll(last_mask))];
                    out[it] = j;
                }
                nc = 1;
            }
        }
    }
}

// Clouds that do not fit in one workgroup's registers: every selection step is one
// launch of many workgroups per cloud. Step s first works out the point chosen by step
// s - 1 from the candidates that step's workgroups left in the workspace (every workgroup
// redoes this small reduction itself), then updates the running minima of its own slice
// of the cloud for that centre, streaming coordinates and minima through coalesced
// loads, and leaves its own candidate for step s + 1. The kernel boundary is the
// cross-workgroup barrier; nothing waits inside a kernel.
//
// Points are visited in index order; the reference's tie order is restored by comparing
// positions (see the top of the file) whenever two minima are equal.
template <typename T> struct FpsWideArgs {
    const T *points;     // [B, n, 3] or [B, 3, n]
    int64_t *index;      // [B, k]
    T *min_dist;         // [B, n]
    T *cand_val;         // [2, B, groups]: largest running minimum of a workgroup's slice
    int *cand_pos;       // [2, B, groups]: its position
    int *chosen;         // [2, B]: the point the previous step used as centre
    int groups;          // workgroups per cloud
    int slice;           // points per workgroup
    int batch;           // B
};

// (value, position) pairs ordered by larger value, then lower position.
template <typename T>
__device__ __forceinline__ void fps_keep_better(T &val, int &pos, T oval, int opos)
{
    const bool take = oval > val || (oval == val && opos < pos);
    val = take ? oval : val;
    pos = take ? opos : pos;
}

template <typename T, int NT>
__device__ __forceinline__ void fps_block_best(T &val, int &pos, T *s_val, int *s_pos)
{
    constexpr int NW = NT / TK_WAVE;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const T oval = __shfl_xor(val, o);
        const int opos = __shfl_xor(pos, o);
        fps_keep_better<T>(val, pos, oval, opos);
    }
    __syncthreads();  // the arrays may still be read from an earlier call
    if ((threadIdx.x & (TK_WAVE - 1)) == 0) {
        s_val[threadIdx.x / TK_WAVE] = val;
        s_pos[threadIdx.x / TK_WAVE] = pos;
    }
    __syncthreads();
    val = s_val[0];
    pos = s_pos[0];
#pragma unroll
    for (int w = 1; w < NW; ++w)
        fps_keep_better<T>(val, pos, s_val[w], s_pos[w]);
}

template <typename T, int NT, bool SOA>
__global__ __launch_bounds__(NT) void fps_wide_step_kernel(FpsWideArgs<T> a, FpsLayout L,
                                                           int step)
{
    __shared__ T s_val[NT / TK_WAVE];
    __shared__ int s_pos[NT / TK_WAVE];
    const int tid = threadIdx.x;
    const int g = blockIdx.x, b = blockIdx.y;
    const T *__restrict__ pts = a.points + (int64_t)b * L.n * 3;
    constexpr int NO_POS = 0x7fffffff;

    // ---- the centre of this step: what step - 1 selected ----
    int centre = 0;
    if (step > 1) {
        const int from = (step - 1) & 1;
        const T *cv = a.cand_val + ((int64_t)from * a.batch + b) * a.groups;
        const int *cp = a.cand_pos + ((int64_t)from * a.batch + b) * a.groups;
        T val = (T)0;
        int pos = NO_POS;
        for (int i = tid; i < a.groups; i += NT)
            fps_keep_better<T>(val, pos, cv[i], cp[i]);
        fps_block_best<T, NT>(val, pos, s_val, s_pos);
        // Nothing above zero: no point lies away from the chosen set and the previous
        // choice is emitted again, as the reference does.
        centre = val > (T)0 ? fps_point_of_position(pos, L) : a.chosen[(int64_t)from * a.batch + b];
    }
    if (g == 0 && tid == 0) {
        a.index[(int64_t)b * L.k + (step - 1)] = (int64_t)centre;
        a.chosen[(int64_t)(step & 1) * a.batch + b] = centre;
    }
    if (step >= L.k)  // the last launch only records the last choice
        return;

    // ---- update this workgroup's slice, keep its best candidate ----
    const T cx = fps_coord<SOA>(pts, L.n, centre, 0), cy = fps_coord<SOA>(pts, L.n, centre, 1),
            cz = fps_coord<SOA>(pts, L.n, centre, 2);
    T *__restrict__ md = a.min_dist + (int64_t)b * L.n;
    const int j0 = g * a.slice;
    const int j1 = (j0 + a.slice < L.n) ? j0 + a.slice : L.n;
    T best = (T)0;
    int bpos = NO_POS;
    for (int j = j0 + tid; j < j1; j += NT) {
        T x, y, z;
        if (SOA) {
            x = pts[j], y = pts[(int64_t)L.n + j], z = pts[2 * (int64_t)L.n + j];
        } else {
            const TkPoint3<T> p = tk_load3<T>(pts + (int64_t)j * 3);
            x = p.x, y = p.y, z = p.z;
        }
        const T d = tk_dist2<T>(x, y, z, cx, cy, cz);
        // The first step assigns whatever it computes (sample_farthest_points_kernel.cu:59-64
        // starts from "unset"); a NaN there never compares above anything, which -1 mimics.
        const T nm = step == 1 ? (d != d ? (T)-1 : d) : tk_min<T>(md[j], d);
        md[j] = nm;
        if (nm > (T)0 && nm >= best)
            fps_keep_better<T>(best, bpos, nm, fps_position_of_point(j, L));
    }
    fps_block_best<T, NT>(best, bpos, s_val, s_pos);
    if (tid == 0) {
        const int64_t o = ((int64_t)(step & 1) * a.batch + b) * a.groups + g;
        a.cand_val[o] = best;
        a.cand_pos[o] = bpos;
    }
}

// Workgroups per cloud and points per workgroup of the wide kernel.
inline void fps_wide_shape(int64_t B, int64_t N, int &groups, int &slice)
{
    constexpr int64_t MIN_SLICE = 2048, MAX_GROUPS = 1024;
    int64_t want = (2048 + B - 1) / B;  // about 2048 workgroups in flight
    int64_t g = (N + MIN_SLICE - 1) / MIN_SLICE;
    if (g > want)
        g = want;
    if (g > MAX_GROUPS)
        g = MAX_GROUPS;
    if (g < 1)
        g = 1;
    slice = (int)((N + g - 1) / g);
    groups = (int)((N + slice - 1) / slice);
}

template <typename T> struct FpsWideLayout {
    size_t min_dist, cand_val, cand_pos, chosen, total;
};

template <typename T> FpsWideLayout<T> fps_wide_layout(int64_t B, int64_t N, int groups)
{
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    FpsWideLayout<T> w;
    w.min_dist = 0;
    w.cand_val = up((size_t)B * (size_t)N * sizeof(T));
    w.cand_pos = w.cand_val + up((size_t)2 * B * groups * sizeof(T));
    w.chosen = w.cand_pos + up((size_t)2 * B * groups * sizeof(int));
    w.total = w.chosen + up((size_t)2 * B * sizeof(int));
    return w;
}

FpsLayout fps_layout(int64_t n, int64_t k)
{
    FpsLayout L;
    L.n = (int)n;
    L.k = (int)k;
    int bs = 1, lg = 0;
    // Block size of the reference: smallest power of two >= n, capped at 512
    // (sample_farthest_points_kernel.cu:132-133); its switch runs 32 threads for
    // anything smaller (:153-161).
    while (bs < n && bs < 512) {
        bs *= 2;
        ++lg;
    }
    while (bs < 32) {
        bs *= 2;
        ++lg;
    }
    L.bs = bs;
    L.log2_bs = lg;
    L.c = (int)((n + bs - 1) / bs);
    L.inv_c = 1.0f / (float)L.c;
    return L;
}

// Largest number of positions the register kernel holds for element size `es`.
int64_t fps_register_capacity(size_t es) { return es == 4 ? 1024 * 16 : 1024 * 8; }

template <typename T, int P, int NT>
void fps_launch(const T *points, bool soa, int64_t B, int64_t *index, const FpsLayout &L,
                hipStream_t s)
{
    if (soa)
        hipLaunchKernelGGL((fps_register_kernel<T, P, NT, true>), dim3((unsigned)B), dim3(NT), 0,
                           s, points, index, L, 0);
    else
        hipLaunchKernelGGL((fps_register_kernel<T, P, NT, false>), dim3((unsigned)B), dim3(NT),
                           0, s, points, index, L, 0);
}

template <int P, int NT>
void fps_launch_f32(const float *points, bool soa, int64_t B, int64_t *index,
                    const FpsLayout &L, hipStream_t s)
{
    constexpr int MAXM = 6;  // 4 -> 6 gains 1-4 %, 8 nothing
    if (soa) {
        hipLaunchKernelGGL((fps_multistep_kernel_f32<P, NT, true, MAXM>), dim3((unsigned)B),
                           dim3(NT), 0, s, points, index, L);
        hipLaunchKernelGGL((fps_register_kernel<float, P, NT, true>), dim3((unsigned)B),
                           dim3(NT), 0, s, points, index, L, 1);
    } else {
        hipLaunchKernelGGL((fps_multistep_kernel_f32<P, NT, false, MAXM>), dim3((unsigned)B),
                           dim3(NT), 0, s, points, index, L);
        hipLaunchKernelGGL((fps_register_kernel<float, P, NT, false>), dim3((unsigned)B),
                           dim3(NT), 0, s, points, index, L, 1);
    }
}

// Clouds of 2049 to 16384 points: the region kernel, then the same check for non-finite
// coordinates as above.
template <int P>
int fps_region_launch_f32(const float *points, bool soa, int64_t B, int64_t *index,
                          const FpsLayout &L, hipStream_t s)
{
    constexpr int MAXM = 8, NT = 1024;
    // the sorted list, and behind it the sort's counters, then one coordinate of every point
    constexpr int LDS = NT * P * 4 + (NT * P > 4100 ? NT * P : 4100) * 4;
    if (soa) {
        constexpr auto kernel = fps_region_kernel_f32<P, true, MAXM>;
        const int allowed = tk_allow_dynamic_lds<kernel>(LDS);
        if (allowed != TK3D_OK)
            return allowed;
        hipLaunchKernelGGL(kernel, dim3((unsigned)B), dim3(NT), LDS, s, points, index, L);
        if constexpr (P == 4)  // clouds in sampling order, which the kernel above leaves
            hipLaunchKernelGGL((fps_multistep_kernel_f32<8, 512, true, 6, true>),
                               dim3((unsigned)B), dim3(512), 0, s, points, index, L);
        hipLaunchKernelGGL((fps_register_kernel<float, P, NT, true>), dim3((unsigned)B),
                           dim3(NT), 0, s, points, index, L, 1);
    } else {
        constexpr auto kernel = fps_region_kernel_f32<P, false, MAXM>;
        const int allowed = tk_allow_dynamic_lds<kernel>(LDS);
        if (allowed != TK3D_OK)
            return allowed;
        hipLaunchKernelGGL(kernel, dim3((unsigned)B), dim3(NT), LDS, s, points, index, L);
        if constexpr (P == 4)
            hipLaunchKernelGGL((fps_multistep_kernel_f32<8, 512, false, 6, true>),
                               dim3((unsigned)B), dim3(512), 0, s, points, index, L);
        hipLaunchKernelGGL((fps_register_kernel<float, P, NT, false>), dim3((unsigned)B),
                           dim3(NT), 0, s, points, index, L, 1);
    }
    return TK3D_OK;
}

// fp32: (points per lane, lanes) by cloud size, from timing every shape on an
// MI355X: two waves per SIMD (512 lanes) hide each other's reduction latency; more
// waves only repeat the per-wave reduction.
int fps_dispatch_f32(const float *points, bool soa, int64_t B, int64_t *index,
                     const FpsLayout &L, int64_t npos, hipStream_t s)
{
    if (npos <= 64 * 2)
        fps_launch_f32<2, 64>(points, soa, B, index, L, s);
    else if (npos <= 256 * 2)
        fps_launch_f32<2, 256>(points, soa, B, index, L, s);
    else if (npos <= 512 * 2)
        fps_launch_f32<2, 512>(points, soa, B, index, L, s);
    else if (npos <= 512 * 4)
        fps_launch_f32<4, 512>(points, soa, B, index, L, s);
    // From 2049 points on the region kernel with 4 points per lane, once its prologue is paid
    // for: B=16, 4096 -> 1024 0.44 -> 0.40 ms, 3000 -> 1024 0.47 -> 0.39 ms, 2100 -> 512
    // 0.26 -> 0.21 ms, 4096 -> 4096 1.65 -> 1.38 ms; 4096 -> 384 is level, -> 256 10 % behind.
    else if (npos > 512 * 4 && npos <= 512 * 8 && L.k >= (npos <= 512 * 6 ? 256 : 512))
        return fps_region_launch_f32<4>(points, soa, B, index, L, s);
    else if (npos <= 512 * 8)
        fps_launch_f32<8, 512>(points, soa, B, index, L, s);
    // Beyond 4096 points the region kernel (sixteen waves; its prologue costs about 30 us) wins
    // from a few hundred samples on: B=16, 8192 -> 2048 1.20 -> 0.94 ms, B=4, 10000 -> 512
    // 0.53 -> 0.34 ms, B=8, 16384 -> 512 0.51 -> 0.38 ms; at 4096 points it is level with the
    // kernel above at 1024 samples and behind it below.
    else if (npos <= 512 * 16 && L.k >= 256)
        return fps_region_launch_f32<8>(points, soa, B, index, L, s);
    else if (npos <= 512 * 16)
        fps_launch_f32<16, 512>(points, soa, B, index, L, s);
    else if (L.k >= 256)
        return fps_region_launch_f32<16>(points, soa, B, index, L, s);
    else
        fps_launch_f32<32, 512>(points, soa, B, index, L, s);
    return TK3D_OK;
}

// Coordinates of the picks: sampled[b, i, :] = points[b, index[b, i], :] in the layout of
// the input cloud ([B,K,3], or [B,3,K] with SOA). A launch of its own after the
// selection kernel: storing the coordinates from the selection loop changed that loop's
// register allocation and cost it 4-9 %, far more than this pass.
template <typename T, bool SOA>
__global__ __launch_bounds__(256) void fps_gather_kernel(const T *__restrict__ points,
                                                         const int64_t *__restrict__ index,
                                                         T *__restrict__ sampled, int n, int k)
{
    const int b = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= k)
        return;
    const T *__restrict__ pts = points + (int64_t)b * n * 3;
    T *__restrict__ so = sampled + (int64_t)b * k * 3;
    const int64_t j = index[(int64_t)b * k + i];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        const T v = fps_coord<SOA>(pts, n, j, a);
        if (SOA)
            so[(int64_t)a * k + i] = v;
        else
            so[(int64_t)i * 3 + a] = v;
    }
}

template <typename T>
int fps_finish(const T *points, bool soa, int64_t B, int64_t N, int64_t K,
               const int64_t *index, T *sampled, hipStream_t s)
{
    const int rc = tk_launch_status();
    if (rc != TK3D_OK || !sampled)
        return rc;
    const dim3 grid((unsigned)((K + 255) / 256), (unsigned)B);
    if (B > 65535)
        return TK3D_ERR_UNSUPPORTED;
    if (soa)
        hipLaunchKernelGGL((fps_gather_kernel<T, true>), grid, dim3(256), 0, s, points, index,
                           sampled, (int)N, (int)K);
    else
        hipLaunchKernelGGL((fps_gather_kernel<T, false>), grid, dim3(256), 0, s, points, index,
                           sampled, (int)N, (int)K);
    return tk_launch_status();
}

template <typename T>
int fps(const T *points, bool soa, int64_t B, int64_t N, int64_t K, int64_t *index, T *sampled,
        void *workspace, size_t workspace_bytes, void *stream)
{
    if (B < 0 || N < 0)
        return TK3D_ERR_BAD_SIZE;
    if (K <= 0 || K > N)
        return TK3D_ERR_BAD_K;
    if (N > ((int64_t)1 << 23) || B > TK_MAX_I32 || !tk_fits(TK_MAX_ELEMS, B, N, 3))
        return TK3D_ERR_UNSUPPORTED;
    if (B == 0)
        return TK3D_OK;
    if (!points || !index)
        return TK3D_ERR_NULL_POINTER;
    hipStream_t s = (hipStream_t)stream;
    const FpsLayout L = fps_layout(N, K);
    const int64_t npos = (int64_t)L.bs * L.c;
    if (npos <= fps_register_capacity(sizeof(T))) {
        if constexpr (sizeof(T) == 4) {
            const int rc = fps_dispatch_f32(points, soa, B, index, L, npos, s);
            if (rc != TK3D_OK)
                return rc;
            return fps_finish<T>(points, soa, B, N, K, index, sampled, s);
        }
        // Fewest points per lane that still covers the cloud: short serial chains.
        if (npos <= 256 * 1)
            fps_launch<T, 1, 256>(points, soa, B, index, L, s);
        else if (npos <= 256 * 2)
            fps_launch<T, 2, 256>(points, soa, B, index, L, s);
        else if (npos <= 512 * 2)
            fps_launch<T, 2, 512>(points, soa, B, index, L, s);
        else if (npos <= 1024 * 2)
            fps_launch<T, 2, 1024>(points, soa, B, index, L, s);
        else if (npos <= 1024 * 4)
            fps_launch<T, 4, 1024>(points, soa, B, index, L, s);
        else if (npos <= 1024 * 8)
            fps_launch<T, 8, 1024>(points, soa, B, index, L, s);
        else if constexpr (sizeof(T) == 4)
            fps_launch<T, 16, 1024>(points, soa, B, index, L, s);
        return fps_finish<T>(points, soa, B, N, K, index, sampled, s);
    }
    // Larger clouds: one launch per selection step, many workgroups per cloud.
    int groups, slice;
    fps_wide_shape(B, N, groups, slice);
    const FpsWideLayout<T> w = fps_wide_layout<T>(B, N, groups);
    if (!workspace || workspace_bytes < w.total || ((uintptr_t)workspace & 7) != 0)
        return TK3D_ERR_WORKSPACE;
    if (B > 65535)
        return TK3D_ERR_UNSUPPORTED;
    char *base = (char *)workspace;
    FpsWideArgs<T> a;
    a.points = points;
    a.index = index;
    a.min_dist = (T *)(base + w.min_dist);
    a.cand_val = (T *)(base + w.cand_val);
    a.cand_pos = (int *)(base + w.cand_pos);
    a.chosen = (int *)(base + w.chosen);
    a.groups = groups;
    a.slice = slice;
    a.batch = (int)B;
    const dim3 grid((unsigned)groups, (unsigned)B);
    for (int64_t step = 1; step <= K; ++step) {
        // The last launch has nothing to update: one workgroup per cloud records the choice.
        const dim3 gr = step == K ? dim3(1u, (unsigned)B) : grid;
        if (soa)
            hipLaunchKernelGGL((fps_wide_step_kernel<T, 256, true>), gr, dim3(256), 0, s, a, L,
                               (int)step);
        else
            hipLaunchKernelGGL((fps_wide_step_kernel<T, 256, false>), gr, dim3(256), 0, s, a, L,
                               (int)step);
    }
    return fps_finish<T>(points, soa, B, N, K, index, sampled, s);
}

// Workspace of tk3d_sample_farthest_points_static_f32: lives in the library's device
// image, one copy per GPU, for callers that cannot allocate. In host code the array's
// name is only a handle for hipGetSymbolAddress; kernels are handed the address that
// call returns for the current device.
__device__ __align__(256) unsigned char fps_static_scratch[TK3D_FPS_STATIC_WORKSPACE_BYTES];

// Device address of fps_static_scratch on the current device, looked up once per device.
int fps_static_scratch_address(void **address)
{
    constexpr int MAX_DEVICES = 64;
    static std::atomic<void *> known[MAX_DEVICES];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES)
        return TK3D_ERR_UNSUPPORTED;
    void *p = known[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(fps_static_scratch));
        if (e != hipSuccess)
            return (int)e;
        if (!p)
            return TK3D_ERR_WORKSPACE;
        known[dev].store(p, std::memory_order_release);  // every thread finds the same value
    }
    *address = p;
    return TK3D_OK;
}

}  // namespace

extern "C" {

size_t tk3d_sample_farthest_points_workspace_bytes(int64_t B, int64_t N, size_t elem_size)
{
    if (B <= 0 || N <= 0 || (elem_size != 4 && elem_size != 8))
        return 0;
    const FpsLayout L = fps_layout(N, 1);
    const int64_t npos = (int64_t)L.bs * L.c;
    if (npos <= fps_register_capacity(elem_size))
        return 0;
    int groups, slice;
    fps_wide_shape(B, N, groups, slice);
    return elem_size == 4 ? fps_wide_layout<float>(B, N, groups).total
                          : fps_wide_layout<double>(B, N, groups).total;
}

int tk3d_sample_farthest_points_f32(const float *points, int64_t B, int64_t N,
                                    int64_t num_samples, int64_t *index, void *workspace,
                                    size_t workspace_bytes, void *stream)
{
    return fps<float>(points, false, B, N, num_samples, index, nullptr, workspace,
                      workspace_bytes, stream);
}

int tk3d_sample_farthest_points_static_f32(const float *points, int64_t B, int64_t N,
                                           int64_t num_samples, int64_t *index, void *stream)
{
    const size_t need = tk3d_sample_farthest_points_workspace_bytes(B, N, sizeof(float));
    if (need > (size_t)TK3D_FPS_STATIC_WORKSPACE_BYTES)
        return TK3D_ERR_WORKSPACE;
    void *scratch = nullptr;
    if (need > 0) {
        const int rc = fps_static_scratch_address(&scratch);
        if (rc != TK3D_OK)
            return rc;
    }
    // Nothing in the workspace has to start at zero: the first step assigns every running
    // minimum and each later step reads only what the step before it wrote.
    return fps<float>(points, false, B, N, num_samples, index, nullptr, scratch,
                      need > 0 ? (size_t)TK3D_FPS_STATIC_WORKSPACE_BYTES : 0, stream);
}

int tk3d_sample_farthest_points_f64(const double *points, int64_t B, int64_t N,
                                    int64_t num_samples, int64_t *index, void *workspace,
                                    size_t workspace_bytes, void *stream)
{
    return fps<double>(points, false, B, N, num_samples, index, nullptr, workspace,
                       workspace_bytes, stream);
}

int tk3d_sample_farthest_points_gather_f32(const float *points, int channels_first,
                                           int64_t B, int64_t N, int64_t num_samples,
                                           int64_t *index, float *sampled, void *workspace,
                                           size_t workspace_bytes, void *stream)
{
    return fps<float>(points, channels_first != 0, B, N, num_samples, index, sampled,
                      workspace, workspace_bytes, stream);
}

int tk3d_sample_farthest_points_gather_f64(const double *points, int channels_first,
                                           int64_t B, int64_t N, int64_t num_samples,
                                           int64_t *index, double *sampled, void *workspace,
                                           size_t workspace_bytes, void *stream)
{
    return fps<double>(points, channels_first != 0, B, N, num_samples, index, sampled,
                       workspace, workspace_bytes, stream);
}

}  // extern "C"

// Sliding-window register-tile engine for definition-based 2D cross-correlation on
// gfx950 (64-lane wavefronts, 160 KB LDS per CU).
//
//   out[v,u][sy][sx] = sum over (yr, xr) of V_v[yr+sy][xr+sx] * U_u[yr][xr]
//
// V is the "left" matrix array, U the "right" one. One kernel template covers the
// sliding-window kernel families of the reference (naive_shuffle.cu,
// naive_shuffle_multirow_both.cu, naive_shuffle_multimat_right.cu,
// naive_shuffle_one_to_many_multirow_both_multimat_right.cu,
// naive_shuffle_n_to_m_multimat_both.cu,
// naive_shuffle_n_to_m_multirow_both_multimat_both.cu); it is not derived from
// their warp-shuffle conveyor, which has no efficient 64-lane equivalent:
//
//   * a lane owns a register tile of A adjacent y shifts x B adjacent x shifts for
//     NV left x NU right matrices (NV*NU*A*B accumulators);
//   * the 64 lanes of a wavefront are laid out LX x LY over shifts and LV x LU over
//     left / right matrices, so small matrices get narrow shift tiles (less work
//     wasted on partial overlaps) without losing register-level reuse;
//   * a block stages a band of RL left rows and the matching band of right rows in
//     LDS, zero padded, so the inner loop has no bounds checks;
//   * per left row and K right columns a lane reads one B+K-1 wide left window and
//     one new right row of K values; the A right rows it needs are kept in a
//     register ring that rotates by one row per step (the y loop is unrolled A times
//     so every ring index is static). That is NV*NU*A*B*K FMAs for
//     NV*ceil((B+K-1)/v) + NU*ceil(K/v) 128-bit LDS reads (v = 16 / sizeof(T));
//   * the reduction over left rows can be split into chunks (work items) whose
//     partial sums are added with hardware float atomics, which is what fills 256
//     CUs when a single large pair has only ~1000 wavefront tiles.
#pragma once

#include <hip/hip_runtime.h>

namespace xcorr {

template <typename T>
struct EngineArgs {
    const T *V;
    const T *U;
    T *out;
    int W, H;           // matrix cols, rows
    int nV, nU;         // matrix counts
    int group_m;        // 0: all pairs, out index v*nU + u. >0: left v pairs with right [v*m, (v+1)*m), out index = right index
    int rows_per_chunk; // left rows one work item reduces over
    int dist;           // 0 none, 1 rectangle, 2 triangle (how worker ids map to (y tile, chunk))
    int atomic;         // 1: atomicAdd partial sums into a zeroed output
    int ntx, nty;       // number of block tiles in x and y
    int nworkers_y;     // number of (y tile, chunk) workers
    int nvg, nug;       // left / right matrix groups
};

template <typename T, int A_, int B_, int K_, int NV_, int NU_, int LX_, int LY_, int LV_, int LU_, int WX_, int WY_,
          int RL_, int KBX_, int MINB_>
struct EngineCfg {
    using value_type = T;
    static constexpr int A = A_, B = B_, K = K_, NV = NV_, NU = NU_;
    static constexpr int LX = LX_, LY = LY_, LV = LV_, LU = LU_;
    static constexpr int WX = WX_, WY = WY_, RL = RL_, KBX = KBX_, MINB = MINB_;
    static constexpr int VK = 16 / (int)sizeof(T); // elements per 128-bit LDS access
    static constexpr int TXW = LX * B, TYW = LY * A; // wavefront tile (shifts)
    static constexpr int TXB = TXW * WX, TYB = TYW * WY; // block tile (shifts)
    static constexpr int NWAVES = WX * WY, NT = 64 * NWAVES;
    static constexpr int VWIN = B + K - 1;
    static constexpr int VWIN_VECS = (VWIN + VK - 1) / VK;
    static constexpr int KVECS = K / VK;
    static constexpr int NVB = LV * NV, NUB = LU * NU; // matrices per block
    // LDS geometry (elements)
    static constexpr int PV = TXB - B + KBX - K + VWIN_VECS * VK;
    static constexpr int VBAND = RL * PV;
    static constexpr int RU = RL + TYB - 1;
    static constexpr int PU = KBX + VK;
    static constexpr int UBAND = RU * PU;
    static constexpr int LDS_ELEMS = NVB * VBAND + NUB * UBAND;
    static constexpr int LDS_BYTES = LDS_ELEMS * (int)sizeof(T);
    static_assert(LX * LY * LV * LU == 64, "lane layout must cover one wavefront");
    static_assert(B % VK == 0 && K % VK == 0 && KBX % K == 0 && RL % A == 0, "tile alignment");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

template <typename T>
struct vec128;
template <>
struct vec128<float> {
    typedef float type __attribute__((ext_vector_type(4)));
};
template <>
struct vec128<double> {
    typedef double type __attribute__((ext_vector_type(2)));
};

__device__ __forceinline__ void atomic_add(float *p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add(double *p, double v) { unsafeAtomicAdd(p, v); }

// Number of left rows that overlap any shift of y tile `ty`, and the first such row.
template <class C>
__device__ __host__ __forceinline__ void tile_rows(int ty, int H, int &lo, int &hi) {
    int syb = -(H - 1) + ty * C::TYB;
    lo = syb > 0 ? syb : 0;
    int h = syb + C::TYB - 1 + H;
    hi = h < H ? h : H;
}

template <class C>
__global__ __launch_bounds__(C::NT, C::MINB) void engine_kernel(EngineArgs<typename C::value_type> g) {
    using T = typename C::value_type;
    using vec = typename vec128<T>::type;
    constexpr int A = C::A, B = C::B, K = C::K, NV = C::NV, NU = C::NU, VK = C::VK;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *Vs = reinterpret_cast<T *>(smem_raw);
    T *Us = Vs + C::NVB * C::VBAND;

    const int tid = threadIdx.x;
    const int W = g.W, H = g.H;

    // ---- decode the work item (block-uniform) ----
    int item = blockIdx.x;
    const int mat = item % (g.nvg * g.nug);
    item /= (g.nvg * g.nug);
    const int worker = item % g.nworkers_y;
    const int txi = item / g.nworkers_y;
    const int ug = mat % g.nug, vg = mat / g.nug;
    // x tiles are visited centre-out: the block index order is the dispatch order and
    // central tiles have the longest overlaps
    const int txc = g.ntx / 2;
    const int tx = (txi & 1) ? txc - (txi + 1) / 2 : txc + txi / 2;

    int ty, chunk;
    if (g.dist == 0) {
        ty = worker;
        chunk = 0;
    } else if (g.dist == 1) {
        ty = worker % g.nty;
        chunk = worker / g.nty;
    } else {
        int w = worker;
        ty = 0;
        for (; ty < g.nty; ++ty) {
            int lo, hi;
            tile_rows<C>(ty, H, lo, hi);
            int n = (hi - lo + g.rows_per_chunk - 1) / g.rows_per_chunk;
            if (w < n) break;
            w -= n;
        }
        chunk = w;
        if (ty >= g.nty) return;
    }
    int row_lo, row_hi;
    tile_rows<C>(ty, H, row_lo, row_hi);
    const int clo = row_lo + chunk * g.rows_per_chunk;
    int chi = clo + g.rows_per_chunk;
    if (chi > row_hi) chi = row_hi;
    if (clo >= chi) return; // surplus worker of the rectangle distribution

    const int syb = -(H - 1) + ty * C::TYB;
    const int sxb = -(W - 1) + tx * C::TXB;

    // matrices of this block
    const int v_first = vg * C::NVB;
    int u_first, u_limit;
    if (g.group_m > 0) {
        u_first = v_first * g.group_m + ug * C::NUB;
        u_limit = (v_first + 1) * g.group_m;
    } else {
        u_first = ug * C::NUB;
        u_limit = g.nU;
    }

    // right columns with any overlap for this block tile, aligned down to the staging width
    int xr_lo = -(sxb + C::TXB - 1);
    if (xr_lo < 0) xr_lo = 0;
    xr_lo = (xr_lo / C::KBX) * C::KBX;
    int xr_hi = W - sxb;
    if (xr_hi > W) xr_hi = W;

    // ---- lane coordinates ----
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wx = wave % C::WX, wy = wave / C::WX;
    const int lx = lane % C::LX;
    const int ly = (lane / C::LX) % C::LY;
    const int lv = (lane / (C::LX * C::LY)) % C::LV;
    const int lu = lane / (C::LX * C::LY * C::LV);
    const int sxw = sxb + wx * C::TXW; // first x shift of the wavefront tile
    const int syw = syb + wy * C::TYW;
    const T *Vs_lane = Vs + lv * NV * C::VBAND + wx * C::TXW + lx * B;
    const int lane_ru0 = C::TYB - 1 - (wy * C::TYW + ly * A);
    const T *Us_lane = Us + lu * NU * C::UBAND + lane_ru0 * C::PU;

    T acc[NV][NU][A][B];
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int n = 0; n < NU; ++n)
#pragma unroll
            for (int a = 0; a < A; ++a)
#pragma unroll
                for (int b = 0; b < B; ++b) acc[i][n][a][b] = T(0);

    const size_t HW = (size_t)W * H;

    for (int yl0 = clo; yl0 < chi; yl0 += C::RL) {
        // groups of A left rows of this stage that can overlap this wavefront's y shifts
        int jj_lo = 0, jj_hi = C::RL / A;
        {
            // rows yl in [syw, syw + TYW - 1 + H - 1] and yl < chi
            int first = syw - yl0;                     // first useful row index j
            int last = syw + C::TYW + H - 2 - yl0;     // last useful row index j
            if (chi - 1 - yl0 < last) last = chi - 1 - yl0;
            if (first > 0) jj_lo = first / A;
            int h = last < 0 ? 0 : last / A + 1;
            if (h < jj_hi) jj_hi = h;
        }
        for (int x0 = xr_lo; x0 < xr_hi; x0 += C::KBX) {
            __syncthreads(); // everyone is done reading the previous stage
            // ---- stage the left band: rows [yl0, yl0+RL), columns xl = x0 + sxb + col ----
            {
                const int xbase = x0 + sxb;
                constexpr int TOT = C::NVB * C::VBAND;
#pragma unroll 4
                for (int idx = tid; idx < TOT; idx += C::NT) {
                    int col = idx % C::PV;
                    int t = idx / C::PV;
                    int row = t % C::RL;
                    int band = t / C::RL;
                    int v = v_first + band, yl = yl0 + row, xl = xbase + col;
                    T val = T(0);
                    if (v < g.nV && yl < chi && (unsigned)xl < (unsigned)W) val = g.V[(size_t)v * HW + (size_t)yl * W + xl];
                    Vs[idx] = val;
                }
            }
            // ---- stage the right band: rows yr = yl0 - syb - TYB + 1 + row, columns xr = x0 + col ----
            {
                const int yr0 = yl0 - syb - C::TYB + 1;
                constexpr int TOT = C::NUB * C::UBAND;
#pragma unroll 4
                for (int idx = tid; idx < TOT; idx += C::NT) {
                    int col = idx % C::PU;
                    int t = idx / C::PU;
                    int row = t % C::RU;
                    int band = t / C::RU;
                    int u = u_first + band, yr = yr0 + row, xr = x0 + col;
                    T val = T(0);
                    if (u < u_limit && col < C::KBX && (unsigned)yr < (unsigned)H && xr < W)
                        val = g.U[(size_t)u * HW + (size_t)yr * W + xr];
                    Us[idx] = val;
                }
            }
            __syncthreads();

            // ---- K-column chunks of this stage that overlap this wavefront's x shifts ----
            int kc_lo = 0, kc_hi = C::KBX / K;
            {
                // need (x0 + kc*K + K-1) + (sxw + TXW-1) >= 0 and (x0 + kc*K) + sxw <= W-1 and x0 + kc*K < W
                int need = -(sxw + C::TXW - 1) - (K - 1) - x0;
                if (need > 0) kc_lo = (need + K - 1) / K;
                int lim = W - 1 - sxw - x0;
                if (W - 1 - x0 < lim) lim = W - 1 - x0;
                int h = lim < 0 ? 0 : lim / K + 1;
                if (h < kc_hi) kc_hi = h;
            }
            if (jj_lo >= jj_hi) continue;

            for (int kc = kc_lo; kc < kc_hi; ++kc) {
                const T *vp = Vs_lane + kc * K + jj_lo * A * C::PV;
                const T *up = Us_lane + kc * K + jj_lo * A * C::PU;
                // ring[n][s] holds right row (j - a) of matrix n in slot s = (j - a) mod A
                T ring[NU][A][K];
#pragma unroll
                for (int n = 0; n < NU; ++n)
#pragma unroll
                    for (int a = 1; a < A; ++a)
#pragma unroll
                        for (int q = 0; q < C::KVECS; ++q) {
                            vec r = *reinterpret_cast<const vec *>(up + n * C::UBAND - a * C::PU + q * VK);
#pragma unroll
                            for (int e = 0; e < VK; ++e) ring[n][(A - a) % A][q * VK + e] = r[e];
                        }
#pragma unroll 1
                for (int jj = jj_lo; jj < jj_hi; ++jj) {
#pragma unroll
                    for (int s = 0; s < A; ++s) {
#pragma unroll
                        for (int n = 0; n < NU; ++n)
#pragma unroll
                            for (int q = 0; q < C::KVECS; ++q) {
                                vec r = *reinterpret_cast<const vec *>(up + n * C::UBAND + s * C::PU + q * VK);
#pragma unroll
                                for (int e = 0; e < VK; ++e) ring[n][s][q * VK + e] = r[e];
                            }
                        T vw[NV][C::VWIN_VECS * VK];
#pragma unroll
                        for (int i = 0; i < NV; ++i)
#pragma unroll
                            for (int q = 0; q < C::VWIN_VECS; ++q) {
                                vec r = *reinterpret_cast<const vec *>(vp + i * C::VBAND + s * C::PV + q * VK);
#pragma unroll
                                for (int e = 0; e < VK; ++e) vw[i][q * VK + e] = r[e];
                            }
#pragma unroll
                        for (int k = 0; k < K; ++k)
#pragma unroll
                            for (int i = 0; i < NV; ++i)
#pragma unroll
                                for (int n = 0; n < NU; ++n)
#pragma unroll
                                    for (int a = 0; a < A; ++a)
#pragma unroll
                                        for (int b = 0; b < B; ++b)
                                            acc[i][n][a][b] += vw[i][b + k] * ring[n][(s - a + A) % A][k];
                    }
                    vp += A * C::PV;
                    up += A * C::PU;
                }
            }
        }
    }

    // ---- write the register tiles ----
    const int Sx = 2 * W - 1, Sy = 2 * H - 1;
    const size_t out_area = (size_t)Sx * Sy;
    const int ox0 = sxw + lx * B + (W - 1);
    const int oy0 = syw + ly * A + (H - 1);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = v_first + lv * NV + i;
        if (v >= g.nV) continue;
#pragma unroll
        for (int n = 0; n < NU; ++n) {
            const int u = u_first + lu * NU + n;
            if (u >= u_limit) continue;
            const size_t mat_index = g.group_m > 0 ? (size_t)u : (size_t)v * g.nU + u;
            T *o = g.out + mat_index * out_area;
#pragma unroll
            for (int a = 0; a < A; ++a) {
                const int oy = oy0 + a;
                if (oy < 0 || oy >= Sy) continue;
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    const int ox = ox0 + b;
                    if (ox < 0 || ox >= Sx) continue;
                    T *p = o + (size_t)oy * Sx + ox;
                    if (g.atomic)
                        atomic_add(p, acc[i][n][a][b]);
                    else
                        *p = acc[i][n][a][b];
                }
            }
        }
    }
}

// fills n elements with zero (a plain kernel rather than a memset node, so callers may capture it)
template <typename T>
__global__ void zero_fill_kernel(T *p, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = T(0);
}

} // namespace xcorr

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
//     LDS, zero padded, so the inner loop has no bounds checks; its wavefronts either own
//     adjacent shift tiles (WX x WY) or share one tile and split its reduction (WZ);
//   * per left row and K right columns a lane reads one B+K-1 wide left window and
//     one new right row of K values; the A right rows it needs are kept in a
//     register ring that rotates by one row per step (the y loop is unrolled so every
//     ring index is static), and every LDS read is issued one step ahead of its use. That is
//     NV*NU*A*B*K FMAs for NV*ceil((B+K-1)/v) + NU*ceil(K/v) 128-bit LDS reads (v = 16 / sizeof(T));
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
    int dist;           // 0 none, 1 rectangle, 2 triangle, 3 triangle by levels (how worker ids map to (y tile, chunk))
    int atomic;         // 1: atomicAdd partial sums into a zeroed output
    int ntx, nty;       // number of block tiles in x and y
    int nworkers_y;     // number of (y tile, chunk) workers
    int nvg, nug;       // left / right matrix groups
    int total_items;    // nvg * nug * nworkers_y * ntx * x_chunks
    int x_chunks;       // >1: the right columns a tile overlaps are cut into chunks of x_chunk_cols (atomic adds)
    int x_chunk_cols;   // multiple of K * WZ
    // Work queues of a persistent launch (matrix-core sweep): block b belongs to queue b % queues and takes item b first, then
    // the items b % queues + gridDim.x + queues * k for the k it draws from its queue's counter (one counter for all blocks
    // is drawn from a thousand times at once when equal work items end together, and the memory system serves one address
    // at some tens of nanoseconds per draw: 39 -> 28 microseconds for a launch of 1280 equal items). Queue i's counter is
    // queue[32 i] (128 bytes apart), queue[32 i + 1] counts its blocks that are done; all are zero before the launch and the
    // last block of a queue zeroes its pair again.
    // nullptr: block b takes the items b, b + gridDim.x, ... (with one block per work item: exactly one).
    int queues;
    // Ordered accumulation (matrix-core sweep, dist 3): tickets[tile] is the chunk of the tile that may add itself to the output
    // next. Chunk 0 stores, chunk c waits for tickets[tile] == c, adds itself to what is there and passes the ticket on; the last
    // chunk leaves 0. The sums of a tile are thus always formed in chunk order: the same bits every run, no atomic adds, no
    // cleared output. All zero before the launch. nullptr: off.
    unsigned *tickets;
    unsigned *queue;
};

// WZ_ > 1: the WZ_ wavefronts of a workgroup (WX_ = WY_ = 1) work on the SAME tile of shifts and
// matrices and split the reduction: a stage holds WZ_ (or a multiple) chunks of K columns, staged
// by all threads together, and wavefront w sweeps the chunks kc = w (mod WZ_) over all rows of
// the stage. The wavefronts do the same amount of work per stage, so the barriers around a stage
// cost little (wavefronts that own different shift tiles skip different parts of a stage and
// wait for each other), the block tile is as small as the wavefront tile (less work on partial
// overlaps), and the longest work item of a launch is WZ_ times shorter. The partial sums are
// added through LDS before the tile is written (or atomically added, once per block, when the
// reduction is also split over work items).
// SB_: 128-bit pieces a thread loads from global memory before it writes the first of them to LDS when staging a band set.
// DB_ = 1: two sets of LDS bands. While the wavefronts sweep one, the next stage is copied into the
// other by the memory pipeline itself (loads that write LDS directly, no registers, no waiting
// wavefront), and one barrier per stage is enough.
// PG_ = 1 ("paired groups"): the tile serves requests with group_m > 0 only and lays its LV_ lanes over left matrices that
// each bring their OWN group of right matrices: lane (lv, lu) pairs left matrix v_first + lv with right matrix
// (v_first + lv) * group_m + ug * LU_ * NU_ + lu * NU_ + n, so the block holds LV_ left bands and LV_ * LU_ * NU_ right bands.
// With one right matrix per left matrix (independent pairs) no other tile can lay lanes over matrices at all.
template <typename T, int A_, int B_, int K_, int NV_, int NU_, int LX_, int LY_, int LV_, int LU_, int WX_, int WY_,
          int RL_, int KBX_, int MINB_, int WZ_ = 1, int DB_ = 0, int SB_ = 8, int PG_ = 0>
struct EngineCfg {
    using value_type = T;
    static constexpr int MFMA = 0; // (1: the matrix-core sweep of engine_mfma.hpp, a configuration type of its own)
    static constexpr int A = A_, B = B_, K = K_, NV = NV_, NU = NU_;
    static constexpr int LX = LX_, LY = LY_, LV = LV_, LU = LU_;
    static constexpr int WX = WX_, WY = WY_, RL = RL_, KBX = KBX_, MINB = MINB_, WZ = WZ_, DB = DB_, SB = SB_, PG = PG_;
    static constexpr int VK = 16 / (int)sizeof(T); // elements per 128-bit LDS access
    static constexpr int TXW = LX * B, TYW = LY * A; // wavefront tile (shifts)
    static constexpr int TXB = TXW * WX, TYB = TYW * WY; // block tile (shifts)
    static constexpr int NWAVES = WX * WY * WZ, NT = 64 * NWAVES;
    static constexpr int G = A + 1; // left rows per unrolled group = slots of the right-row ring
    static constexpr int VWIN = B + K - 1;
    static constexpr int VWIN_VECS = (VWIN + VK - 1) / VK;
    static constexpr int KVECS = K / VK;
    static constexpr int NVB = LV * NV;              // left matrices per block
    static constexpr int NUL = LU * NU;              // right matrices per block that one left matrix meets
    static constexpr int NUB = PG ? NVB * NUL : NUL; // right bands per block
    // LDS geometry (elements)
    static constexpr int PV = TXB - B + KBX - K + VWIN_VECS * VK;
    // Band sizes are padded to an odd number of 128-bit pieces: lanes laid over matrices read
    // the same row and column of different bands in one instruction, and an odd stride puts
    // eight such reads on eight different groups of four LDS banks.
    static constexpr int odd_pieces(int n) { return ((n / VK) % 2) ? n : n + VK; }
    // Left bands, when lanes are laid over left matrices: an LDS pass serves 16 consecutive lanes, i.e. all LX x
    // positions of up to 16 / LX left bands, and their 128-bit window reads must fall on 16 different groups of four
    // banks: the pieces lv * (NV * band) + lx * (B / VK) must differ modulo 16. The smallest band size at or above
    // the rows it has to hold that achieves this is taken (the odd size alone left two-way conflicts on the tiles
    // with two x lanes: 37 % of the LDS cycles of the fp64 pair tile).
    static constexpr bool left_reads_collide(int band_elems) {
        bool seen[16] = {};
        const int combos = LX * LV < 16 ? LX * LV : 16;
        for (int c = 0; c < combos; ++c) {
            const int lx = c % LX, lv = (c / LX) % LV;
            const int piece = (lv * NV * (band_elems / VK) + lx * (B / VK)) % 16;
            if (seen[piece]) return true;
            seen[piece] = true;
        }
        return false;
    }
    static constexpr int left_band(int n) {
        if (LV > 1 && LX * (B / VK) <= 16)
            for (int extra = 0; extra < 16; ++extra)
                if (!left_reads_collide(n + extra * VK)) return n + extra * VK;
        return odd_pieces(n);
    }
    static constexpr int VBAND = left_band((RL + 1) * PV); // one spare row: the last step prefetches past the stage
    static constexpr int RU = RL + TYB - 1;
    static constexpr int PU = KBX + VK;
    static constexpr int UBAND = odd_pieces((RU + 1) * PU);
    static constexpr int LDS_ELEMS = NVB * VBAND + NUB * UBAND;
    // in-block reduction: one output row of the tile per wavefront and pass, [owner][source][lane][RED_ROW]
    static constexpr int RED_ROW = NV * NU * B;
    static constexpr int RED_ELEMS = WZ > 1 ? WZ * WZ * 64 * RED_ROW : 0;
    static constexpr int LDS_BUFFERS = DB ? 2 : 1;
    static constexpr int LDS_BYTES = (LDS_ELEMS * LDS_BUFFERS > RED_ELEMS ? LDS_ELEMS * LDS_BUFFERS : RED_ELEMS) * (int)sizeof(T);
    static_assert(LX * LY * LV * LU == 64, "lane layout must cover one wavefront");
    static_assert(!PG || NV == 1, "paired groups: one left matrix per lane");
    static_assert(WZ == 1 || (WX == 1 && WY == 1 && (A % WZ == 0 || A < WZ)), "wavefronts that split a reduction share one wavefront tile");
    static_assert((KBX / K) % WZ == 0, "every wavefront gets the same number of column chunks per stage");
    static_assert(B % VK == 0 && K % VK == 0 && KBX % K == 0 && RL % G == 0, "tile alignment");
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

// What one workgroup works on: a block tile of shifts, a group of matrices, a chunk of left rows and (when the columns
// are cut) a chunk of right columns.
struct WorkItem {
    int tile, chunk, chunks;       // which tile of the launch (matrix group, x tile, y tile), which chunk of its rows, of how many
    int clo, chi;                  // left rows [clo, chi)
    int syb, sxb;                  // first y / x shift of the block tile
    int v_first, u_first, u_limit; // first left matrix, first right matrix, end of the right matrices this left group meets
    int xr_lo, xr_hi, w_hi;        // right columns [xr_lo, xr_hi) to reduce over; w_hi bounds what a partial last stage may sweep
};

// Decodes work item number `item` (in launch order); false when there is nothing to do for it (surplus workers of the rectangle
// distribution, column chunks beyond a narrow tile's overlap). C supplies the block tile (TXB, TYB), the matrices per
// block (NVB, NUL, NUB) and the column granule K.
template <class C, typename T>
__device__ __forceinline__ bool decode_work_item(const EngineArgs<T> &g, int item, WorkItem &wi) {
    const int W = g.W, H = g.H;
    if (item >= g.total_items) return false;
    const int xch = item % g.x_chunks;
    item /= g.x_chunks;
    const int mat = item % (g.nvg * g.nug);
    item /= (g.nvg * g.nug);
    const int rc = g.rows_per_chunk;
    // (by levels: `item` numbers (level, x tile, y tile of the level), decoded below)
    const int worker = g.dist == 3 ? item : item % g.nworkers_y;
    int txi = g.dist == 3 ? 0 : item / g.nworkers_y;
    const int ug = mat % g.nug, vg = mat / g.nug;
    // x and y tiles are visited centre-out: the block index order is the dispatch order, and
    // central tiles have the longest overlaps, so the longest work items start first
    const int txc = g.ntx / 2, tyc = g.nty / 2;

    int tyi, chunk;
    if (g.dist == 0) {
        tyi = worker;
        chunk = 0;
    } else if (g.dist == 1) {
        tyi = worker % g.nty;
        chunk = worker / g.nty;
    } else if (g.dist == 3) {
        // by levels: first chunk 0 of every tile of the launch (x tiles slowest, y tiles fastest, as in the other orders), then
        // chunk 1 of the tiles that have one, ... - a tile's chunks lie a whole level of the launch apart in launch order, so
        // that one has long finished when the next wants to add itself on top (ordered accumulation).
        // The y tiles with more than R rows are those from R / TYB to (2H - 2 - R) / TYB.
        int w = worker, R = 0;
        chunk = 0;
        tyi = -1;
        for (; R < H; ++chunk, R += rc) {
            const int lo = R / C::TYB;
            int hi = (2 * H - 2 - R) / C::TYB;
            if (hi > g.nty - 1) hi = g.nty - 1;
            const int n = hi - lo + 1;
            if (n <= 0) continue;
            if (w < n * g.ntx) {
                txi = w / n;
                tyi = lo + w % n;
                break;
            }
            w -= n * g.ntx;
        }
        if (tyi < 0) return false;
    } else {
        int w = worker;
        tyi = 0;
        for (; tyi < g.nty; ++tyi) {
            int lo, hi;
            tile_rows<C>((tyi & 1) ? tyc - (tyi + 1) / 2 : tyc + tyi / 2, H, lo, hi);
            int n = (hi - lo + rc - 1) / rc;
            if (w < n) break;
            w -= n;
        }
        chunk = w;
        if (tyi >= g.nty) return false;
    }
    const int tx = (txi & 1) ? txc - (txi + 1) / 2 : txc + txi / 2;
    // (by levels the y tiles are taken in ascending order: all chunks of a level are equally long)
    const int ty = g.dist == 3 ? tyi : (tyi & 1) ? tyc - (tyi + 1) / 2 : tyc + tyi / 2;
    int row_lo, row_hi;
    tile_rows<C>(ty, H, row_lo, row_hi);
    wi.tile = (mat * g.ntx + tx) * g.nty + ty;
    wi.chunk = chunk;
    wi.chunks = (row_hi - row_lo + rc - 1) / rc;
    wi.clo = row_lo + chunk * rc;
    wi.chi = wi.clo + rc;
    if (wi.chi > row_hi) wi.chi = row_hi;
    if (wi.clo >= wi.chi) return false; // surplus worker of the rectangle distribution

    wi.syb = -(H - 1) + ty * C::TYB;
    wi.sxb = -(W - 1) + tx * C::TXB;

    // matrices of this block
    wi.v_first = vg * C::NVB;
    if (g.group_m > 0) {
        // (paired groups: of lane lv = 0; left matrix v_first + lv owns the same slice of its own group, group_m further on)
        wi.u_first = wi.v_first * g.group_m + ug * C::NUL;
        wi.u_limit = (wi.v_first + 1) * g.group_m;
    } else {
        wi.u_first = ug * C::NUB;
        wi.u_limit = g.nU;
    }

    // right columns with any overlap for this block tile, from the first K-column chunk that has some on: the first
    // stage then starts with useful chunks for all wavefronts that split it (aligned to the staging width instead,
    // the first and the last stage of a tile were both partly empty)
    int xr_lo = -(wi.sxb + C::TXB - 1);
    if (xr_lo < 0) xr_lo = 0;
    xr_lo = (xr_lo / C::K) * C::K;
    int xr_hi = W - wi.sxb;
    if (xr_hi > W) xr_hi = W;
    // this work item's chunk of those columns: [xr_lo, xr_hi) shrinks to it, and w_hi (= W when the
    // columns are not cut) bounds the columns a partial last stage may sweep
    wi.w_hi = W;
    if (g.x_chunks > 1) {
        const int lo = xr_lo + xch * g.x_chunk_cols;
        int hi = lo + g.x_chunk_cols;
        if (hi > xr_hi) hi = xr_hi;
        if (lo >= hi) return false; // the tile overlaps fewer columns than the widest one
        xr_lo = lo;
        xr_hi = hi;
        wi.w_hi = hi;
    }
    wi.xr_lo = xr_lo;
    wi.xr_hi = xr_hi;
    return true;
}

// Fills the LDS image of NB bands (ROWS rows of PITCH elements, BAND elements apart) from NB
// matrices that are `mat_stride` elements apart in global memory. Image element (band, row, col)
// is src[band][row0 + row][col0 + col] if band < nbands, row_lo <= row < row_hi and
// col_lo <= col < col_hi, and zero otherwise (the caller passes ranges that keep the reads
// inside the matrices). Every thread moves 128-bit pieces; the loads of up to eight pieces are
// issued back to back before the first LDS write (C::SB of them), so their latencies overlap.
// (The bands come in groups of NBL: band b is matrix src + (b / NBL) * group_stride + (b % NBL) * mat_stride and exists if
// b % NBL < nbands and b / NBL < ngroups; a single group when NBL == NB.)
template <class C, int NB, int NBL, int ROWS, int PITCH, int BAND>
__device__ __forceinline__ void stage_bands(typename C::value_type *lds, const typename C::value_type *src, size_t mat_stride,
                                            size_t group_stride, int W, int nbands, int ngroups, int row_lo, int row_hi, int row0,
                                            int col0, int col_lo, int col_hi, int tid) {
    using T = typename C::value_type;
    using vec = typename vec128<T>::type;
    constexpr int VK = C::VK, PP = PITCH / VK, TOTP = NB * ROWS * PP;
    constexpr int ITER = (TOTP + C::NT - 1) / C::NT;
    constexpr int BATCH = ITER < C::SB ? ITER : C::SB;
    static_assert(PITCH % VK == 0 && BAND % VK == 0, "128-bit LDS pieces");
#pragma unroll
    for (int it0 = 0; it0 < ITER; it0 += BATCH) {
        vec val[BATCH];
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
            const int p = tid + (it0 + j) * C::NT;
            const int col = (p % PP) * VK, row = (p / PP) % ROWS, band = p / (PP * ROWS);
            vec v;
#pragma unroll
            for (int e = 0; e < VK; ++e) v[e] = T(0);
            if (it0 + j < ITER && band % NBL < nbands && band / NBL < ngroups && row >= row_lo && row < row_hi && col + VK > col_lo && col < col_hi) {
                const T *q = src + (size_t)(band / NBL) * group_stride + (size_t)(band % NBL) * mat_stride + (size_t)(row0 + row) * W +
                             (ptrdiff_t)(col0 + col);
                if (col >= col_lo && col + VK <= col_hi) {
                    __builtin_memcpy(&v, q, sizeof(vec)); // element-aligned only
                } else {
#pragma unroll
                    for (int e = 0; e < VK; ++e)
                        if (col + e >= col_lo && col + e < col_hi) v[e] = q[e];
                }
            }
            val[j] = v;
        }
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
            const int p = tid + (it0 + j) * C::NT;
            const int col = (p % PP) * VK, row = (p / PP) % ROWS, band = p / (PP * ROWS);
            if (it0 + j < ITER && p < TOTP) *reinterpret_cast<vec *>(lds + band * BAND + row * PITCH + col) = val[j];
        }
    }
}

// Lane i of the wavefront copies the 16 bytes at its own global address to LDS address
// lds_wave_base + 16 * i, without passing through registers; completion is counted by vmcnt.
// `lds_wave_base` must be the same for all lanes. The LDS address travels in M0; the compiler
// builtin is used (not inline assembly) so that the compiler writes M0 itself and keeps the wait
// state the hardware needs between an SALU write of M0 and the LDS-DMA instruction that reads it.
// The compiler does not order ordinary LDS reads after this copy: callers wait (dma_wait) and
// pass a barrier before anything reads the destination.
__device__ __forceinline__ void dma16(const void *gptr, void *lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gptr,
                                     (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
}
__device__ __forceinline__ void dma_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// stage_bands with the copies done by dma16: pieces that lie fully inside the matrices are copied
// asynchronously, pieces outside are zeroed and pieces that straddle a matrix edge are assembled
// element by element with ordinary stores. The image is addressed linearly in 128-bit pieces
// (band * BAND/VK + row * PITCH/VK + column piece), which is what makes the 64 pieces of one
// wavefront-wide copy contiguous in LDS.
template <class C, int NB, int NBL, int ROWS, int PITCH, int BAND>
__device__ __forceinline__ void stage_bands_async(typename C::value_type *lds, const typename C::value_type *src, size_t mat_stride,
                                                  size_t group_stride, int W, int nbands, int ngroups, int row_lo, int row_hi, int row0,
                                                  int col0, int col_lo, int col_hi, int tid) {
    using T = typename C::value_type;
    using vec = typename vec128<T>::type;
    constexpr int VK = C::VK, PP = PITCH / VK, BANDP = BAND / VK, TOTP = NB * BANDP;
    constexpr int ITER = (TOTP + C::NT - 1) / C::NT;
    static_assert(PITCH % VK == 0 && BAND % VK == 0, "128-bit LDS pieces");
    // first 128-bit piece of this wavefront in iteration 0 (the same for all its lanes)
    const int wave_piece = __builtin_amdgcn_readfirstlane(tid & ~63);
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int p = tid + it * C::NT;
        const int band = p / BANDP, q = p % BANDP, row = q / PP, col = (q % PP) * VK;
        if (p < TOTP && row < ROWS) {
            const bool inside = band % NBL < nbands && band / NBL < ngroups && row >= row_lo && row < row_hi;
            const T *gp = src + (size_t)(band / NBL) * group_stride + (size_t)(band % NBL) * mat_stride + (ptrdiff_t)(row0 + row) * W +
                          (ptrdiff_t)(col0 + col);
            if (inside && col >= col_lo && col + VK <= col_hi) {
                dma16(gp, lds + (size_t)(wave_piece + it * C::NT) * VK);
            } else {
                // zero the piece, then patch in the elements of a piece that straddles an edge (the
                // patch is kept apart from the zeroing so that only it waits for its loads)
                vec zero;
#pragma unroll
                for (int e = 0; e < VK; ++e) zero[e] = T(0);
                *reinterpret_cast<vec *>(lds + (size_t)p * VK) = zero;
                if (inside && col + VK > col_lo && col < col_hi) {
#pragma unroll
                    for (int e = 0; e < VK; ++e)
                        if (col + e >= col_lo && col + e < col_hi) lds[(size_t)p * VK + e] = gp[e];
                }
            }
        }
    }
}

// Inner loops of one stage for one lane: for every K-column chunk kc in [kc_lo, kc_hi) sweep
// the staged left rows from `row0` on: `groups` groups of G rows and `tail` (< G) more rows after
// them. (The sweep starts at the first row that can overlap this wavefront's shifts, not at a
// multiple of G: on small matrices the rows before it were a tenth of the work.)
//
// Register plan per lane: NV*NU*A*B accumulators, a ring of G = A+1 right rows (row j in
// slot j mod G, so the row of the next step is fetched while the current step still uses
// all A of its rows) and ONE left window that is refilled in place: the FMAs of a step walk
// the window element by element (anti-diagonals b + k = e of the B x K product grid), and
// as soon as the last element of a 128-bit piece has been consumed the same piece of the
// next row is requested. Every LDS read is thus in flight for at least half a step of FMAs
// before its first use, without a second window buffer (which would push the tile past
// 128 VGPRs and below four wavefronts per SIMD).
template <class C>
__device__ __forceinline__ void compute_stage(const typename C::value_type *Vs_lane, const typename C::value_type *Us_lane,
                                              typename C::value_type (&acc)[C::NV][C::NU][C::A][C::B], int kc_lo,
                                              int kc_hi, int row0, int groups, int tail) {
    using T = typename C::value_type;
    using vec = typename vec128<T>::type;
    constexpr int A = C::A, B = C::B, K = C::K, NV = C::NV, NU = C::NU, VK = C::VK, G = C::G;
    constexpr int VW = C::VWIN_VECS * VK;
    for (int kc = kc_lo; kc < kc_hi; kc += C::WZ) { // (kc_lo is this wavefront's first chunk)
        const T *vp = Vs_lane + kc * K + row0 * C::PV;
        const T *up = Us_lane + kc * K + row0 * C::PU;
        T ring[NU][G][K];
        T vw[NV][VW];
        // rows -(A-1) .. 0 of the right band, window of left row 0
#pragma unroll
        for (int n = 0; n < NU; ++n)
#pragma unroll
            for (int a = A - 1; a >= 0; --a)
#pragma unroll
                for (int q = 0; q < C::KVECS; ++q) {
                    vec r = *reinterpret_cast<const vec *>(up + n * C::UBAND - a * C::PU + q * VK);
#pragma unroll
                    for (int e = 0; e < VK; ++e) ring[n][(G - a) % G][q * VK + e] = r[e];
                }
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int q = 0; q < C::VWIN_VECS; ++q) {
                vec r = *reinterpret_cast<const vec *>(vp + i * C::VBAND + q * VK);
#pragma unroll
                for (int e = 0; e < VK; ++e) vw[i][q * VK + e] = r[e];
            }
        // `tail` left rows follow the full groups: the last group stops after them
        auto group = [&](int steps) __attribute__((always_inline)) {
#pragma unroll
            for (int s = 0; s < G; ++s) {
                if (s > 0 && s >= steps) break;
                // right row s+1 (at s = G-1: the first row of the next group, or the spare
                // row the bands keep at their end)
#pragma unroll
                for (int n = 0; n < NU; ++n)
#pragma unroll
                    for (int q = 0; q < C::KVECS; ++q) {
                        vec r = *reinterpret_cast<const vec *>(up + n * C::UBAND + (s + 1) * C::PU + q * VK);
#pragma unroll
                        for (int e = 0; e < VK; ++e) ring[n][(s + 1) % G][q * VK + e] = r[e];
                    }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < C::VWIN; ++e) {
#pragma unroll
                    for (int k = 0; k < K; ++k) {
                        const int b = e - k;
                        if (b < 0 || b >= B) continue;
#pragma unroll
                        for (int i = 0; i < NV; ++i)
#pragma unroll
                            for (int n = 0; n < NU; ++n)
#pragma unroll
                                for (int a = 0; a < A; ++a) acc[i][n][a][b] += vw[i][e] * ring[n][(s - a + G) % G][k];
                    }
                    if (e % VK == VK - 1 || e == C::VWIN - 1) {
                        // this 128-bit piece of the window is consumed: refill it from the next row
                        // (the scheduling fences keep the compiler from sinking the read down to
                        // its first use in the next step, which would expose the LDS latency)
                        const int q = e / VK;
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int i = 0; i < NV; ++i) {
                            vec r = *reinterpret_cast<const vec *>(vp + i * C::VBAND + (s + 1) * C::PV + q * VK);
#pragma unroll
                            for (int x = 0; x < VK; ++x) vw[i][q * VK + x] = r[x];
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        };
#pragma unroll 1
        for (int jj = 0; jj < groups; ++jj) {
            group(G);
            vp += G * C::PV;
            up += G * C::PU;
        }
        if (tail > 0) group(tail);
    }
}

template <class C>
__global__ __launch_bounds__(C::NT, C::MINB) void engine_kernel(EngineArgs<typename C::value_type> g) {
    using T = typename C::value_type;
    using vec = typename vec128<T>::type;
    constexpr int A = C::A, B = C::B, K = C::K, NV = C::NV, NU = C::NU, VK = C::VK;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int tid = (int)threadIdx.x;
    const int group = C::WZ > 1 ? __builtin_amdgcn_readfirstlane(tid >> 6) : 0; // which share of the column chunks
    T *Vs = reinterpret_cast<T *>(smem_raw);
    T *Us = Vs + C::NVB * C::VBAND;
    const int W = g.W, H = g.H;

    // ---- the work item (uniform over the threads that share it) ----
    WorkItem wi;
    if (!decode_work_item<C>(g, (int)blockIdx.x, wi)) return;
    const int clo = wi.clo, chi = wi.chi, syb = wi.syb, sxb = wi.sxb, v_first = wi.v_first, u_first = wi.u_first, u_limit = wi.u_limit;
    const int xr_lo = wi.xr_lo, xr_hi = wi.xr_hi, w_hi = wi.w_hi;

    // ---- lane coordinates ----
    const int lane = tid & 63;
    const int wave = C::WZ > 1 ? 0 : __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wx = wave % C::WX, wy = wave / C::WX;
    // x fastest, y slowest: the eight lanes an LDS access serves together then differ in what
    // selects the LEFT address (x, left matrix) and share the right-row address, or differ in
    // the right matrix only; rows that are a multiple of A apart (different y) would always
    // fall on the same banks
    const int lx = lane % C::LX;
    const int lv = (lane / C::LX) % C::LV;
    const int lu = (lane / (C::LX * C::LV)) % C::LU;
    const int ly = lane / (C::LX * C::LV * C::LU);
    const int sxw = sxb + wx * C::TXW; // first x shift of the wavefront tile
    const int syw = syb + wy * C::TYW;
    const T *Vs_lane = Vs + lv * NV * C::VBAND + wx * C::TXW + lx * B;
    const int lane_ru0 = C::TYB - 1 - (wy * C::TYW + ly * A);
    const T *Us_lane = Us + ((C::PG ? lv * C::NUL : 0) + lu * NU) * C::UBAND + lane_ru0 * C::PU;

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

    // Stages: bands of RL left rows (outer) times blocks of KBX right columns (inner).
    const int nxs = xr_hi > xr_lo ? (xr_hi - xr_lo + C::KBX - 1) / C::KBX : 0;
    const int nstages = nxs * ((chi - clo + C::RL - 1) / C::RL);

    // fills one set of bands with the stage at left rows [yl0, yl0+RL), right columns [x0, x0+KBX)
    auto stage = [&](T *buf, int yl0, int x0) __attribute__((always_inline)) {
        // left band: rows [yl0, yl0+RL), columns xl = x0 + sxb + col
        const int xbase = x0 + sxb;
        const int rows_ok = chi - yl0 < C::RL ? chi - yl0 : C::RL;
        const int nbv = g.nV - v_first < C::NVB ? g.nV - v_first : C::NVB;
        const int vc_lo = xbase < 0 ? -xbase : 0;
        const int vc_hi = W - xbase < C::PV ? W - xbase : C::PV;
        // right band: rows yr = yl0 - syb - TYB + 1 + row, columns xr = x0 + col
        const int yr0 = yl0 - syb - C::TYB + 1;
        const int nbu = u_limit - u_first < C::NUL ? u_limit - u_first : C::NUL;
        // paired groups: one group of right bands per left matrix of the block, group_m matrices apart
        const int ngu = C::PG ? nbv : 1;
        const size_t gstride = C::PG ? (size_t)g.group_m * HW : 0;
        const int ur_lo = yr0 < 0 ? -yr0 : 0;
        const int ur_hi = H - yr0 < C::RU + 1 ? H - yr0 : C::RU + 1;
        const int uc_hi = W - x0 < C::KBX ? W - x0 : C::KBX;
        T *ubuf = buf + C::NVB * C::VBAND;
        if constexpr (C::DB) {
            stage_bands_async<C, C::NVB, C::NVB, C::RL + 1, C::PV, C::VBAND>(buf, g.V + (size_t)v_first * HW, HW, 0, W, nbv, 1, 0, rows_ok, yl0,
                                                                             xbase, vc_lo, vc_hi, tid);
            stage_bands_async<C, C::NUB, C::NUL, C::RU + 1, C::PU, C::UBAND>(ubuf, g.U + (size_t)u_first * HW, HW, gstride, W, nbu, ngu, ur_lo, ur_hi,
                                                                             yr0, x0, 0, uc_hi, tid);
        } else {
            stage_bands<C, C::NVB, C::NVB, C::RL + 1, C::PV, C::VBAND>(buf, g.V + (size_t)v_first * HW, HW, 0, W, nbv, 1, 0, rows_ok, yl0, xbase,
                                                                       vc_lo, vc_hi, tid);
            stage_bands<C, C::NUB, C::NUL, C::RU + 1, C::PU, C::UBAND>(ubuf, g.U + (size_t)u_first * HW, HW, gstride, W, nbu, ngu, ur_lo, ur_hi, yr0,
                                                                       x0, 0, uc_hi, tid);
        }
    };
    // this wavefront's part of a staged stage
    auto compute = [&](int buf_offset, int yl0, int x0) __attribute__((always_inline)) {
        // left rows of this stage that can overlap this wavefront's y shifts:
        // rows yl in [syw, syw + TYW - 1 + H - 1] and yl < chi
        int row0, nrows;
        {
            int first = syw - yl0;                 // first useful row index j
            int last = syw + C::TYW + H - 2 - yl0; // last useful row index j
            if (chi - 1 - yl0 < last) last = chi - 1 - yl0;
            if (last > C::RL - 1) last = C::RL - 1;
            row0 = first > 0 ? first : 0;
            nrows = last + 1 - row0;
        }
        // K-column chunks of this stage that overlap this wavefront's x shifts: need
        // (x0 + kc*K + K-1) + (sxw + TXW-1) >= 0 and (x0 + kc*K) + sxw <= W-1 and x0 + kc*K < W
        int kc_lo = 0, kc_hi = C::KBX / K;
        {
            int need = -(sxw + C::TXW - 1) - (K - 1) - x0;
            if (need > 0) kc_lo = (need + K - 1) / K;
            int lim = W - 1 - sxw - x0;
            if (w_hi - 1 - x0 < lim) lim = w_hi - 1 - x0;
            int h = lim < 0 ? 0 : lim / K + 1;
            if (h < kc_hi) kc_hi = h;
        }
        if (C::WZ > 1) kc_lo += (group - kc_lo % C::WZ + C::WZ) % C::WZ; // this wavefront's chunks: kc = group (mod WZ)
        if (nrows > 0) compute_stage<C>(Vs_lane + buf_offset, Us_lane + buf_offset, acc, kc_lo, kc_hi, row0, nrows / C::G, nrows % C::G);
    };

    if constexpr (C::DB) {
        // stage s+1 is copied into one set of bands while stage s is swept in the other
        if (nstages > 0) stage(Vs, clo, xr_lo);
        int yl0 = clo, x0 = xr_lo; // stage being computed
        for (int st = 0; st < nstages; ++st) {
            dma_wait();
            __syncthreads(); // stage st has landed for everyone, and everyone is done with stage st-1
            int yl1 = yl0, x1 = x0 + C::KBX;
            if (x1 >= xr_hi) {
                x1 = xr_lo;
                yl1 += C::RL;
            }
            const int cur = (st & 1) * C::LDS_ELEMS;
            if (st + 1 < nstages) stage(Vs + (C::LDS_ELEMS - cur), yl1, x1);
            compute(cur, yl0, x0);
            yl0 = yl1;
            x0 = x1;
        }
    } else {
        for (int yl0 = clo; yl0 < chi; yl0 += C::RL) {
            for (int x0 = xr_lo; x0 < xr_hi; x0 += C::KBX) {
                __syncthreads(); // everyone is done reading the previous stage
                stage(Vs, yl0, x0);
                __syncthreads();
                compute(0, yl0, x0);
            }
        }
    }

    // ---- write the register tiles ----
    const int Sx = 2 * W - 1, Sy = 2 * H - 1;
    const size_t out_area = (size_t)Sx * Sy;
    const int ox0 = sxw + lx * B + (W - 1);
    const int oy0 = syw + ly * A + (H - 1);
    if (C::WZ > 1) {
        // Add the partial tiles of the WZ wavefronts. In pass q wavefront w ends up with the
        // sums of tile row q*WZ + w: everyone deposits rows q*WZ .. q*WZ+WZ-1, then reads back
        // all WZ versions of its own row (in wavefront order, so the result is deterministic).
        T *red = reinterpret_cast<T *>(smem_raw);
        constexpr int RR = C::RED_ROW;
        // tile rows summed per pass: one per wavefront, or a single one (by wavefront 0) when
        // the tile has fewer rows than the block has wavefronts
        constexpr int OWN = A % C::WZ == 0 ? C::WZ : 1;
#pragma unroll
        for (int q = 0; q < A / OWN; ++q) {
            __syncthreads(); // bands, or the previous pass, are no longer read
#pragma unroll
            for (int o = 0; o < OWN; ++o) {
                T *dst = red + ((size_t)(o * C::WZ + group) * 64 + lane) * RR;
#pragma unroll
                for (int i = 0; i < NV; ++i)
#pragma unroll
                    for (int n = 0; n < NU; ++n)
#pragma unroll
                        for (int b = 0; b < B; b += VK) {
                            vec piece;
#pragma unroll
                            for (int e = 0; e < VK; ++e) piece[e] = acc[i][n][q * OWN + o][b + e];
                            *reinterpret_cast<vec *>(dst + (i * NU + n) * B + b) = piece;
                        }
            }
            __syncthreads();
            if (group >= OWN) continue;
            T sum[NV][NU][B];
#pragma unroll
            for (int src = 0; src < C::WZ; ++src) {
                const T *from = red + ((size_t)(group * C::WZ + src) * 64 + lane) * RR;
#pragma unroll
                for (int i = 0; i < NV; ++i)
#pragma unroll
                    for (int n = 0; n < NU; ++n)
#pragma unroll
                        for (int b = 0; b < B; b += VK) {
                            vec piece = *reinterpret_cast<const vec *>(from + (i * NU + n) * B + b);
#pragma unroll
                            for (int e = 0; e < VK; ++e) sum[i][n][b + e] = src == 0 ? piece[e] : sum[i][n][b + e] + piece[e];
                        }
            }
            const int oy = oy0 + q * OWN + group;
            if (oy < 0 || oy >= Sy) continue;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = v_first + lv * NV + i;
                if (v >= g.nV) continue;
#pragma unroll
                for (int n = 0; n < NU; ++n) {
                    const int u = u_first + (C::PG ? lv * g.group_m : 0) + lu * NU + n;
                    if (u >= u_limit + (C::PG ? lv * g.group_m : 0)) continue;
                    const size_t mat_index = g.group_m > 0 ? (size_t)u : (size_t)v * g.nU + u;
                    T *o = g.out + mat_index * out_area + (size_t)oy * Sx;
#pragma unroll
                    for (int b = 0; b < B; ++b) {
                        const int ox = ox0 + b;
                        if (ox < 0 || ox >= Sx) continue;
                        if (g.atomic)
                            atomic_add(o + ox, sum[i][n][b]);
                        else
                            o[ox] = sum[i][n][b];
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = v_first + lv * NV + i;
        if (v >= g.nV) continue;
#pragma unroll
        for (int n = 0; n < NU; ++n) {
            const int u = u_first + (C::PG ? lv * g.group_m : 0) + lu * NU + n;
            if (u >= u_limit + (C::PG ? lv * g.group_m : 0)) continue;
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

// Matrix-core sweep for the grouped families of the sliding-window engine.
//
//   out[v,u][sy][sx] = sum over (yl, xr) of V_v[yl][xr+sx] * U_u[yl-sy][xr]
//
// For ONE left row yl and a few right columns xr this is a small matrix product whose result does not move as yl and
// xr advance: D[i][j] += sum_k Ua[i][k] * Vb[k][j] with
//     i <-> (right matrix u_i, y shift sy_i):   Ua[i][k] = U_{u_i}[yl - sy_i][x_k]      (a window of right rows)
//     j <-> (left matrix v_j, x shift sx_j):    Vb[k][j] = V_{v_j}[yl][x_k + sx_j]      (a Hankel matrix of one left row)
// so the whole reduction over (yl, xr) accumulates into the same P x P result tile of v_mfma_f32_32x32x2_f32 (P = 32,
// two k slots), v_mfma_f32_16x16x4_f32 or v_mfma_f64_16x16x4_f64 (P = 16, four k slots). Nothing is multiplied that the definition does not
// multiply, except the zero padding at tile edges that the register-tile sweep has as well. The instructions run at
// the rate of the vector FMA peak (64 cycles each on this chip; the 16 x 16 fp32 one 32), but one stands for 2048 / 1024 FMAs: the
// LDS reads and address arithmetic around it weigh little (about two cycles of the matrix pipeline per other
// instruction issued on the SIMD), the shader clock stays at 2.35 GHz on data that holds the vector-FMA loop at 2.0-2.1,
// and operand reuse happens inside the matrix core instead of in registers: small shift tiles (many matrices per tile)
// cost nothing extra.
//
// Lane l of a wavefront (p = l % P, kk = l / P) supplies row i = p of Ua and column j = p of Vb for k slot kk. The k
// slots of the EV instructions of a step (4 for the fp32 tiles, 2 for the fp64 tile) are assigned
// x_k = x0 + EV * kk + e, e = 0 .. EV-1, so the right operand of a step is ONE aligned LDS read of EV elements per lane
// and the left operand EV consecutive elements. A step covers 8 right columns with every instruction (16 with the 16 x 16 fp32
// one). The work items
// (tiles, chunks of rows and columns, centre-out order), the zero-padded LDS bands and the four wavefronts of a block
// that share one tile are those of the register-tile sweep (engine.hpp); the staging by loads that write LDS directly
// (BandDma), the deal of a stage's steps to the wavefronts (mfma_stage, mfma_stage_fine) and the persistent blocks that take
// their work items from a queue (mfma_kernel) are this file's.
//
// Result layout of the instructions (lane l, accumulator element r): column j = l % P; row i = 8 * (r / 4) + 4 * (l / 32) + r % 4
// for the 32 x 32 fp32 instruction, i = 4 * (l / 16) + r for the 16 x 16 fp32 one and i = 4 * r + l / 16 for the fp64 one. The P lanes of a row are adjacent x shifts: 128-byte runs (two
// runs of 64 bytes in different result rows for the tiles whose columns hold the x shifts twice, see JYO_ below).
#pragma once

#include <type_traits>

#include "engine.hpp"

namespace xcorr {

// The instruction of an element type and the layout of its result tile. FINE = 1 takes the smaller fp32 instruction (half the FMAs per
// instruction at the same rate per cycle): tiles of 16 x 16 shifts for the sweep that trims every result tile to its own overlap.
template <typename T, int FINE = 0>
struct MfmaOp;
template <>
struct MfmaOp<float, 0> {
    typedef float acc_t __attribute__((ext_vector_type(16)));
    static constexpr int P = 32, ACC = 16, EV = 4;
    static constexpr int REG_BITS = 0b11011, LANE_BITS = 0b00100; // which bits of a result row come from the element index / the lane
    static __device__ __forceinline__ int row(int r, int kk) { return 8 * (r / 4) + 4 * kk + r % 4; } // of element r in lanes l / P = kk
    static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
};
template <>
struct MfmaOp<float, 1> { // v_mfma_f32_16x16x4_f32: 32 cycles, four k slots; element r of lanes l / 16 = kk is result row 4 kk + r
    typedef float acc_t __attribute__((ext_vector_type(4)));
    static constexpr int P = 16, ACC = 4, EV = 4;
    static constexpr int REG_BITS = 0b0011, LANE_BITS = 0b1100;
    static __device__ __forceinline__ int row(int r, int kk) { return 4 * kk + r; }
    static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
};
template <>
struct MfmaOp<double, 0> {
    typedef double acc_t __attribute__((ext_vector_type(4)));
    static constexpr int P = 16, ACC = 4, EV = 2;
    static constexpr int REG_BITS = 0b1100, LANE_BITS = 0b0011;
    static __device__ __forceinline__ int row(int r, int kk) { return 4 * r + kk; }
    static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
};
template <>
struct MfmaOp<double, 1> : MfmaOp<double, 0> {};

constexpr int popcount_c(int x) { return x == 0 ? 0 : (x & 1) + popcount_c(x >> 1); }

// JV_ / IU_: left / right matrices laid over the columns / rows of one result tile (P / JV_ x shifts, P / IU_ y shifts).
// MJX_ x MJV_ result tiles per wavefront along x shifts / further left matrices, NIY_ x NIU_ along y shifts / further
// right matrices: the wavefront holds MJX_ * MJV_ * NIY_ * NIU_ result tiles and every operand it reads feeds
// NIY_ * NIU_ (left) or MJX_ * MJV_ (right) instructions.
// NC_: accumulator sets per result tile. The VK instructions of a step that feed one result tile form a dependent chain;
// with NC_ > 1 they alternate between NC_ sets that are added up at the end, so a wavefront with few result tiles still
// has independent instructions in flight (measured on the one-tile fp32 sweep: 0.89 -> 0.96 of the instruction's peak).
// JYO_: copies of the x shifts of a result tile's columns, IY left rows apart: column j <-> (copy c_j, x shift sx_j) reads
// Vb[k][j] = V[yb + c_j * IY][x_k + sx_j] while row i reads U[yb - sy_i][x_k], so the tile holds the y shifts sy_i + c_j * IY:
// P / JYO_ x shifts by IY * JYO_ y shifts of one left matrix instead of P by IY (a squarer tile sweeps fewer rows and columns that
// only some of its shifts overlap). The copies come from the same LDS band, IY rows further down: they cost (JYO_ - 1) * IY
// more rows per band and per chunk of left rows, no staging.
// FINE_: the sweep of a stage goes result tile by result tile of the wavefront, each over the rows and column steps that ITS shifts
// overlap, instead of all tiles over the union (mfma_stage_fine): the zeros a block multiplies at the edges of the matrices are those
// of a footprint of one result tile (P x P shifts), the work items (staging, epilogue, queue draws) those of the whole block tile.
// For launches whose matrices are small against the block tile and share nothing between pairs.
template <typename T, int JV_, int IU_, int MJX_, int MJV_, int NIY_, int NIU_, int RL_, int KBX_, int MINB_, int NC_ = 1, int WZ_ = 4, int JYO_ = 1,
          int FINE_ = 0>
struct MfmaCfg {
    using value_type = T;
    using Op = MfmaOp<T, FINE_>;
    static constexpr int MFMA = 1, PG = 0, DB = 0, FINE = FINE_;
    static constexpr int P = Op::P, ACC = Op::ACC, KS = 64 / P;
    static constexpr int VK = 16 / (int)sizeof(T);
    static constexpr int EV = Op::EV;   // consecutive elements a lane reads per operand and step = instructions per step and result tile
    static constexpr int K = KS * EV; // right columns per step (8)
    static constexpr int JV = JV_, JYO = JYO_, JX = P / (JV_ * JYO_), IU = IU_, IY = P / IU_;
    static constexpr int MJX = MJX_, MJV = MJV_, NIY = NIY_, NIU = NIU_;
    static constexpr int TJ = MJX * MJV, TI = NIY * NIU; // result tiles of a wavefront
    static constexpr int IYB = IY * NIY;                   // y shifts among the rows of the result tiles: the window of right rows of a left row
    static constexpr int TXB = JX * MJX, TYB = IYB * JYO, TXW = TXB, TYW = IYB;
    static constexpr int NVB = JV * MJV, NUL = IU * NIU, NUB = NUL;
    // (the copies of the x shifts are reported as half or quarter wavefronts along y)
    static constexpr int WX = 1, WY = JYO, WZ = WZ_, NWAVES = WZ, NT = 64 * NWAVES;
    static constexpr int RL = RL_, KBX = KBX_, MINB = MINB_, NC = NC_;
    // what the launch record and the planner call the tile: shifts and matrices per lane, lanes over each
    static constexpr int A = (1 << popcount_c(Op::REG_BITS & (IY - 1))) * NIY;
    static constexpr int B = MJX;
    static constexpr int NV = MJV;
    static constexpr int NU = (1 << popcount_c(Op::REG_BITS & ~(IY - 1) & (P - 1))) * NIU;
    static constexpr int LX = JX, LV = JV;
    static constexpr int LY = 1 << popcount_c(Op::LANE_BITS & (IY - 1));
    static constexpr int LU = 1 << popcount_c(Op::LANE_BITS & ~(IY - 1));
    // LDS geometry (elements). Left band: RL rows of every column a shift of the tile can meet in a stage.
    // (+ VK - 1: the band starts at the 128-bit boundary of the matrix row at or below its first column, see mfma_kernel)
    // The copies of the x shifts read rows IY apart with one instruction, P lanes a pass: with IY rows JX elements apart modulo
    // the P x 4 bytes (fp64: P x 8) those lanes touch, they fall on P consecutive banks like the lanes of a single row (measured
    // with IY rows a multiple of that apart: 0.35 conflict cycles per LDS cycle). No multiple of 128 bits does that for 8 rows:
    // such a band keeps its rows on 64-bit boundaries only and is filled with 64-bit LDS stores.
    static constexpr int BANK_ELEMS = 256 / (int)sizeof(T);
    static constexpr int PVC = (TXB + KBX - 1 + (VK - 1) + VK - 1) / VK * VK; // columns of a left band
    static constexpr int left_pitch() {
        int n = PVC;
        if (JYO > 1)
            while ((IY * n) % (P * (int)sizeof(T) / 4) != JX || (n * (int)sizeof(T)) % 8 != 0) n += 1;
        return n;
    }
    static constexpr int PV = left_pitch();
    static constexpr int VROWS = RL + (JYO - 1) * IY; // rows of a left band
    // Lanes p = 0 .. P-1 read element (left matrix p / JX, column p % JX) of one row with one instruction: with the bands
    // JX (modulo the 256 bytes of the banks) apart they fall on P consecutive banks like the lanes of a single matrix.
    static constexpr int left_band(int n) {
        if (JV == 1) return (n + VK - 1) / VK * VK;
        int b = n;
        while (b % BANK_ELEMS != JX % BANK_ELEMS) b += VK;
        return b;
    }
    static constexpr int VBAND = left_band((VROWS + 1) * PV); // one spare row: the sweep reads one row ahead
    // Right band: an LDS pass serves the reads of 32 consecutive lanes, and the EV-element pieces they touch must differ
    // modulo 32 (measured: one collision doubles the pass). Those lanes are rows p = 0 .. P-1 apart and, for the 16-row
    // tiles, two k slots one piece apart: the row pitch is an odd number of pieces (P = 32) or twice an odd number
    // (P = 16), and the bands of the IU matrices of a result tile continue the row sequence (band stride = -IY rows
    // modulo 32 pieces).
    static constexpr int RU = RL + IYB - 1;
    static constexpr int right_pitch() {
        int n = KBX + VK;
        while (n % VK != 0 || (P == 32 ? (n / EV) % 2 != 1 : (n / EV) % 4 != 2)) n += EV;
        return n;
    }
    static constexpr int PU = right_pitch();
    static constexpr int right_band(int n) {
        if (IU == 1) return n;
        int b = n;
        while ((b / EV) % 32 != (32 - (IY * (PU / EV)) % 32) % 32) b += VK;
        return b;
    }
    static constexpr int UBAND = right_band((RU + 1) * PU);
    static constexpr int LDS_ELEMS = NVB * VBAND + NUB * UBAND;
    // in-block reduction: per pass every wavefront ends up with one quad (four consecutive accumulator elements per lane)
    static constexpr int NQ = TJ * TI * ACC / 4;
    static constexpr int QP = WZ < 4 ? WZ : 4; // quads per pass (= wavefronts that add and write in a pass)
    static constexpr int RED_ELEMS = QP * WZ * 64 * 4;
    static constexpr int BAND_BYTES = (LDS_ELEMS > RED_ELEMS ? LDS_ELEMS : RED_ELEMS) * (int)sizeof(T);
    static constexpr int LDS_BYTES = BAND_BYTES + 16; // + two slots through which thread 0 hands the block its next work item
    static_assert(P % (JV * JYO) == 0 && P % IU == 0, "whole matrices per result tile");
    static_assert(FINE == 0 || (JYO == 1 && MJV == 1 && NIU == 1), "tile-by-tile sweep: the result tiles of a block differ in their shifts only");
    static_assert(JYO == 1 || (JV == 1 && NIY == 1), "copies of the x shifts: one left matrix per result tile, one tile along y");
    static_assert(EV % NC == 0, "the instructions of a step are dealt evenly to the accumulator sets");
    static_assert(WZ > 1 && (FINE != 0 ? KBX % K == 0 : (KBX / K) % WZ == 0), "every wavefront gets the same number of column chunks per stage");
    static_assert((PV % VK == 0 || JYO > 1) && VBAND % VK == 0 && UBAND % VK == 0, "128-bit LDS pieces");
    static_assert(LX * LY * LV * LU * WY == 64, "lane bookkeeping");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

// Staging of NB bands (ROWS rows x COLS columns each; row pitch PITCH and band stride BAND in LDS) by loads that write LDS
// directly (buffer_load ... lds: no registers, no LDS store instructions, completion counted by vmcnt). One such instruction
// moves GRAN bytes per lane to 64 consecutive pieces of LDS, so the image of a band is taken as a run of pieces
// q = 0 .. ROWS * PITCH / PE - 1 (PE elements each), piece q being (row, column) = (q / PP, (q % PP) * PE); lane l of copy j
// fetches piece 64 j + l. Every band has a buffer descriptor of its own that covers exactly the rows that may be read (the
// matrix, or the chunk of left rows of the work item): a piece of a row outside them has an offset below zero or beyond the
// descriptor's size and the hardware writes zeros for it - the zero padding above and below the matrices costs nothing. Left and
// right of the matrices the offset would fall into a neighbouring row: there (and only in stages that reach over the edge) the
// lane's column is compared and the offset replaced by one that is out of range. A piece that straddles the right edge (widths
// that are not a multiple of the piece) is loaded whole and its tail zeroed afterwards (fix_right_edge).
// Per lane and copy two registers are kept: byte offset and column of the piece relative to the stage origin. A wavefront copies
// the bands w, w + WZ, ... whole (NB a multiple of WZ), or the copies w, w + WZ, ... of the only band.
// GRAN = 4 (one fp32 element per lane) serves images whose rows are not 128 bits apart.
using buffer_rsrc = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ buffer_rsrc make_rsrc(const void *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), (short)0, (int)bytes, 0x00020000);
}
template <int GRAN>
__device__ __forceinline__ void dma_piece(buffer_rsrc r, void *lds_wave_base, unsigned voffset) {
    // (the size must be a literal for the builtin)
    if constexpr (GRAN == 16)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void *)lds_wave_base, 16, (int)voffset, 0, 0, 0);
    else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void *)lds_wave_base, 4, (int)voffset, 0, 0, 0);
    static_assert(GRAN == 16 || GRAN == 4, "piece sizes the instruction has");
}

template <class C, int NB, int ROWS, int COLS, int PITCH, int BAND, int GRAN>
struct BandDma {
    using T = typename C::value_type;
    static constexpr int EB = (int)sizeof(T);
    static constexpr int PE = GRAN / EB;        // elements per piece
    static constexpr int PP = PITCH / PE;       // pieces per image row
    static constexpr int Q = ROWS * PP;         // pieces of a band image (the spare row behind them is not loaded)
    static constexpr int J = (Q + 63) / 64;     // wavefront-wide copies per band
    static constexpr bool OWN = NB >= C::WZ;    // a wavefront copies whole bands
    static constexpr int NBW = OWN ? NB / C::WZ : 1;
    static constexpr int TJ = OWN ? J : (J + C::WZ - 1) / C::WZ;
    static constexpr unsigned OUTSIDE = 0x80000000u; // an offset no descriptor covers (a matrix has at most 2^31 bytes)
    static_assert(GRAN % EB == 0 && PITCH % PE == 0 && (BAND * EB) % GRAN == 0, "whole pieces");
    static_assert(NB == 1 || NB % C::WZ == 0, "bands per block: one, or a multiple of the wavefronts");
    static_assert(COLS <= PITCH, "image rows hold the columns");
    unsigned lane_off[TJ]; // (row * W + column) * EB of the lane's piece in copy t
    int lane_col[TJ];      // its first column; beyond the image's columns (padding of the pitch): a number no matrix is wide
    buffer_rsrc rsrc[NBW];

    // copy t of this wavefront is copy j of its band(s)
    __device__ __forceinline__ static int copy_index(int t, int wave) { return OWN ? t : wave + t * C::WZ; }

    __device__ __forceinline__ void init(int lane, int wave, int W) {
#pragma unroll
        for (int t = 0; t < TJ; ++t) {
            const int q = 64 * copy_index(t, wave) + lane;
            const int row = q / PP, col = (q % PP) * PE;
            lane_off[t] = (unsigned)((row * W + col) * EB);
            lane_col[t] = col < COLS ? col : (1 << 28);
        }
    }
    // The bands of a work item: band b is the matrix `first + b * mat_stride`, of which the rows [row_lo, row_lo + rows) exist
    // (the others read as zero); bands from `nbands` on do not exist.
    __device__ __forceinline__ void set_item(const T *first, size_t mat_stride, int W, int row_lo, int rows, int nbands, int wave) {
#pragma unroll
        for (int i = 0; i < NBW; ++i) {
            const int b = OWN ? wave + i * C::WZ : 0;
            rsrc[i] = make_rsrc(first + (size_t)b * mat_stride + (size_t)row_lo * W, b < nbands ? (unsigned)rows * (unsigned)W * EB : 0u);
        }
    }
    // Stage whose image row 0, column 0 is row `row0` (relative to row_lo of set_item), column `col0` of the matrices.
    template <bool CHECK>
    __device__ __forceinline__ void copy(T *lds, int W, int row0, int col0, int lane, int wave) const {
        const unsigned origin = (unsigned)(((long long)row0 * W + col0) * EB); // (modulo 2^32: a matrix has at most 2^31 bytes)
#pragma unroll
        for (int i = 0; i < NBW; ++i) {
            T *band = lds + (OWN ? wave + i * C::WZ : 0) * BAND;
#pragma unroll
            for (int t = 0; t < TJ; ++t) {
                const int j = copy_index(t, wave);
                if (!OWN && t == TJ - 1 && j >= J) continue; // (wavefront-uniform)
                unsigned voffset = lane_off[t] + origin;
                if (CHECK) voffset = (unsigned)(col0 + lane_col[t]) < (unsigned)W ? voffset : OUTSIDE;
                char *dst = reinterpret_cast<char *>(band) + j * 64 * GRAN;
                if (t == TJ - 1 && Q % 64 != 0) {
                    // the last copy of a band: lanes behind the image's end must not write (the next band starts there)
                    if (64 * j + lane < Q) dma_piece<GRAN>(rsrc[i], dst, voffset);
                } else {
                    dma_piece<GRAN>(rsrc[i], dst, voffset);
                }
            }
        }
    }
    __device__ __forceinline__ void stage(T *lds, int W, int row0, int col0, int lane, int wave) const {
        // (with the padding of the pitch inside the matrix too, no lane needs its column checked)
        if (col0 >= 0 && col0 + PITCH <= W)
            copy<false>(lds, W, row0, col0, lane, wave);
        else
            copy<true>(lds, W, row0, col0, lane, wave);
    }
    // After the copies have landed: a piece that begins inside the matrix and ends beyond its last column has brought the
    // first elements of the next row along; they become the zeros that belong there. Only for widths that are not a multiple of
    // the piece, in stages that hold the last column.
    __device__ __forceinline__ void fix_right_edge(T *lds, int W, int col0, int lane, int wave) const {
        if (PE == 1 || W % PE == 0 || col0 + COLS <= W) return;
#pragma unroll
        for (int i = 0; i < NBW; ++i) {
            T *band = lds + (OWN ? wave + i * C::WZ : 0) * BAND;
#pragma unroll
            for (int t = 0; t < TJ; ++t) {
                const int j = copy_index(t, wave);
                const int q = 64 * j + lane, col = col0 + lane_col[t];
                if (q < Q && j < J && col < W && col + PE > W) {
#pragma unroll
                    for (int e = 1; e < PE; ++e)
                        if (col + e >= W) band[q * PE + e] = T(0);
                }
            }
        }
    }
};

// One band (ROWS rows x COLS columns, row pitch PITCH) whose image rows are only 64 bits apart in LDS - the left band of the tiles
// with copies of the x shifts - goes through registers: 128-bit buffer loads with the same descriptor (rows outside the work
// item's read as zero), two 64-bit LDS stores per piece. The band starts at any column: in stages that reach over the left or
// right edge of the matrix a piece may lie partly outside, and its elements are zeroed one by one before they are stored.
template <class C, int ROWS, int COLS, int PITCH>
struct BandLoad {
    using T = typename C::value_type;
    using vec = typename vec128<T>::type;
    static constexpr int EB = (int)sizeof(T), VK = C::VK, PPC = COLS / VK, TOT = ROWS * PPC, ITER = (TOT + C::NT - 1) / C::NT;
    static constexpr unsigned OUTSIDE = 0x80000000u;
    static_assert(COLS % VK == 0 && (PITCH * EB) % 8 == 0 && VK == 4, "pieces of four elements, rows on 64-bit boundaries");
    unsigned lane_off[ITER];
    int lane_col[ITER];
    int lds_at[ITER]; // element offset in the image
    buffer_rsrc rsrc;
    __device__ __forceinline__ void init(int tid, int W) {
#pragma unroll
        for (int i = 0; i < ITER; ++i) {
            const int p = tid + i * C::NT;
            const int row = p / PPC, col = (p % PPC) * VK;
            lane_off[i] = (unsigned)((row * W + col) * EB);
            lane_col[i] = col;
            lds_at[i] = row * PITCH + col;
        }
    }
    __device__ __forceinline__ void set_item(const T *first, int W, int row_lo, int rows, int nbands) {
        rsrc = make_rsrc(first + (size_t)row_lo * W, nbands > 0 ? (unsigned)rows * (unsigned)W * EB : 0u);
    }
    template <bool CHECK>
    __device__ __forceinline__ void copy(T *lds, int W, int row0, int col0, int tid) const {
        typedef unsigned uvec __attribute__((ext_vector_type(4)));
        typedef T half_t __attribute__((ext_vector_type(VK / 2)));
        const unsigned origin = (unsigned)(((long long)row0 * W + col0) * EB); // (modulo 2^32: a matrix has at most 2^31 bytes)
        uvec val[ITER];
#pragma unroll
        for (int i = 0; i < ITER; ++i) {
            if ((i + 1) * C::NT > TOT && tid + i * C::NT >= TOT) continue;
            unsigned voffset = lane_off[i] + origin;
            if (CHECK) {
                const int cs = col0 + lane_col[i];
                voffset = cs > -VK && cs < W ? voffset : OUTSIDE;
            }
            val[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voffset, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < ITER; ++i) {
            if ((i + 1) * C::NT > TOT && tid + i * C::NT >= TOT) continue;
            vec v;
            __builtin_memcpy(&v, &val[i], sizeof(v));
            if (CHECK) {
                const int cs = col0 + lane_col[i];
#pragma unroll
                for (int e = 0; e < VK; ++e)
                    if ((unsigned)(cs + e) >= (unsigned)W) v[e] = T(0);
            }
            half_t lo, hi;
#pragma unroll
            for (int e = 0; e < VK / 2; ++e) lo[e] = v[e], hi[e] = v[VK / 2 + e];
            *reinterpret_cast<half_t *>(lds + lds_at[i]) = lo;
            *reinterpret_cast<half_t *>(lds + lds_at[i] + VK / 2) = hi;
        }
    }
    __device__ __forceinline__ void stage(T *lds, int W, int row0, int col0, int tid) const {
        if (col0 >= 0 && col0 + COLS <= W)
            copy<false>(lds, W, row0, col0, tid);
        else
            copy<true>(lds, W, row0, col0, tid);
    }
};

// Wavefront `wave`'s share of one staged stage: column chunks [kc_lo, kc_hi) x left rows [row0, row0 + nrows).
template <class C>
__device__ __forceinline__ void mfma_stage(const typename C::value_type *Vs_lane, const typename C::value_type *Us_lane,
                                           typename C::Op::acc_t (&acc)[C::TJ][C::TI][C::NC], int wave, int kc_lo, int kc_hi, int row0, int nrows) {
    using T = typename C::value_type;
    typedef T evec __attribute__((ext_vector_type(C::EV))); // one right-operand read: EV consecutive elements, aligned
    constexpr int EV = C::EV;
    auto load = [](const T *vp, const T *up, evec (&a)[C::TI], T (&b)[C::TJ][EV]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < C::TI; ++t)
            a[t] = *reinterpret_cast<const evec *>(up + (t / C::NIY) * C::IU * C::UBAND - (t % C::NIY) * C::IY * C::PU);
#pragma unroll
        for (int s = 0; s < C::TJ; ++s)
#pragma unroll
            for (int e = 0; e < EV; ++e) b[s][e] = vp[(s / C::MJX) * C::JV * C::VBAND + (s % C::MJX) * C::JX + e];
    };
    auto multiply = [&](const evec (&a)[C::TI], const T (&b)[C::TJ][EV]) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < EV; ++e)
#pragma unroll
            for (int s = 0; s < C::TJ; ++s)
#pragma unroll
                for (int t = 0; t < C::TI; ++t) acc[s][t][e % C::NC] = C::Op::mma(a[t][e], b[s][e], acc[s][t][e % C::NC]);
    };
    // A stage whose useful column chunks divide evenly among the WZ wavefronts is dealt chunk by chunk (kc = wave mod WZ).
    // Otherwise - the tile overlaps only part of the stage's columns, the rule on small matrices - the (chunk, row) steps
    // are numbered row-fastest and cut into WZ equal runs, so that the wavefronts stay within one step of each other
    // (dealing whole chunks left three of four idle where a tile overlaps a single chunk of a stage).
    const int nkc = kc_hi - kc_lo;
    int kc_a, kc_b, kc_step, j_first, j_last; // chunks kc_a, kc_a + kc_step, ... < kc_b; rows from j_first in the first and up to j_last in the last chunk
    if (nkc % C::WZ == 0) {
        kc_a = kc_lo + wave;
        kc_b = kc_hi;
        kc_step = C::WZ;
        j_first = 0;
        j_last = nrows;
    } else {
        const int steps = nkc * nrows;
        const int first = steps * wave / C::WZ, last = steps * (wave + 1) / C::WZ; // [first, last)
        if (first >= last) return;
        kc_a = kc_lo + first / nrows;
        kc_b = kc_lo + (last - 1) / nrows + 1;
        kc_step = 1;
        j_first = first % nrows;
        j_last = (last - 1) % nrows + 1;
    }
    for (int kc = kc_a; kc < kc_b; kc += kc_step) {
        // (wavefront-uniform by construction; said so that the loop below is counted in scalar registers)
        const int ja = __builtin_amdgcn_readfirstlane(kc == kc_a ? j_first : 0);
        const int jb = __builtin_amdgcn_readfirstlane(kc + kc_step >= kc_b ? j_last : nrows);
        const T *vp = Vs_lane + kc * C::K + (row0 + ja) * C::PV;
        const T *up = Us_lane + kc * C::K + (row0 + ja) * C::PU;
        // two operand sets: the reads of the next row are issued before the instructions of the current one (the read
        // past the last row of a sweep lands in the spare row the bands end with and is not used); four rows per trip
        // so that the addresses advance once per sixteen-plus instructions
        evec a0[C::TI], a1[C::TI];
        T b0[C::TJ][EV], b1[C::TJ][EV];
        load(vp, up, a0, b0);
        int j = ja;
#pragma unroll 1
        for (; j + 4 <= jb; j += 4) {
            load(vp + C::PV, up + C::PU, a1, b1);
            multiply(a0, b0);
            load(vp + 2 * C::PV, up + 2 * C::PU, a0, b0);
            multiply(a1, b1);
            load(vp + 3 * C::PV, up + 3 * C::PU, a1, b1);
            multiply(a0, b0);
            vp += 4 * C::PV;
            up += 4 * C::PU;
            load(vp, up, a0, b0);
            multiply(a1, b1);
        }
#pragma unroll 1
        for (; j + 2 <= jb; j += 2) {
            load(vp + C::PV, up + C::PU, a1, b1);
            multiply(a0, b0);
            vp += 2 * C::PV;
            up += 2 * C::PU;
            load(vp, up, a0, b0);
            multiply(a1, b1);
        }
        if (j < jb) multiply(a0, b0);
    }
}

// The same for a FINE tile: the wavefront's result tiles (s along x, t along y) are swept one after the other, tile (s, t) over the
// column steps [ka_s, kb_s) and rows [ja_t, ja_t + nt_t) of the stage that its own P x P shifts overlap. The (step, tile, row) triples of
// the stage are numbered row-fastest and cut into WZ equal runs, one per wavefront.
// Stage geometry: its first right column is x0, its first base row yl0; the block tile's first shifts are (sxb, syb); the work item
// holds the right columns below w_hi and the left rows below chi.
template <class C>
__device__ __forceinline__ void mfma_stage_fine(const typename C::value_type *Vs_lane, const typename C::value_type *Us_lane,
                                                typename C::Op::acc_t (&acc)[C::TJ][C::TI][C::NC], int wave, int x0, int sxb, int W, int w_hi,
                                                int yl0, int syb, int H, int chi) {
    using T = typename C::value_type;
    typedef T evec __attribute__((ext_vector_type(C::EV)));
    constexpr int EV = C::EV, K = C::K, NKC = C::KBX / C::K;
    // rows of tile t: base rows yb = yl0 + j whose window meets the right matrix, yb in [syb + t IY, syb + t IY + IY - 1 + H - 1], yb < chi
    int ja[C::TI], nt[C::TI], rows_all = 0;
#pragma unroll
    for (int t = 0; t < C::TI; ++t) {
        const int first = syb + t * C::IY - yl0;
        int last = first + C::IY + H - 2;
        if (chi - 1 - yl0 < last) last = chi - 1 - yl0;
        if (last > C::RL - 1) last = C::RL - 1;
        ja[t] = first > 0 ? first : 0;
        nt[t] = last + 1 - ja[t] > 0 ? last + 1 - ja[t] : 0;
        rows_all += nt[t];
    }
    // column steps of tile s (x shifts sxb + s JX ...): (x0 + kc K + K - 1) + (sx + JX - 1) >= 0, (x0 + kc K) + sx <= W - 1, x0 + kc K < w_hi
    int ka[C::TJ], kb[C::TJ], steps_all = 0;
#pragma unroll
    for (int s = 0; s < C::TJ; ++s) {
        const int sx = sxb + s * C::JX;
        const int need = -(sx + C::JX - 1) - (K - 1) - x0;
        ka[s] = need > 0 ? (need + K - 1) / K : 0;
        int lim = W - 1 - sx - x0;
        if (w_hi - 1 - x0 < lim) lim = w_hi - 1 - x0;
        kb[s] = lim < 0 ? 0 : lim / K + 1;
        if (kb[s] > NKC) kb[s] = NKC;
        if (kb[s] < ka[s]) kb[s] = ka[s];
        steps_all += kb[s] - ka[s];
    }
    const int total = steps_all * rows_all;
    const int lo = total * wave / C::WZ, hi = total * (wave + 1) / C::WZ; // this wavefront's run [lo, hi)
    if (lo >= hi) return;
    int pos = 0;
#pragma unroll 1
    for (int kc = 0; kc < NKC; ++kc) {
#pragma unroll
        for (int s = 0; s < C::TJ; ++s) {
            if (kc < ka[s] || kc >= kb[s]) continue;
#pragma unroll
            for (int t = 0; t < C::TI; ++t) {
                const int begin = (lo > pos ? lo : pos) - pos, end = (hi < pos + nt[t] ? hi : pos + nt[t]) - pos;
                pos += nt[t];
                if (begin >= end) continue;
                const int j0 = __builtin_amdgcn_readfirstlane(ja[t] + begin), n = __builtin_amdgcn_readfirstlane(end - begin);
                const T *vp = Vs_lane + kc * K + j0 * C::PV + s * C::JX;
                const T *up = Us_lane + kc * K + j0 * C::PU - t * C::IY * C::PU;
                auto load = [](const T *v, const T *u, evec &a, T (&b)[EV]) __attribute__((always_inline)) {
                    a = *reinterpret_cast<const evec *>(u);
#pragma unroll
                    for (int e = 0; e < EV; ++e) b[e] = v[e];
                };
                auto multiply = [&](const evec &a, const T (&b)[EV]) __attribute__((always_inline)) {
#pragma unroll
                    for (int e = 0; e < EV; ++e) acc[s][t][e % C::NC] = C::Op::mma(a[e], b[e], acc[s][t][e % C::NC]);
                };
                // (as in mfma_stage: the reads of the next row before the instructions of the current one, four rows per trip; the read
                // past the last row lands in the spare row of the bands)
                evec a0, a1;
                T b0[EV], b1[EV];
                load(vp, up, a0, b0);
                int j = 0;
#pragma unroll 1
                for (; j + 4 <= n; j += 4) {
                    load(vp + C::PV, up + C::PU, a1, b1);
                    multiply(a0, b0);
                    load(vp + 2 * C::PV, up + 2 * C::PU, a0, b0);
                    multiply(a1, b1);
                    load(vp + 3 * C::PV, up + 3 * C::PU, a1, b1);
                    multiply(a0, b0);
                    vp += 4 * C::PV;
                    up += 4 * C::PU;
                    load(vp, up, a0, b0);
                    multiply(a1, b1);
                }
#pragma unroll 1
                for (; j + 2 <= n; j += 2) {
                    load(vp + C::PV, up + C::PU, a1, b1);
                    multiply(a0, b0);
                    vp += 2 * C::PV;
                    up += 2 * C::PU;
                    load(vp, up, a0, b0);
                    multiply(a1, b1);
                }
                if (j < n) multiply(a0, b0);
            }
        }
    }
}

// One block = four wavefronts that take work items one after the other. A launch is either one block per work item
// (gridDim.x = total_items, g.queue == nullptr) or PERSISTENT: as many blocks as the device holds at a time, each taking its own
// index as first item and every further one from the launch's queue counter (g.queue), i.e. in launch order - heaviest first -
// as blocks become free, which is what the hardware's own dispatch does with one block per item, minus what a fresh workgroup costs
// (measured on MI355X: 10 microseconds between the end of a block and the first instruction of its successor in the same slot,
// plus the set-up below; a work item of the 64x64 matrices lasts 35).
template <class C>
__global__ __launch_bounds__(C::NT, C::MINB) void mfma_kernel(EngineArgs<typename C::value_type> g) {
    using T = typename C::value_type;
    using vec = typename vec128<T>::type;
    using acc_t = typename C::Op::acc_t;
    constexpr int VK = C::VK, K = C::K, P = C::P;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    // Everything outside the sweep is latency (address arithmetic, loads, barriers) and a few instructions; the sweeps of the
    // other wavefronts of the SIMD are long runs of matrix instructions that the arbiter would otherwise serve first.
    __builtin_amdgcn_s_setprio(2);
    const int tid = (int)threadIdx.x;
    const int group = __builtin_amdgcn_readfirstlane(tid >> 6); // which share of the column chunks
    T *Vs = reinterpret_cast<T *>(smem_raw);
    T *Us = Vs + C::NVB * C::VBAND;
    int *handover = reinterpret_cast<int *>(smem_raw + C::BAND_BYTES); // two slots behind the bands: the next item, alternating
    const int W = g.W, H = g.H;
    const size_t HW = (size_t)W * H;
    const int Sx = 2 * W - 1, Sy = 2 * H - 1;
    const size_t out_area = (size_t)Sx * Sy;

    // ---- lane coordinates inside a result tile ----
    const int lane = tid & 63;
    const int p = lane % P, kk = lane / P;
    const int vj = p / C::JX / C::JYO, yo = p / C::JX % C::JYO, sxl = p % C::JX; // column j = p: left matrix, copy, x shift
    const int ui = p / C::IY, syl = p % C::IY; // row i = p: right matrix, y shift
    const T *Vs_lane0 = Vs + vj * C::VBAND + yo * C::IY * C::PV + sxl + C::EV * kk;
    const T *Us_lane = Us + ui * C::UBAND + (C::IYB - 1 - syl) * C::PU + C::EV * kk;

    // (the left band of the tiles with copies of the x shifts has rows that are not 128 bits apart: through registers)
    constexpr bool LEFT_DMA = C::PV % VK == 0;
    using LeftDma = BandDma<C, C::NVB, C::VROWS, C::PVC, C::PV, C::VBAND, 16>;
    using LeftLoad = BandLoad<C, C::VROWS, C::PVC, C::PV>;
    std::conditional_t<LEFT_DMA, LeftDma, LeftLoad> left_band;
    BandDma<C, C::NUB, C::RU, C::KBX, C::PU, C::UBAND, 16> right_dma; // (the padding columns of a right row are never read)
    if constexpr (LEFT_DMA)
        left_band.init(lane, group, W);
    else
        left_band.init(tid, W);
    right_dma.init(lane, group, W);

    // The queue this block draws from; the k-th draw stands for item my_queue + gridDim.x + queues * k. (Letting a block whose
    // queue is empty draw from the others was measured: every block then ends with up to eight draws nothing hides, and all
    // five benchmark workloads ran 1-2 % slower.)
    const int my_queue = g.queue != nullptr ? (int)(blockIdx.x % (unsigned)g.queues) : 0;
    unsigned *const queue = g.queue != nullptr ? g.queue + 32 * my_queue : nullptr;
    auto next_item = [&](unsigned drawn) __attribute__((always_inline)) { return (int)(my_queue + gridDim.x + (unsigned)g.queues * drawn); };
    // ordered accumulation: the ticket this block still has to pass on (once the stores of its last item have arrived) and its value
    unsigned *owed_ticket = nullptr;
    unsigned owed_value = 0;
    int item = (int)blockIdx.x;
    for (int turn = 0; item < g.total_items; ++turn) {
        // The item after this one is asked for when the last bands of this one have arrived (the answer of the contended counter
        // takes several times as long as a band, and every wait for bands would be a wait for it as well: it travels during the
        // last sweep) and is handed to the block before the barrier of the in-block reduction (slot `turn & 1`: a wavefront may
        // still read this turn's slot while thread 0, one barrier ahead at most, writes the next turn's).
        unsigned fetched = 0;
        WorkItem wi;
        const bool something_to_do = decode_work_item<C>(g, item, wi);
        if (something_to_do) {
            // (the same for all threads; said so that everything derived from them - loop bounds, buffer descriptors - stays in scalar registers)
            auto uniform = [](int x) __attribute__((always_inline)) { return __builtin_amdgcn_readfirstlane(x); };
            const int clo = uniform(wi.clo), chi = uniform(wi.chi), syb = uniform(wi.syb), sxb = uniform(wi.sxb), v_first = uniform(wi.v_first),
                      u_first = uniform(wi.u_first), u_limit = uniform(wi.u_limit);
            const int xr_lo = uniform(wi.xr_lo), xr_hi = uniform(wi.xr_hi), w_hi = uniform(wi.w_hi);
            // ordered accumulation: this item is chunk `chunk` of `chunks` of tile `tile` (see EngineArgs::tickets)
            const bool ordered = g.tickets != nullptr && uniform(wi.chunks) > 1;
            const int chunk = uniform(wi.chunk);
            unsigned *const ticket = g.tickets != nullptr ? g.tickets + uniform(wi.tile) : nullptr;
            unsigned ticket_seen = ~0u; // (thread 0: what the ticket read when it was last looked at)
            // With AL the left bands start at the 128-bit boundary of the matrix rows at or below the tile's first column (x0 is a
            // multiple of 8): every staged piece is then aligned in global memory and, where the width is a multiple of VK, wholly
            // inside or outside the matrix; the lanes read `left_shift` columns further in.
            const int left_shift = ((sxb % VK) + VK) % VK;
            const T *Vs_lane = Vs_lane0 + left_shift;

            acc_t acc[C::TJ][C::TI][C::NC];
#pragma unroll
            for (int s = 0; s < C::TJ; ++s)
#pragma unroll
                for (int t = 0; t < C::TI; ++t)
#pragma unroll
                    for (int c = 0; c < C::NC; ++c)
#pragma unroll
                        for (int r = 0; r < C::ACC; ++r) acc[s][t][c][r] = T(0);

            const int nbv = g.nV - v_first < C::NVB ? g.nV - v_first : C::NVB;
            const int nbu = u_limit - u_first < C::NUL ? u_limit - u_first : C::NUL;
            // of the left matrices the rows [clo, chi) of this work item exist, of the right matrices all
            if constexpr (LEFT_DMA)
                left_band.set_item(g.V + (size_t)v_first * HW, HW, W, clo, chi - clo, nbv, group);
            else
                left_band.set_item(g.V + (size_t)v_first * HW, W, clo, chi - clo, nbv);
            right_dma.set_item(g.U + (size_t)u_first * HW, HW, W, 0, H, nbu, group);

            // Stages: bands of RL left rows (outer) times blocks of KBX right columns (inner). (Fetching the next stage into
            // registers before the current one is swept, to hide the load latency behind the matrix instructions, measured
            // 2 % slower on large matrices and no faster on small ones: the other blocks of the CU already cover it.)
            // yl0: the left row of the first copy (the base row yb of the header); the last copy is (JYO - 1) * IY rows ahead of it.
            // Base rows below syb or from syb + IYB + H - 1 on meet no right row.
            int yl_begin = clo - (C::JYO - 1) * C::IY, yl_end = chi;
            if (C::JYO > 1) {
                if (yl_begin < syb) yl_begin = syb;
                if (yl_end > syb + C::IYB + H - 1) yl_end = syb + C::IYB + H - 1;
            }
            for (int yl0 = yl_begin; yl0 < yl_end; yl0 += C::RL) {
                for (int x0 = xr_lo; x0 < xr_hi; x0 += C::KBX) {
                    if (owed_ticket != nullptr) asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // (the stores of the previous item)
                    __syncthreads(); // everyone is done reading the previous stage (or adding up the previous item's tiles)
                    if (owed_ticket != nullptr) {
                        // everybody's stores of the previous item have arrived in memory: its tile's next chunk may go
                        if (tid == 0) __hip_atomic_store(owed_ticket, owed_value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        owed_ticket = nullptr;
                    }
                    {
                        // left band: rows [yl0, yl0+VROWS) of the chunk's rows [clo, chi), columns xl = x0 + sxb - shift + col (the 128-bit boundary at or below x0 + sxb)
                        const int xbase = x0 + sxb - left_shift;
                        // right band: rows yr = yl0 - syb - IYB + 1 + row, columns xr = x0 + col
                        const int yr0 = yl0 - syb - C::IYB + 1;
                        right_dma.stage(Us, W, yr0, x0, lane, group);
                        if constexpr (LEFT_DMA)
                            left_band.stage(Vs, W, yl0 - clo, xbase, lane, group);
                        else
                            left_band.stage(Vs, W, yl0 - clo, xbase, tid);
                        dma_wait();
                        if constexpr (LEFT_DMA) left_band.fix_right_edge(Vs, W, xbase, lane, group);
                        right_dma.fix_right_edge(Us, W, x0, lane, group);
                    }
                    __syncthreads();
                    if (yl0 + C::RL >= yl_end && x0 + C::KBX >= xr_hi && tid == 0) {
                        if (g.queue != nullptr) fetched = atomicAdd(queue, 1u);
                        // (a first look at the ticket, while the last stage is swept: the chunk before this one ended long ago)
                        if (ordered && chunk > 0) ticket_seen = __hip_atomic_load(ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    // base rows of this stage whose window of right rows meets the right matrix: yb in [syb, syb + IYB - 1 + H - 1], yb < chi
                    int first = syb - yl0;
                    int last = syb + C::IYB + H - 2 - yl0;
                    if (chi - 1 - yl0 < last) last = chi - 1 - yl0;
                    if (last > C::RL - 1) last = C::RL - 1;
                    const int row0 = first > 0 ? first : 0;
                    const int nrows = last + 1 - row0;
                    // column chunks of this stage that overlap the tile's x shifts: (x0 + kc*K + K-1) + (sxb + TXB-1) >= 0,
                    // (x0 + kc*K) + sxb <= W-1 and x0 + kc*K < w_hi
                    int kc_lo = 0, kc_hi = C::KBX / K;
                    {
                        int need = -(sxb + C::TXB - 1) - (K - 1) - x0;
                        if (need > 0) kc_lo = (need + K - 1) / K;
                        int lim = W - 1 - sxb - x0;
                        if (w_hi - 1 - x0 < lim) lim = w_hi - 1 - x0;
                        int h = lim < 0 ? 0 : lim / K + 1;
                        if (h < kc_hi) kc_hi = h;
                    }
                    if (nrows > 0 && kc_hi > kc_lo) {
                        __builtin_amdgcn_s_setprio(0);
                        if constexpr (C::FINE != 0)
                            mfma_stage_fine<C>(Vs_lane, Us_lane, acc, group, x0, sxb, W, w_hi, yl0, syb, H, chi);
                        else
                            mfma_stage<C>(Vs_lane, Us_lane, acc, group, kc_lo, kc_hi, row0, nrows);
                        __builtin_amdgcn_s_setprio(2);
                    }
                }
            }

            // ---- add the accumulator sets of every result tile, then the partial tiles of the WZ wavefronts through LDS, and write ----
#pragma unroll
            for (int s = 0; s < C::TJ; ++s)
#pragma unroll
                for (int t = 0; t < C::TI; ++t)
#pragma unroll
                    for (int c = 1; c < C::NC; ++c)
#pragma unroll
                        for (int r = 0; r < C::ACC; ++r) acc[s][t][0][r] += acc[s][t][c][r];
            // The accumulator elements of a lane are numbered tile * ACC + r and taken in quads of four. In pass q everyone
            // deposits quads q*QP .. q*QP + QP-1; wavefront w < QP then adds the WZ versions of quad q*QP + w in wavefront order
            // (deterministic) and writes it: P adjacent x shifts across the lanes.
            if (g.queue != nullptr && tid == 0) handover[turn & 1] = next_item(fetched);
            T *red = reinterpret_cast<T *>(smem_raw);
            constexpr int PASSES = (C::NQ + C::QP - 1) / C::QP;
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                __syncthreads(); // the bands, or the previous pass, are no longer read
#pragma unroll
                for (int o = 0; o < C::QP; ++o) {
                    const int Q = q * C::QP + o;
                    if (Q < C::NQ) {
                        const int tile = Q * 4 / C::ACC, r0 = Q * 4 % C::ACC;
                        T *dst = red + ((size_t)(o * C::WZ + group) * 64 + lane) * 4;
#pragma unroll
                        for (int e = 0; e < 4; e += VK) {
                            vec piece;
#pragma unroll
                            for (int x = 0; x < VK; ++x) piece[x] = acc[tile / C::TI][tile % C::TI][0][r0 + e + x];
                            *reinterpret_cast<vec *>(dst + e) = piece;
                        }
                    }
                }
                if (ordered && q == 0 && chunk > 0 && tid == 0) {
                    // Wait for the chunk before this one to have added itself. It was handed out a whole level of work items
                    // earlier, so the ticket is usually there already; the bound only makes sure that the kernel ends whatever
                    // happens (about a second; the sums of this tile are then wrong and the ticket is not passed on).
                    // (Ticket and output are read and written by accesses that pass the caches by - device-scope atomics - and
                    // are ordered by hand: the predecessor's stores have arrived before it writes the ticket, this block reads
                    // the output after it has seen the ticket. An acquire / release pair would flush and invalidate the whole
                    // L2 of an XCD per work item: measured 6.5 x slower.)
                    int polls = 0;
                    while (ticket_seen != (unsigned)chunk && ++polls < (1 << 22)) {
                        __builtin_amdgcn_s_sleep(16);
                        ticket_seen = __hip_atomic_load(ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
                __syncthreads();
                const int Q = q * C::QP + group;
                const int tile = Q * 4 / C::ACC, r0 = Q * 4 % C::ACC;
                const int s = tile / C::TI, t = tile % C::TI;
                const int v = v_first + (s / C::MJX) * C::JV + vj;
                const int ox = sxb + (s % C::MJX) * C::JX + sxl + (W - 1);
                if (group < C::QP && Q < C::NQ && v < g.nV && ox >= 0 && ox < Sx) {
                    T sum[4];
#pragma unroll
                    for (int src = 0; src < C::WZ; ++src) {
                        const T *from = red + ((size_t)(group * C::WZ + src) * 64 + lane) * 4;
#pragma unroll
                        for (int e = 0; e < 4; e += VK) {
                            vec piece = *reinterpret_cast<const vec *>(from + e);
#pragma unroll
                            for (int x = 0; x < VK; ++x) sum[e + x] = src == 0 ? piece[x] : sum[e + x] + piece[x];
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int i = C::Op::row(r0 + e, kk); // result row: right matrix, y shift
                        const int u = u_first + (t / C::NIY) * C::IU + i / C::IY;
                        const int oy = syb + yo * C::IYB + (t % C::NIY) * C::IY + i % C::IY + (H - 1);
                        if (u < u_limit && oy >= 0 && oy < Sy) {
                            const size_t mat_index = g.group_m > 0 ? (size_t)u : (size_t)v * g.nU + u;
                            T *o = g.out + mat_index * out_area + (size_t)oy * Sx + ox;
                            if (g.atomic) {
                                atomic_add(o, sum[e]);
                            } else if (ordered) {
                                // (loads and stores that every CU of the device sees at once: they pass the caches by)
                                const T before = chunk > 0 ? __hip_atomic_load(o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : T(0);
                                __hip_atomic_store(o, chunk > 0 ? before + sum[e] : sum[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            } else {
                                *o = sum[e];
                            }
                        }
                    }
                }
            }
            if (ordered) {
                // the next chunk of this tile may go once these stores have arrived: said at the first barrier of the next item
                // (the last chunk leaves the ticket at 0)
                owed_ticket = ticket;
                owed_value = chunk + 1 == uniform(wi.chunks) ? 0u : (unsigned)(chunk + 1);
            }
        }
        // ---- the next item ----
        if (g.queue == nullptr) {
            item += (int)gridDim.x;
        } else {
            if (!something_to_do) {
                if (tid == 0) handover[turn & 1] = next_item(atomicAdd(queue, 1u));
                __syncthreads();
            }
            item = __builtin_amdgcn_readfirstlane(handover[turn & 1]);
        }
    }
    if (owed_ticket != nullptr) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) __hip_atomic_store(owed_ticket, owed_value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (queue != nullptr && tid == 0) {
        // The last block of a queue to finish zeroes it for the next launch that uses it. (Every block's last draw precedes its
        // count here: the draw's answer ended its loop. gridDim.x is a multiple of the number of queues.)
        if (atomicAdd(queue + 1, 1u) == gridDim.x / (unsigned)g.queues - 1) {
            __hip_atomic_store(queue, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(queue + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

} // namespace xcorr

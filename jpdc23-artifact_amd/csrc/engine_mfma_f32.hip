// fp32 specialisations of the matrix-core sweep (engine_mfma.hpp): v_mfma_f32_32x32x2_f32, result tiles of 32 columns
// (left matrices x x shifts) by 32 rows (right matrices x y shifts). Four wavefronts share a block's tile and split
// the steps of every stage.
// Names: m<x shifts>x<y shifts> of the block tile, l / r = left / right matrices per block.
#include "engine_registry.hpp"

namespace xcorr {

//                              T   JV IU MJX MJV NIY NIU  RL KBX MINB NC WZ JYO FINE
// one pair per block
using M_32x32 = MfmaCfg<float, 1, 1, 1, 1, 1, 1, 32, 64, 4>;
using M_64x32 = MfmaCfg<float, 1, 1, 2, 1, 1, 1, 32, 64, 4>;
// rows of a result tile over right matrices (one_to_many, n_to_mn) ...
using M_32x8_r4 = MfmaCfg<float, 1, 4, 1, 1, 1, 1, 32, 32, 4>;
// (two result tiles per wavefront: stages of 16 rows keep them at 128 registers and four blocks per CU, 3-8 % faster than stages of 32
// rows at three blocks)
using M_32x8_r8 = MfmaCfg<float, 1, 4, 1, 1, 1, 2, 16, 32, 4>;
// the same right matrices with a square tile of shifts: the columns of a result tile are 16 x shifts twice, 8 left rows apart
using M_16x16_r4 = MfmaCfg<float, 1, 4, 1, 1, 1, 1, 32, 32, 4, 1, 4, 2>;
using M_16x16_r8 = MfmaCfg<float, 1, 4, 1, 1, 1, 2, 16, 32, 4, 1, 4, 2>;
// (four copies 4 rows apart with 8 right matrices - 8 x 16 shifts, MfmaCfg<float, 1, 8, 1, 1, 1, 1, 32, 32, 3, 1, 4, 4> - measured
// 2-8 % behind M_16x16_r4 wherever it ran, its eight right bands leave three blocks per CU: not compiled)
// ... and rows over right, columns over left matrices (n_to_m)
// (stages of 16 rows: 112 registers, four blocks per CU; 32 rows at three blocks 4-10 % slower)
using M_8x8_l4r4 = MfmaCfg<float, 4, 4, 1, 1, 1, 1, 16, 32, 4>;
// two result tiles per wavefront over eight right matrices: half the work items, each staging 1.5 x the bands for twice the products (128
// registers, four blocks per CU): 6-16 % faster than the 4 x 4 tile on 16x16 ... 64x64 matrices, level at 128x128. (Eight left matrices instead:
// 2-4 % behind this one; the fp64 counterparts need 168 registers or 64 KB of LDS and are 8-14 % slower than the fp64 4 x 4 tile: not compiled.)
using M_8x8_l4r8 = MfmaCfg<float, 4, 4, 1, 1, 1, 2, 16, 32, 4>;
// one pair per block, two by two result tiles of the 16 x 16 instruction per wavefront, each swept over its own overlap only: for
// many small pairs that share nothing (thousands of left matrices with one right matrix each), where 32 x 32 shifts of one pair sweep
// (1 + 31 / size)^2 of what a shift needs and 16 x 16 shifts (1 + 15 / size)^2
using M_32x32_s16 = MfmaCfg<float, 1, 1, 2, 1, 2, 1, 32, 32, 6, 1, 4, 1, 1>;
// four by four result tiles: a pair of up to 32x32 is one work item
using M_64x64_s16 = MfmaCfg<float, 1, 1, 4, 1, 4, 1, 32, 32, 5, 1, 4, 1, 1>;
// (stages of 64 columns instead of 32: 1-2 % slower on 32x32 ... 96x96 pairs with either tile; stages of 16 rows: 5 % slower on 32x32)
// The same sweep with four right matrices in the rows of a result tile (4 y shifts each) and four result tiles down a wavefront: the 16 x 16
// shifts of the m16x16_r4 tile above, trimmed along y to 4 shifts at a time. C4 0.641 -> 0.598 ms, C3 4.30 -> 4.19 ms, 1 x 256 of 64x64 119 -> 106 us.
// (Stages of 32 rows at four or five blocks per CU: +0.7 %; stages of 64 columns: +17 %; two accumulator sets: level; 32 x 16 shifts per block: +5 %;
// eight right matrices with 2 y shifts each: +13 %.)
using M_16x16_r4_s4 = MfmaCfg<float, 1, 4, 1, 1, 4, 1, 16, 32, 5, 1, 4, 1, 1>;

static const EngineSpec specs[] = {
    // (issue and staging factors of the run-time model: fitted to launches of 16x16 ... 1024x1024 matrices, 1 ... 1024 pairs)
    make_spec<M_32x32>("f32_m32x32", 0.716, 1.0),
    make_spec<M_64x32>("f32_m64x32", 0.749, 1.0),
    make_spec<M_32x8_r4>("f32_m32x8_r4", 0.707, 1.0),
    make_spec<M_32x8_r8>("f32_m32x8_r8", 0.782, 1.0),
    make_spec<M_8x8_l4r4>("f32_m8x8_l4r4", 0.750, 1.0),
    make_spec<M_16x16_r4>("f32_m16x16_r4", 0.677, 1.0),
    make_spec<M_16x16_r8>("f32_m16x16_r8", 0.703, 1.0),
    make_spec<M_8x8_l4r8>("f32_m8x8_l4r8", 0.745, 1.0),
    make_spec<M_32x32_s16>("f32_m32x32_s16", 0.83, 1.0),
    make_spec<M_64x64_s16>("f32_m64x64_s16", 0.84, 1.0),
    make_spec<M_16x16_r4_s4>("f32_m16x16_r4_s4", 0.68, 1.0),
};

const EngineSpec *engine_mfma_specs_f32(int *count) {
    *count = (int)(sizeof(specs) / sizeof(specs[0]));
    return specs;
}

} // namespace xcorr

// fp64 specialisations of the matrix-core sweep (engine_mfma.hpp): v_mfma_f64_16x16x4_f64 result tiles of 16 columns
// (left matrices x x shifts) by 16 rows (right matrices x y shifts). A wavefront needs at least two result tiles per
// operand it reads (one tile alone is bound by the LDS reads).
// Names: m<x shifts>x<y shifts> of the block tile, l / r = left / right matrices per block.
#include "engine_registry.hpp"

namespace xcorr {

//                               T    JV IU MJX MJV NIY NIU  RL KBX MINB
using D_32x32 = MfmaCfg<double, 1, 1, 2, 1, 2, 1, 32, 32, 4>;
using D_32x16 = MfmaCfg<double, 1, 1, 2, 1, 1, 1, 32, 32, 4>;
using D_32x8_r4 = MfmaCfg<double, 1, 2, 2, 1, 1, 2, 16, 32, 4>;
// (the same right matrices with 16 x 16 shifts - the columns of a result tile 8 x shifts twice, 8 left rows apart, as the fp32 file
// has them - measured level with D_32x8_r4 from 64x64 matrices on and 6 % faster on 32x32 only: not compiled)
// (stages of 12 rows: 128 registers and 40 KB of LDS, four blocks per CU; 16 rows at three blocks 2 % slower,
// 8 rows at four blocks level with that)
using D_8x8_l4r4 = MfmaCfg<double, 2, 2, 1, 2, 1, 2, 12, 32, 4>;

// D_32x32 with the sweep that goes result tile by result tile, each over the rows and column steps its own 16 x 16 shifts overlap
// (engine_mfma.hpp, FINE_): for many small pairs that share nothing - 2000 independent pairs of 32x32 / 64x64 / 128x128: 0.24 / 0.45 / 0.64 ->
// 0.32 / 0.55 / 0.71 of the fp64 peak. (The pair tile trimmed the same way, 4 x 4 shifts at a time, is 8 % SLOWER on C5: its one-tile runs are
// bound by their LDS reads.)
using D_32x32_s16 = MfmaCfg<double, 1, 1, 2, 1, 2, 1, 32, 32, 4, 1, 4, 1, 1>;

// ... and with four right matrices in the rows of a result tile (4 y shifts each), four result tiles down a wavefront: 16 x 16 shifts per block,
// trimmed along y to 4 at a time. Against D_32x8_r4: 1 x 64 of 128x128 0.666 -> 0.622 ms, 1 x 256 of 64x64 0.224 -> 0.201 ms, n-to-mn 8 x 16 of
// 128x128 1.274 -> 1.213 ms, level at 256x256. (32 x 16 shifts per block: ahead at 64x64 and 256x256 by 1-3 %, 4 % behind at 128x128; stages of 12 rows:
// level; of 8 rows: 4-6 % behind. Not compiled.)
using D_16x16_r4_s4 = MfmaCfg<double, 1, 4, 1, 1, 4, 1, 16, 32, 4, 1, 4, 1, 1>;

static const EngineSpec specs[] = {
    make_spec<D_32x32>("f64_m32x32", 0.696, 1.0),
    make_spec<D_32x16>("f64_m32x16", 0.697, 1.0),
    make_spec<D_32x8_r4>("f64_m32x8_r4", 0.705, 1.0),
    make_spec<D_8x8_l4r4>("f64_m8x8_l4r4", 0.730, 1.0),
    make_spec<D_32x32_s16>("f64_m32x32_s16", 0.80, 1.0),
    make_spec<D_16x16_r4_s4>("f64_m16x16_r4_s4", 0.73, 1.0),
};

const EngineSpec *engine_mfma_specs_f64(int *count) {
    *count = (int)(sizeof(specs) / sizeof(specs[0]));
    return specs;
}

} // namespace xcorr

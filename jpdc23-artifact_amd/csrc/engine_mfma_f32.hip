// fp32 specialisations of the matrix-core sweep (engine_mfma.hpp): v_mfma_f32_32x32x2_f32, result tiles of 32 columns
// (left matrices x x shifts) by 32 rows (right matrices x y shifts). Four wavefronts share a block's tile and split
// the steps of every stage.
// Names: m<x shifts>x<y shifts> of the block tile, l / r = left / right matrices per block.
#include "engine_registry.hpp"

namespace xcorr {

//                              T   JV IU MJX MJV NIY NIU  RL KBX MINB AL
// one pair per block
using M_32x32 = MfmaCfg<float, 1, 1, 1, 1, 1, 1, 32, 64, 4>;
using M_64x32 = MfmaCfg<float, 1, 1, 2, 1, 1, 1, 32, 64, 4>;
// rows of a result tile over right matrices (one_to_many, n_to_mn) ...
using M_32x8_r4 = MfmaCfg<float, 1, 4, 1, 1, 1, 1, 32, 32, 4>;
using M_32x8_r8 = MfmaCfg<float, 1, 4, 1, 1, 1, 2, 32, 32, 3>;
// ... and rows over right, columns over left matrices (n_to_m)
using M_8x8_l4r4 = MfmaCfg<float, 4, 4, 1, 1, 1, 1, 32, 32, 3, 1>;

static const EngineSpec specs[] = {
    // (issue and staging factors of the run-time model: fitted to launches of 16x16 ... 1024x1024 matrices, 1 ... 1024 pairs)
    make_spec<M_32x32>("f32_m32x32", 0.82, 1.0),
    make_spec<M_64x32>("f32_m64x32", 0.82, 1.0),
    make_spec<M_32x8_r4>("f32_m32x8_r4", 0.82, 1.0),
    make_spec<M_32x8_r8>("f32_m32x8_r8", 0.88, 1.0),
    make_spec<M_8x8_l4r4>("f32_m8x8_l4r4", 0.96, 1.0),
};

const EngineSpec *engine_mfma_specs_f32(int *count) {
    *count = (int)(sizeof(specs) / sizeof(specs[0]));
    return specs;
}

} // namespace xcorr

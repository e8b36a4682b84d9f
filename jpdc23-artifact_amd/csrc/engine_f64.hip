// fp64 specialisations of the sliding-window engine. The reference has no fp64 GPU
// path (its double instantiations are commented out, e.g.
// naive_shuffle_multirow_both.cu:701-710); these use v_fma_f64 with K = 2 columns per
// 128-bit LDS access. An 8x8 tile of doubles needs ~190 VGPRs (two wavefronts per SIMD).
#include <vector>

#include "engine_registry.hpp"

namespace xcorr {

//                              T       A  B  K NV NU  LX LY LV LU  WX WY  RL KBX MINB WZ
// one output row per lane, 2x2 wavefronts over the shifts
using R_1x1 = EngineCfg<double, 1, 8, 2, 1, 1, 8, 8, 1, 1, 2, 2, 8, 16, 4>;
using R_2x2 = EngineCfg<double, 1, 4, 2, 2, 2, 8, 8, 1, 1, 2, 2, 8, 16, 4>;
// the same with 32 x 8 shifts per wavefront and two wavefronts per block, for small matrices
using N_1x1 = EngineCfg<double, 1, 4, 2, 1, 1, 8, 8, 1, 1, 1, 2, 8, 8, 4>;
using N_2x2 = EngineCfg<double, 1, 4, 2, 2, 2, 8, 8, 1, 1, 1, 2, 8, 8, 4>;
// grouped tiles: four wavefronts share one tile and its bands and take every fourth chunk of columns of a stage
using Z_88 = EngineCfg<double, 8, 8, 2, 1, 1, 8, 8, 1, 1, 1, 1, 36, 16, 2, 4>;
using Z_44 = EngineCfg<double, 4, 4, 2, 1, 1, 8, 8, 1, 1, 1, 1, 20, 16, 4, 4>;
using Z_88_u4 = EngineCfg<double, 8, 8, 2, 1, 1, 4, 4, 1, 4, 1, 1, 36, 8, 2, 4>;
using Z_88_u16 = EngineCfg<double, 8, 8, 2, 1, 1, 2, 2, 1, 16, 1, 1, 36, 8, 2, 4>;
using Z_88_v4u4 = EngineCfg<double, 8, 8, 2, 1, 1, 2, 2, 4, 4, 1, 1, 36, 8, 2, 4>;
using Z_88_v8u8 = EngineCfg<double, 8, 8, 2, 1, 1, 1, 1, 8, 8, 1, 1, 36, 8, 2, 4>;
// 8x4 tiles of doubles fit 168 VGPRs: three wavefronts per SIMD
using Y_84_u4 = EngineCfg<double, 8, 4, 2, 1, 1, 4, 4, 1, 4, 1, 1, 36, 8, 3, 4>;
using Y_84 = EngineCfg<double, 8, 4, 2, 1, 1, 8, 8, 1, 1, 1, 1, 36, 16, 3, 4>;
// lanes over pairs of small matrices: two sets of bands, filled by direct-to-LDS loads while the
// other set is swept (last parameter; measured +8 % on 64x64 matrices, nothing on the fp32 tiles)
using D_84_v4u4 = EngineCfg<double, 8, 4, 2, 1, 1, 2, 2, 4, 4, 1, 1, 18, 8, 3, 4, 1>;
using D_84_v4u8 = EngineCfg<double, 8, 4, 2, 1, 1, 2, 1, 4, 8, 1, 1, 18, 8, 3, 4, 1>;

// 4x4 tiles with lanes over right matrices, for many small matrices
using Z_44_u4 = EngineCfg<double, 4, 4, 2, 1, 1, 4, 4, 1, 4, 1, 1, 20, 8, 4, 4>;
using Z_44_u8 = EngineCfg<double, 4, 4, 2, 1, 1, 4, 2, 1, 8, 1, 1, 20, 8, 4, 4>;

static const EngineSpec specs[] = {
    make_spec<R_1x1>("f64_a1b8"),
    make_spec<R_2x2>("f64_a1b4_l2r2"),
    make_spec<Z_88>("f64_a8b8", 0.705, 0.0),
    make_spec<Z_44>("f64_a4b4", 0.761, 0.638),
    make_spec<Z_88_u4>("f64_a8b8_lr4", 0.716, 1.26),
    make_spec<Z_88_u16>("f64_a8b8_lr16", 0.766, 5.832),
    make_spec<Z_88_v4u4>("f64_a8b8_ll4lr4", 0.807, 0.137),
    make_spec<Z_88_v8u8>("f64_a8b8_ll8lr8", 0.637, 12.851),
    make_spec<Y_84_u4>("f64_a8b4_lr4", 0.733, 0.0),
    make_spec<Y_84>("f64_a8b4", 0.676, 0.0),
    make_spec<D_84_v4u4>("f64_a8b4_ll4lr4", 0.81, 0.0),
    make_spec<D_84_v4u8>("f64_a8b4_ll4lr8", 0.84, 0.0),
    make_spec<Z_44_u4>("f64_a4b4_lr4", 0.82, 1.0),
    make_spec<Z_44_u8>("f64_a4b4_lr8", 0.85, 1.0),
    make_spec<N_1x1>("f64_a1b4"),
    make_spec<N_2x2>("f64_a1b4_l2r2_narrow"),
};

// the register-tile specialisations above followed by the matrix-core ones (engine_mfma_f64.hip): one table, built once
const EngineSpec *engine_specs_f64(int *count) {
    static const std::vector<EngineSpec> all = [] {
        std::vector<EngineSpec> v(specs, specs + sizeof(specs) / sizeof(specs[0]));
        int n = 0;
        const EngineSpec *m = engine_mfma_specs_f64(&n);
        v.insert(v.end(), m, m + n);
        return v;
    }();
    *count = (int)all.size();
    return all.data();
}

} // namespace xcorr

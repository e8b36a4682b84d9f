// fp32 specialisations of the sliding-window engine (the gfx950-tuned set that
// replaces the reference's template cross-products, CMakeLists.txt:16-46).
//
// Unless its comment says otherwise a tile keeps its register budget at or below 128 VGPRs (four
// wavefronts per SIMD: plain v_fmac_f32 only reaches the vector peak with at least two wavefronts
// issuing per SIMD) and its LDS bands at or below ~40 KB per four-wavefront block so four blocks
// share a CU; the tiles whose comment names 168 registers measured faster with three.
// Names: a<y shifts>b<x shifts> per lane, r/l = right/left matrices per lane, lr/ll = lanes
// laid over right/left matrices.
#include <vector>

#include "engine_registry.hpp"

namespace xcorr {

//                             T      A  B  K NV NU  LX LY LV LU  WX WY  RL KBX MINB WZ
// one output row per lane (families: shuffle, split-row, multimat-right, multimat-both); four
// wavefronts tile 2x2 over the shifts
using R_1x1 = EngineCfg<float, 1, 8, 4, 1, 1, 8, 8, 1, 1, 2, 2, 8, 32, 4>;
using R_1x4 = EngineCfg<float, 1, 8, 4, 1, 4, 8, 8, 1, 1, 2, 2, 8, 32, 4>;
using R_2x2 = EngineCfg<float, 1, 8, 4, 2, 2, 8, 8, 1, 1, 2, 2, 8, 32, 4>;
// the same with 32 x 8 shifts per wavefront and two wavefronts per block (32 x 16 shifts), for matrices so small that
// the tiles above mostly cover shifts that do not exist
using N_1x1 = EngineCfg<float, 1, 4, 4, 1, 1, 8, 8, 1, 1, 1, 2, 8, 16, 4>;
using N_1x4 = EngineCfg<float, 1, 4, 4, 1, 4, 8, 8, 1, 1, 1, 2, 8, 16, 4>;
using N_2x2 = EngineCfg<float, 1, 4, 4, 2, 2, 8, 8, 1, 1, 1, 2, 8, 16, 4>;
// grouped tiles: four wavefronts share one tile and its bands and take every fourth chunk of columns of
// a stage (WZ = 4). Lanes over shifts only ...
using Z_84 = EngineCfg<float, 8, 4, 4, 1, 1, 8, 8, 1, 1, 1, 1, 36, 32, 4, 4>;
using Z_88 = EngineCfg<float, 8, 8, 4, 1, 1, 8, 8, 1, 1, 1, 1, 36, 32, 4, 4>;
using Z_44 = EngineCfg<float, 4, 4, 4, 1, 1, 8, 8, 1, 1, 1, 1, 20, 32, 4, 4>;
// ... and lanes over right matrices (one_to_many, n_to_mn) or over pairs (n_to_m) of small matrices
using Z_84_u4 = EngineCfg<float, 8, 4, 4, 1, 1, 4, 4, 1, 4, 1, 1, 36, 16, 4, 4>;
using Z_88_u4 = EngineCfg<float, 8, 8, 4, 1, 1, 4, 4, 1, 4, 1, 1, 36, 16, 4, 4>;
// (the bands of sixteen right matrices allow three blocks per CU anyway, so these two are compiled for 168 registers:
// 8-17 % faster than at 128)
using Z_84_u16 = EngineCfg<float, 8, 4, 4, 1, 1, 2, 2, 1, 16, 1, 1, 18, 16, 3, 4>;
using Z_88_u16 = EngineCfg<float, 8, 8, 4, 1, 1, 2, 2, 1, 16, 1, 1, 18, 16, 3, 4>;
using Z_84_v4u4 = EngineCfg<float, 8, 4, 4, 1, 1, 2, 2, 4, 4, 1, 1, 18, 16, 4, 4>;
using Z_88_v4u4 = EngineCfg<float, 8, 8, 4, 1, 1, 2, 2, 4, 4, 1, 1, 18, 16, 4, 4>;
using Z_88_v8u8 = EngineCfg<float, 8, 8, 4, 1, 1, 1, 1, 8, 8, 1, 1, 18, 16, 4, 4>;
// (168 registers, three wavefronts per SIMD: measured 1.6-3 % faster than at 128, where 42 registers spill; with that budget all nine
// pieces a thread stages per band set are loaded before the first LDS write - last parameter -, another 1 %)
using Z_84_u8 = EngineCfg<float, 8, 4, 4, 1, 1, 4, 2, 1, 8, 1, 1, 36, 16, 3, 4, 0, 12>;
// lanes over 4 x 8 pairs: 8x8 shifts per wavefront, the least tile-edge work for n_to_m of small matrices (also 168 registers:
// 3-4 % faster than at 128, and than the 4 x 4 pair tile, on 32x32 and 64x64 matrices)
using Z_84_v4u8 = EngineCfg<float, 8, 4, 4, 1, 1, 2, 1, 4, 8, 1, 1, 18, 16, 3, 4>;

// 4x4 tiles with lanes over right matrices: 16x16 / 16x8 shifts per block, for many small matrices (planner's pick before
// and with them: n_to_m 16 x 16 of 32x32 25.7 -> 20.9 us, 8 x 16 of 48x48 38.6 -> 30.4 us, one_to_many 1 x 64 of 96x96 186 -> 158 us)
using Z_44_u4 = EngineCfg<float, 4, 4, 4, 1, 1, 4, 4, 1, 4, 1, 1, 20, 16, 4, 4>;
using Z_44_u8 = EngineCfg<float, 4, 4, 4, 1, 1, 4, 2, 1, 8, 1, 1, 20, 16, 4, 4>;

// paired groups: lanes over 8 left matrices that each bring their own right matrices (n_to_mn with few right matrices per
// left one, independent pairs); half as many staged rows as the tiles above so that three or four blocks share a CU
//                                T    A  B  K NV NU  LX LY LV LU  WX WY  RL KBX MINB WZ DB SB PG
using P_84_p8 = EngineCfg<float, 8, 4, 4, 1, 1, 4, 2, 8, 1, 1, 1, 18, 16, 3, 4, 0, 12, 1>;

static const EngineSpec specs[] = {
    make_spec<R_1x1>("f32_a1b8"),
    make_spec<R_1x4>("f32_a1b8_r4"),
    make_spec<R_2x2>("f32_a1b8_l2r2"),
    make_spec<Z_84>("f32_a8b4", 0.713, 2.629),
    make_spec<Z_88>("f32_a8b8", 0.749, 8.237),
    make_spec<Z_44>("f32_a4b4", 0.833, 0.743),
    make_spec<Z_84_u4>("f32_a8b4_lr4", 0.66, 5.288),
    make_spec<Z_88_u4>("f32_a8b8_lr4", 0.692, 10.581),
    make_spec<Z_84_u16>("f32_a8b4_lr16", 0.82, 4.421),
    make_spec<Z_88_u16>("f32_a8b8_lr16", 0.76, 8.433),
    make_spec<Z_84_v4u4>("f32_a8b4_ll4lr4", 0.875, 0.973),
    make_spec<Z_88_v4u4>("f32_a8b8_ll4lr4", 0.78, 6.347),
    make_spec<Z_88_v8u8>("f32_a8b8_ll8lr8", 0.956, 5.555),
    make_spec<Z_84_u8>("f32_a8b4_lr8", 0.64, 6.951),
    make_spec<Z_84_v4u8>("f32_a8b4_ll4lr8", 0.90, 0.973),
    make_spec<Z_44_u4>("f32_a4b4_lr4", 0.86, 2.5),
    make_spec<Z_44_u8>("f32_a4b4_lr8", 0.87, 2.5),
    make_spec<N_1x1>("f32_a1b4"),
    make_spec<N_1x4>("f32_a1b4_r4"),
    make_spec<N_2x2>("f32_a1b4_l2r2"),
    make_spec<P_84_p8>("f32_a8b4_pairs8", 0.60, 9.0),
};

// the register-tile specialisations above followed by the matrix-core ones (engine_mfma_f32.hip): one table, built once
const EngineSpec *engine_specs_f32(int *count) {
    static const std::vector<EngineSpec> all = [] {
        std::vector<EngineSpec> v(specs, specs + sizeof(specs) / sizeof(specs[0]));
        int n = 0;
        const EngineSpec *m = engine_mfma_specs_f32(&n);
        v.insert(v.end(), m, m + n);
        return v;
    }();
    *count = (int)all.size();
    return all.data();
}

} // namespace xcorr

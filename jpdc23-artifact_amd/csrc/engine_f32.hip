// fp32 specialisations of the sliding-window engine (the gfx950-tuned set that
// replaces the reference's template cross-products, CMakeLists.txt:16-46).
//
// Every tile keeps its register budget at or below 128 VGPRs (four wavefronts per SIMD:
// plain v_fmac_f32 only reaches the vector peak with at least two wavefronts issuing per
// SIMD, and an even number of resident wavefronts measured best) and its LDS bands at or
// below ~40 KB per four-wavefront block so four blocks share a CU.
#include "engine_registry.hpp"

namespace xcorr {

//                          T      A  B  K NV NU  LX LY LV LU  WX WY  RL KBX MINB
// one output row per lane (families: shuffle, split-row, multimat-right, multimat-both)
using R_1x1 = EngineCfg<float, 1, 8, 4, 1, 1, 8, 8, 1, 1, 2, 2, 8, 32, 4>;
using R_1x4 = EngineCfg<float, 1, 8, 4, 1, 4, 8, 8, 1, 1, 2, 2, 8, 32, 4>;
using R_2x2 = EngineCfg<float, 1, 8, 4, 2, 2, 8, 8, 1, 1, 2, 2, 8, 32, 4>;
// grouped (several y shifts per lane)
using G_88 = EngineCfg<float, 8, 8, 4, 1, 1, 8, 8, 1, 1, 2, 2, 18, 32, 4>;
using G_88_w1 = EngineCfg<float, 8, 8, 4, 1, 1, 8, 8, 1, 1, 1, 1, 18, 32, 4>;
using G_44 = EngineCfg<float, 4, 4, 4, 1, 1, 8, 8, 1, 1, 2, 2, 20, 32, 4>;
using G_44_w1 = EngineCfg<float, 4, 4, 4, 1, 1, 8, 8, 1, 1, 1, 1, 20, 32, 4>;
using G_88_u4 = EngineCfg<float, 8, 8, 4, 1, 1, 4, 4, 1, 4, 2, 2, 18, 16, 4>;
using G_88_u16 = EngineCfg<float, 8, 8, 4, 1, 1, 2, 2, 1, 16, 2, 2, 9, 8, 4>;
using G_88_v8u8 = EngineCfg<float, 8, 8, 4, 1, 1, 1, 1, 8, 8, 2, 2, 9, 16, 4>;
using G_88_v4u4 = EngineCfg<float, 8, 8, 4, 1, 1, 2, 2, 4, 4, 2, 2, 18, 16, 4>;
using G_48_n2 = EngineCfg<float, 4, 8, 4, 1, 2, 8, 8, 1, 1, 2, 2, 20, 32, 4>;
using G_44_n22 = EngineCfg<float, 4, 4, 4, 2, 2, 8, 8, 1, 1, 2, 2, 20, 32, 4>;
// four independent wavefronts per workgroup (last parameter), one tile and one set of bands each
using I_88 = EngineCfg<float, 8, 8, 4, 1, 1, 8, 8, 1, 1, 1, 1, 18, 8, 4, 4>;
using I_88b = EngineCfg<float, 8, 8, 4, 1, 1, 8, 8, 1, 1, 1, 1, 9, 16, 4, 4>;
using I_44 = EngineCfg<float, 4, 4, 4, 1, 1, 8, 8, 1, 1, 1, 1, 20, 16, 4, 4>;
using I_88_u4 = EngineCfg<float, 8, 8, 4, 1, 1, 4, 4, 1, 4, 1, 1, 9, 8, 4, 4>;
using I_88_v8u8 = EngineCfg<float, 8, 8, 4, 1, 1, 1, 1, 8, 8, 1, 1, 9, 8, 4, 4>;
using I_88_v4u4 = EngineCfg<float, 8, 8, 4, 1, 1, 2, 2, 4, 4, 1, 1, 9, 8, 4, 4>;
using I_48 = EngineCfg<float, 4, 8, 4, 1, 1, 8, 8, 1, 1, 1, 1, 20, 16, 4, 4>;
using I_84 = EngineCfg<float, 8, 4, 4, 1, 1, 8, 8, 1, 1, 1, 1, 18, 16, 4, 4>;

static const EngineSpec specs[] = {
    make_spec<R_1x1>("f32_a1b8"),
    make_spec<R_1x4>("f32_a1b8_r4"),
    make_spec<R_2x2>("f32_a1b8_l2r2"),
    make_spec<G_88>("f32_a8b8"),
    make_spec<G_88_w1>("f32_a8b8_w1"),
    make_spec<G_44>("f32_a4b4"),
    make_spec<G_44_w1>("f32_a4b4_w1"),
    make_spec<G_88_u4>("f32_a8b8_lr4"),
    make_spec<G_88_u16>("f32_a8b8_lr16"),
    make_spec<G_88_v8u8>("f32_a8b8_ll8lr8"),
    make_spec<G_88_v4u4>("f32_a8b8_ll4lr4"),
    make_spec<G_48_n2>("f32_a4b8_r2"),
    make_spec<G_44_n22>("f32_a4b4_l2r2"),
    make_spec<I_88>("f32_a8b8_i4"),
    make_spec<I_88b>("f32_a8b8_i4_rl9"),
    make_spec<I_44>("f32_a4b4_i4"),
    make_spec<I_88_u4>("f32_a8b8_lr4_i4"),
    make_spec<I_88_v8u8>("f32_a8b8_ll8lr8_i4"),
    make_spec<I_88_v4u4>("f32_a8b8_ll4lr4_i4"),
    make_spec<I_48>("f32_a4b8_i4"),
    make_spec<I_84>("f32_a8b4_i4"),
};

const EngineSpec *engine_specs_f32(int *count) {
    *count = (int)(sizeof(specs) / sizeof(specs[0]));
    return specs;
}

} // namespace xcorr

#ifdef XCORR_ENGINE_PROFILE
// profile builds only: copies out and clears the per-phase cycle table of the f32 kernels
extern "C" int xcorr_debug_engine_profile_f32(unsigned long long *out) { return (int)xcorr::engine_profile_read(out); }
#endif

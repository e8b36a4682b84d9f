// Table of compiled engine specialisations and the host-side planner that maps a
// request (sizes, matrix counts, the reference's tuning integers) onto one of them.
//
// The reference instantiates every value of every tuning integer up to a compile-time
// limit (CMakeLists.txt:16-46, about six hours of build). Here a short list of
// gfx950-tuned tiles is compiled and a request is mapped onto the nearest one; the
// geometry actually used is reported through xcorr_last_launch().
#pragma once

#include <cstdlib>
#include "engine.hpp"
#include "engine_mfma.hpp"
#include "xcorr_common.hpp"

namespace xcorr {

struct EngineSpec {
    const char *name;
    int elem_bytes; // 4 or 8
    int A, B, K, NV, NU;
    int LX, LY, LV, LU;
    int WX, WY, RL, KBX;
    int WZ; // wavefronts per workgroup that split one tile's rows and share the LDS bands
    int PG; // 1: lanes over left matrices that each bring their own group of right matrices (requests with group_m > 0 only)
    int MFMA; // 1: matrix-core sweep (engine_mfma.hpp); A, B, NV, NU, L* then describe what a lane holds of the result tiles
    int lds_bytes;
    int threads;
    // launches the kernel; `args` points at an EngineArgs<T> of the matching type
    hipError_t (*launch)(const void *args, unsigned grid, hipStream_t stream);
    // workgroups of this kernel that one CU of the current device holds at a time (registers and LDS), asked of the runtime
    // once per device; 0 without a device
    int (*resident_blocks_of_device)();
    // calibration of the planner's run-time model for grouped tiles: FMA issue slots a wavefront spends per
    // useful FMA instruction (LDS reads, waits and address arithmetic included), and the relative cost
    // of staging one band
    double issue_factor, stage_factor;
    // matrix-core tiles whose sweep trims every result tile of a block to its own overlap: the shifts of one result tile (else 0)
    int fine_x, fine_y;
    // the same, with the figure of an MI355X where no device can be asked (planning without a GPU)
    int resident_blocks() const;
    int TXW() const { return LX * B; }
    int TYW() const { return LY * A; }
    int TXB() const { return TXW() * WX; }
    int TYB() const { return TYW() * WY; }
    int NVB() const { return LV * NV; }
    int NUB() const { return LU * NU; } // right matrices per block that one left matrix meets
    int right_bands() const { return PG ? NVB() * NUB() : NUB(); }
};

// the kernel a configuration type stands for
template <class C>
constexpr auto kernel_of() {
    if constexpr (C::MFMA != 0)
        return &mfma_kernel<C>;
    else
        return &engine_kernel<C>;
}

template <class C>
hipError_t allow_large_lds() {
    if (C::LDS_BYTES <= 64 * 1024) return hipSuccess;
    // the attribute belongs to the kernel's copy on one device: kept per device of the process
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    const bool tracked = dev >= 0 && dev < 64;
    if (!tracked || !attr_set[dev]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel_of<C>()),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
        if (e != hipSuccess) return e;
        if (tracked) attr_set[dev] = true;
    }
    return hipSuccess;
}

template <class C>
hipError_t launch_engine(const void *args, unsigned grid, hipStream_t stream) {
    using T = typename C::value_type;
    if (hipError_t e = allow_large_lds<C>(); e != hipSuccess) return e;
    kernel_of<C>()<<<dim3(grid), dim3(C::NT), C::LDS_BYTES, stream>>>(*static_cast<const EngineArgs<T> *>(args));
    return hipGetLastError();
}

template <class C>
int resident_blocks_engine() {
    static int blocks[MAX_DEVICES] = {}; // per device: another device may hold another number
    const int dev = current_device();
    if (blocks[dev] == 0) {
        int n = 0;
        if (allow_large_lds<C>() != hipSuccess ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void *>(kernel_of<C>()), C::NT, C::LDS_BYTES) != hipSuccess || n < 1) {
            (void)hipGetLastError();
            return 0; // (not kept: a device may appear later)
        }
        blocks[dev] = n;
    }
    return blocks[dev];
}

template <class C>
constexpr int fine_extent(bool along_x) {
    if constexpr (C::MFMA != 0) {
        if constexpr (C::FINE != 0) return along_x ? C::JX : C::IY;
    }
    return 0;
}

template <class C>
constexpr EngineSpec make_spec(const char *name, double issue_factor = 1.0, double stage_factor = 1.0) {
    return EngineSpec{name,   (int)sizeof(typename C::value_type),
                      C::A,   C::B,
                      C::K,   C::NV,
                      C::NU,  C::LX,
                      C::LY,  C::LV,
                      C::LU,  C::WX,
                      C::WY,  C::RL,
                      C::KBX, C::WZ,
                      C::PG,  C::MFMA, C::LDS_BYTES,
                      C::NT,  &launch_engine<C>, &resident_blocks_engine<C>, issue_factor, stage_factor,
                      fine_extent<C>(true), fine_extent<C>(false)};
}

// defined in engine_f32.hip / engine_f64.hip
const EngineSpec *engine_specs_f32(int *count);
const EngineSpec *engine_specs_f64(int *count);
// defined in engine_mfma_f32.hip / engine_mfma_f64.hip: the matrix-core specialisations, appended to the tables above
const EngineSpec *engine_mfma_specs_f32(int *count);
const EngineSpec *engine_mfma_specs_f64(int *count);

// What a family asks of the engine.
struct EngineRequest {
    const char *family;
    int elem_bytes;
    const void *V, *U;
    void *out;
    int W, H, nV, nU;
    int group_m;          // see EngineArgs
    // hints (0 = none). y_shifts == 1 selects the one-output-row-per-lane specialisations.
    unsigned y_shifts, x_shifts, left_mats, right_mats, lanes_x, lanes_y, waves;
    unsigned spec_index;      // 1-based: use exactly this entry of the specialisation table
    unsigned rows_per_worker; // 0 = planner decides
    unsigned column_chunks;   // 0 = planner decides (grouped families only)
    unsigned matrix_cores;    // 0 = planner decides, 1 = matrix-core tiles only, 2 = register tiles only
    unsigned dist;            // XCORR_DIST_*
    bool caller_zeroes;       // true: split-row contract, output arrives zeroed, always accumulate atomically
    bool may_split;           // planner may split the reduction and clear the output itself
    bool ordered;             // a split reduction adds its chunks in order (tickets in the library's scratch array, matrix-core
                              // tiles only): no atomic adds, no cleared output, the same bits every run
};

struct EnginePlan {
    const EngineSpec *spec;
    int ntx, nty, nworkers_y, nvg, nug;
    int rows_per_chunk, dist, atomic, total_items;
    int x_chunks, x_chunk_cols; // chunks of right columns per tile (1: not cut) and their width
    bool zero_fill;
    bool ordered; // chunks add themselves to the output in order (dist 3, tickets)
    unsigned grid;
    double predicted_us; // of the run-time model (grouped families; 0 where no model was asked)
};

int plan_engine(const EngineRequest &rq, EnginePlan &plan);
int run_engine(const EngineRequest &rq, hipStream_t stream);

} // namespace xcorr

// The planner of the launch layer: which kernels a call of a given shape launches, with what tile, workgroup
// and LDS layout. Host code only, plain C++ (no HIP header): it is compiled and tested without a device.
#ifndef SPHX_PLAN_HPP
#define SPHX_PLAN_HPP

#include <cstddef>
#include <string>

#include "sphx_geometry.hpp"
#include "sphx_pairs_plan.hpp"

namespace sphx {

// The message behind the last status other than SPHX_OK that this thread was handed.
extern thread_local std::string t_error;
int fail(int code, const std::string& what);

// Overrides of single planning decisions, for measurements and tests (sphx_set_switch). None is
// set in normal use: a call is then planned from its shape alone and no environment variable is
// looked at. The variables of the same names are read once, when the library is first used, and
// only if SPHX_DEBUG_SWITCHES is set to something other than 0.
enum Switch : int {
    SW_AZ_SHIFT, SW_CHUNK_SHIFT, SW_GRADIENT_LANES, SW_GRADIENT_LANES_PARTS,
    SW_GRADIENT_LANES_TILE, SW_GRADIENT_LANES_WAVES, SW_GROUP_THREADS, SW_HESSIAN_LANES, SW_HESSIAN_LANES_PARTS, SW_HESSIAN_LANES_TILE, SW_JOB_LIST,
    SW_PAIRS, SW_PAIRS_BATCH, SW_PAIRS_CHUNK, SW_PAIRS_PREP_WAVES, SW_PAIRS_SEQUENCE_WAVES, SW_PAIRS_TILE,
    SW_PREFIX_INSIDE, SW_RECURSIONS_TOGETHER, SW_ROW_PAD,
    SW_SEQUENCE_WAVES, SW_SLICE_WAVES, SW_SPLIT_BELOW, SW_SPLIT_RATIO, SW_SPLIT_SIDES, SW_SPREAD_KINDS, SW_TILE, SW_TILE_LDS_BUDGET,
    SW_TILE_POW2, SW_TILE_SMALL_N, SW_VALUES_ALONE, SW_VALUES_LDS, SW_VALUES_MIN_TILE, SW_VALUES_MIN_WAVES,
    SW_VALUES_PACK, SW_VALUES_TILE_STEP, SW_VALUES_WAVES, SW_VJP_GROUPS_BELOW, SW_VJP_LANES, SW_VJP_MIN_TILE, SW_VJP_STEP_FLOOR, SW_VJP_TILE_STEP, SW_WAVE_PRIORITIES, SW_COUNT
};

// The value of an override as the plan being made sees it, `fallback` where none is set.
int switch_or(Switch which, int fallback);
// Set or clear overrides (sphx_set_switch, sphx_reset_switches); 1 for a name that is none.
int set_switch(const char* name, int value);
void reset_switches();
// Takes this thread's copy of the overrides if they have changed since it last did; returns their generation
// (never 0), by which cached plans know whether they still hold.
unsigned refresh_switches();

struct Launch {
    Tiling g;
    unsigned workgroups;
    unsigned threads;
    unsigned lds_bytes;
};

struct Plan {
    bool lanes;       // values only, short rows: one launch of values_kernel (uses `closed`)
    bool closed_only; // l_max within the closed forms: one launch of closed_form_kernel
    bool whole;       // recursion_kernel evaluates the closed forms too: one launch
                      // otherwise closed_form_kernel<PREFIX> + recursion_kernel: two launches
    bool split_sides; // recursion_kernel takes the entries (l, +m) and (l, -m) as two jobs
    bool pairs;       // values and gradients at large l_max: one launch of pairs_kernel (uses `pairs_launch`)
    Launch closed;
    Launch rec;
    PairsLaunch pairs_launch;
};

// The fused product (sphx_vjp_*): the lane kernels' launch beyond l_max = 6 where the rows of a tile fit LDS,
// else the closed-form or the recursion kernel with the contraction in place of the flush (`plan`).
struct VjpPlan {
    Plan plan;
    Launch lanes;
    bool use_lanes = false;
    bool lane_groups = false; // vjp_groups_kernel: groups of lanes with channels of their own
};

// Choose kernels, tile sizes and LDS layouts. `lds_limit` / `cus` describe the device. `lane_kernels` false:
// only closed_form_kernel and recursion_kernel (the fused product has no other).
int make_plan(size_t n_samples, int l_max, int mode, size_t elem, int lds_limit, int cus, Plan* plan,
              bool lane_kernels = true, bool normalized = true);
// float arrays evaluated in float64 inside the recursion kernel: false where that covers no such shape.
bool make_wide_plan(size_t n_samples, int l_max, int mode, int lds_limit, int cus, Plan* plan, bool normalized);
int make_vjp_plan(size_t n_samples, int l_max, size_t elem, int lds_limit, int cus, VjpPlan* plan);
// One line that names the kernels of a plan with their template arguments and launch geometry.
std::string describe(const Plan& plan, int l_max, int mode, bool is_f64, bool normalized);

} // namespace sphx

#endif

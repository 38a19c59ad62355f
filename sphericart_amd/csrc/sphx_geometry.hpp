// What the planner (host, plain C++) and the kernels (gfx950) both need to know: the description of a launch's
// tiling that the host fills in, and the few constants that fix the shape of a kernel's workgroup. No HIP
// header is included here; the constexpr functions are usable on the device as they are.
#ifndef SPHX_GEOMETRY_HPP
#define SPHX_GEOMETRY_HPP

#include <cstddef>
#include <cstdint>

namespace sphx {

// Everything a kernel needs to know about the tiling; filled in on the host.
struct Tiling {
    unsigned long long n_samples;
    unsigned n_tiles;       // tiles of `tile` points (recursion) or groups of 64 points (closed form)
    unsigned tiles_per_xcd; // workgroups of one XCD walk one contiguous stretch of tiles
    int l_max;
    int ny;                 // (l_max + 1)^2: length of one component row in HBM
    int tile;               // points whose rows are staged in LDS at a time
    unsigned magic_jobs;    // ceil(2^32 / jobs_per_point)
    unsigned jobs_per_point; // entry jobs per point: (l, m >= 0) pairs above the closed-form
                             // limit, or (l, m, side) triples when the sides are split
    unsigned sequence_waves; // waves that run the bare recursions (1 or 2)
    unsigned points_per_pass; // points whose entry jobs fit side by side in the wide waves;
                              // 0: the jobs of all points of a tile as one list
    unsigned vjp_accumulate; // fused product: add to xyz_grad instead of overwriting it
    unsigned az_shift;      // the point tables are made for 2^az_shift tiles at a time
    unsigned chunk_shift;   // a workgroup takes 2^chunk_shift consecutive tiles at a time
    unsigned prefix_inside; // rows that start at l = 7: the recursion kernel writes l <= 6 too
    unsigned slice_waves;   // not 0: this many waves of their own (together: and wave 0) evaluate the closed
                            // forms of l <= 6 (whole rows); 0: the slices go round all waves
    unsigned together;      // recursion_kernel, float64: 1 = the recursions run next to the entries (TOGETHER)
    unsigned row_pad;       // recursion_kernel, whole rows: elements left free after every staged row (0 or 16 bytes' worth)
    unsigned magic_ny;      // ceil(2^32 / ny)
    unsigned priorities;    // recursion_kernel: 1 = the waves that flush run at raised priority, 2 = those that prepare the next tile
    // LDS carve-up, in elements of T: the staged rows come first, rows_elems of them, with the
    // gradient and second-derivative rows at off_dsph and off_ddsph inside a buffer; the other
    // offsets count from the start of dynamic LDS. (recursion_kernel: the row offsets are in
    // elements of the output arrays, the others in numbers of the arithmetic type and count
    // from byte tables_at.)
    unsigned rows_elems, off_dsph, off_ddsph, off_F, off_Q, off_pts, off_iter, off_jobs;
    unsigned tables_at;
    // recursion_kernel, job-list variant: jobs per point of the kinds bulk / |m| = l and l - 1 /
    // m = 0 (the order of the job table), and ceil(2^32 / .) of each (0 where there are none)
    unsigned kind_jobs[3], kind_magic[3];
    // recursion_kernel, jobs point by point: where the jobs with |m| = l, |m| = l - 1 and m = 0 start
    // in the job table when they are moved to wave boundaries of the entry lanes (0: they follow
    // the bulk without gaps); jobs_per_point then counts the gaps too
    unsigned kind_at[3];
};

// a place in the job table of recursion_kernel that holds no job
constexpr unsigned kNoJob = 0xffffffffu;

constexpr unsigned magic_of(unsigned long long divisor) {
    return static_cast<unsigned>(((1ull << 32) + divisor - 1) / divisor);
}

// threads of a workgroup of recursion_kernel that shares its CU with a second one (one alone has twice as many)
constexpr unsigned kRecursionThreads = 512;

// LDS the closed-form kernel may use for one pass over its 64 points: above it the points are taken in
// 2, 4, 8 or 16 passes (l_max = 6 float32 with gradients runs fastest with a single pass, 50 KB)
#ifndef SPHX_PHASE_LDS_BUDGET
#define SPHX_PHASE_LDS_BUDGET (52 * 1024)
#endif

constexpr unsigned components_of(int mode) { return mode == 0 ? 1u : (mode == 1 ? 4u : 13u); }

// LDS elements per point in the closed-form kernel: the rows of all arrays, each array padded
// by one element when (H+1)^2 is even so that the per-point stride is odd (lanes staging the
// same entry of different points then hit different banks).
constexpr unsigned closed_form_pad(int H) { return ((H + 1) * (H + 1)) % 2 == 0 ? 1u : 0u; }

constexpr unsigned closed_form_phases(unsigned elem, int mode, int H) {
    const unsigned ny = (H + 1) * (H + 1);
    const unsigned per_point = (components_of(mode) * ny + (mode + 1) * closed_form_pad(H)) * elem;
    unsigned phases = 1;
    while (phases < 16 && (64 / phases) * per_point > SPHX_PHASE_LDS_BUDGET) {
        phases *= 2;
    }
    return phases;
}

// threads of a workgroup of hessians_lanes_kernel (float64 entries need more than 128 registers; float32 with
// 512 threads and 128 registers per lane was 5-15 % slower at l_max = 2-5 with the same number of waves)
constexpr unsigned kHessianLaneThreads = 256;
template <typename T> constexpr unsigned hessian_lane_threads() { return kHessianLaneThreads; }

} // namespace sphx

#endif

// What every kernel of the launch layer shares: the prefactor tables in constant memory, the
// description of a launch's tiling that the host fills in, and the dynamic LDS array.
#ifndef SPHX_TILING_HPP
#define SPHX_TILING_HPP

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "sphx_device.hpp"
#include "sphx_tables.hpp"

namespace sphx {

constexpr int kTableEntries = (SPHX_TABLE_LMAX + 1) * (SPHX_TABLE_LMAX + 2) / 2;

__constant__ float kF32[kTableEntries];
__constant__ float kQ32[kTableEntries];
__constant__ double kF64[kTableEntries];
__constant__ double kQ64[kTableEntries];

template <typename T> __device__ __forceinline__ const T* table_F();
template <typename T> __device__ __forceinline__ const T* table_Q();
template <> __device__ __forceinline__ const float* table_F<float>() { return kF32; }
template <> __device__ __forceinline__ const float* table_Q<float>() { return kQ32; }
template <> __device__ __forceinline__ const double* table_F<double>() { return kF64; }
template <> __device__ __forceinline__ const double* table_Q<double>() { return kQ64; }

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
    unsigned slice_waves;   // not 0: wave 0 and this many waves of their own evaluate the closed forms
                            // of l <= 6 (whole rows, one row buffer); 0: the slices go round all waves
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

extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

// Output lines are written once and never read back by the kernel: store them with the
// non-temporal hint (measured 10-20 % faster than plain stores here).
#ifndef SPHX_STREAMING_STORES
#define SPHX_STREAMING_STORES true
#endif

// LDS loads a flushing wave of the recursion kernel keeps in flight
#ifndef SPHX_FLUSH_UNROLL
#define SPHX_FLUSH_UNROLL 4
#endif

__host__ __device__ constexpr unsigned magic_of(unsigned long long divisor) {
    return static_cast<unsigned>(((1ull << 32) + divisor - 1) / divisor);
}

} // namespace sphx

#endif

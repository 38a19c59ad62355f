// What the host tells pairs_kernel about a launch. Plain C++: shared by the planner (host only) and the
// kernel.
#ifndef SPHX_PAIRS_TILING_HPP
#define SPHX_PAIRS_TILING_HPP

namespace sphx {

constexpr unsigned kPairsThreads = 1024;
constexpr unsigned kPairsNoJob = 0xffffu;

struct PairsTiling {
    unsigned long long n_samples;
    unsigned n_tiles;
    unsigned tiles_per_xcd;
    int l_max;
    int ny;
    unsigned tile;           // points per tile
    unsigned chunk_shift;    // a workgroup takes 2^chunk_shift consecutive tiles at a time
    unsigned batch_tiles;    // tiles per batch of point records and parked closed forms
    unsigned magic_batch;    // ceil(2^32 / batch_tiles)
    unsigned prep_waves, sequence_waves, entry_waves;
    unsigned slot_waves;     // entry waves that share one point; entry_waves / slot_waves points side by side
    unsigned off_dsph;       // staged gradient rows, in elements of the output type
    unsigned tables_at;      // bytes: where the part of LDS in the arithmetic type starts
    unsigned off_Q, off_F0, off_pts, off_park, off_iter; // in numbers of the arithmetic type, from tables_at
    unsigned point_stride, park_stride, iter_stride;
    unsigned tmz_at;         // where 2(m+1)z starts in a point's record (a multiple of four numbers)
    unsigned q_stride;       // distance between the rows of the Q constants in LDS (a multiple of four)
    // the pair (l << 8 | m) of every lane of the slot_waves waves that share a point
    unsigned short lane_job[kPairsThreads];
};

} // namespace sphx

#endif

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
    // How many batches ahead of the tile being staged the records are prepared: 1, or 2 where a batch is a
    // single tile (the recursions of tile n + 1 run while tile n is flushed, when its records must be complete;
    // the records of tile n + 2 then take the place of those of tile n, which is staged by then). Two buffers of
    // one batch each either way.
    unsigned lookahead;
    unsigned prep_waves, sequence_waves, entry_waves;
    unsigned slot_waves;     // MODE 1: entry waves that share one point; entry_waves / slot_waves points side by side
    unsigned lane_slots;     // MODE 2: points side by side in the entry lanes (the lane table says which lane takes which)
    unsigned off_dsph, off_ddsph; // staged gradient and second-derivative rows, in elements of the output type
    unsigned tables_at;      // bytes: where the part of LDS in the arithmetic type starts
    unsigned off_Q, off_F0, off_pts, off_park, off_iter; // in numbers of the arithmetic type, from tables_at
    unsigned point_stride, park_stride, iter_stride;
    unsigned tmz_at;         // where 2(m+1)z starts in a point's record (a multiple of four numbers)
    unsigned q_stride;       // distance between the rows of the Q constants in LDS (a multiple of four)
    unsigned priorities;     // 1 = the waves that flush run at raised priority, 2 = those that prepare the next tiles
    // the pair of every entry lane, slot << 14 | l << 7 | m (MODE 1: of the slot_waves waves that share a
    // point, slot 0)
    unsigned short lane_job[kPairsThreads];
};

} // namespace sphx

#endif

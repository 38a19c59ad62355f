// recursion_kernel: the general case, persistent workgroups whose waves have roles of their own.
#ifndef SPHX_RECURSION_KERNEL_HPP
#define SPHX_RECURSION_KERNEL_HPP

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "sphx_tiling.hpp"
#include "sphx_closed_form_kernel.hpp"

namespace sphx {

// ---------------------------------------------------------------------------
// l > H through the recursion. NT = 512 or 1024 threads, persistent workgroups
// that walk over tiles of `tile` consecutive points. A tile has two phases with a
// barrier in front of each:
//
//   entries      every wave (but the slice waves), one job per (point, l, m >= 0) of
//                tile i: the entries (l, +-m) of every requested array, chain rule
//                included, staged in LDS in HBM layout (entry_job). Neighbouring
//                lanes take neighbouring m of one (point, l), so their LDS traffic
//                falls on neighbouring banks;
//   flush        most waves stream the staged rows of tile i to HBM with 16-byte
//                stores, and meanwhile
//     wave 0       one batch of up to eight tiles ahead, one lane per point:
//                  normalised coordinates, c_m, s_m, 2(m+1)z into LDS (azimuth_job);
//     waves 1 ..   tile i+1, one lane per (point, l, sequence): the bare Q
//                  recursions, every iterate into LDS (sequence_job);
//                  g.sequence_waves of them.
//
// The entries keep the vector units of the CU busy; the flush waits for the
// stores to drain and issues little. Tables and recursions are short chains of
// dependent operations that only a few lanes can share: in the flush they cost
// no time of their own, and the entries then have every wave. The point tables
// are kept in two buffers, the iterates and the staged rows in one. (A second
// row buffer, flushed by waves of their own while the next tile is computed,
// was built and measured slower on every shape: waves that only flush wait for
// their own LDS loads most of the time, and the tile has to be half as large.)
//
// TOGETHER == true (float64 only) is the other division of the same work: wave 0
// and the sequence waves do their part next to the entries, a tile ahead of them
// (tables in three buffers when a batch is a single tile, iterates in two), the
// waves after them compute the entries, and every wave flushes. In float64 the
// recursions are long enough to hold up a flush that they share, and for solid
// harmonics, whose entries are short, and at high l_max this division is the
// faster one by 5-14 %; the host says which one a launch takes (g.together).
//
// NT = 512: two workgroups share a CU, half of its LDS each. NT = 1024: one
// workgroup has the CU and all of its LDS, its tiles are more than twice as
// large, and with g.slice_waves the closed forms of l <= H have waves of their
// own (the last ones; TOGETHER: next to wave 0).
//
// SPLIT == true (second derivatives, so few points per tile that the (l, m)
// pairs of a tile leave lanes idle): the entries (l, +m) and (l, -m) are two
// jobs.
//
// WHOLE == true: the closed forms of l <= H are evaluated here too (one lane
// per point, the entries in slices that go round all waves) and the tile's
// rows are complete, one contiguous run per array.
// WHOLE == false: the rows start at l = H + 1 (closed_form_kernel<PREFIX>
// writes the part below); every (point, component) row is its own run.
// ---------------------------------------------------------------------------
// (kRecursionThreads, the threads of a workgroup that shares its CU with a second one: sphx_geometry.hpp)

// Values and gradients: at most 128 registers, so that two workgroups of 512 threads or one of
// 1024 fit on a CU (four waves per SIMD) wherever their LDS allows. Only the float64 closed forms exceed that on their own
// and spill a few registers; with 170 registers and one workgroup per CU, l_max = 12 float64
// gradients took 800 us instead of 513 us. The second-derivative kernels keep what they need
// (forced to 128 they spill in the entry jobs: 918 us against 558 us at l_max = 10, float64).
//
// O: the type of xyz and of the output arrays, T the type of the arithmetic. O = float with
// T = double evaluates float arrays in float64: the coordinates are widened as they are read, the
// tables and iterates are float64, and every result is rounded once, as it is staged. The staged
// rows are rows of O, so a tile holds as many points as in the float kernel's and the flush is
// that kernel's.
template <typename T, int MODE, bool NORM, bool WHOLE, bool SPLIT, bool VJP = false, bool LIST = false,
          typename O = T, unsigned NT = kRecursionThreads, bool TOGETHER = false>
__global__ __launch_bounds__(NT, MODE < 2 ? 4 : 1) void recursion_kernel(Tiling g, const O* __restrict__ xyz,
                                                                     O* __restrict__ sph,
                                                                     O* __restrict__ dsph,
                                                                     O* __restrict__ ddsph) {
    static_assert(!VJP || (MODE == 1 && !SPLIT), "the fused product is built on the gradient kernel");
    static_assert(!VJP || std::is_same<T, O>::value, "the fused product stages what it computes");
    static_assert(!TOGETHER || sizeof(T) == 8, "float32 has the recursions in the flush only");
    constexpr int H = MODE == 2 ? 1 : 6;
    constexpr unsigned NYH = (H + 1) * (H + 1);
    constexpr unsigned ARRAYS = MODE + 1; // iterate arrays per point: A, B, C
    // the row buffers, rows of O, come first; everything else is T and counts from g.tables_at
    O* row_lds = reinterpret_cast<O*>(lds_raw);
    T* lds = reinterpret_cast<T*>(lds_raw + g.tables_at);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6); // the same for all lanes: scalar
    const int L = g.l_max;
    const unsigned S = g.tile;
    const unsigned ny = g.ny;
    const unsigned nrow = WHOLE ? ny : ny - NYH; // staged elements per component row
    const unsigned skip = WHOLE ? 0u : NYH;      // first staged entry of a row
    // Distance between staged rows. WHOLE == false: the rows are ny apart in HBM but only nrow
    // long; a stride that equals ny modulo 16 bytes, with the first row placed like its HBM
    // address modulo 16 bytes, puts every staged row at the same position within 16 bytes as
    // its destination, so that the copy is 16-byte loads and stores on both sides.
    constexpr unsigned W16 = 16u / static_cast<unsigned>(sizeof(O));
    // WHOLE, rows a multiple of 64 bytes long (l_max = 3 mod 4): every row would start on the same LDS bank, and
    // whatever takes one point per lane (the closed forms above all) would store all its lanes' numbers to one
    // bank, one after the other (float32 gradients l_max = 11: 59 % of the HBM peak against 66 % at l_max = 10
    // and 12). The host then asks for 16 bytes between the staged rows, g.row_pad elements; the flush skips them
    // (flush_run). They keep a row's 16-byte vectors whole only where the arrays start at multiples of 16 bytes:
    // for other pointers the rows stay back to back.
    const unsigned row_pad =
        WHOLE && !VJP && ((reinterpret_cast<uintptr_t>(sph) | reinterpret_cast<uintptr_t>(dsph) |
                           reinterpret_cast<uintptr_t>(ddsph)) & 15u) == 0
            ? g.row_pad
            : 0u;
    const unsigned row_stride = WHOLE ? nrow + row_pad : nrow + skip % W16;
    const unsigned tri_all = (L + 1) * (L + 2) / 2;

    T* F = lds + g.off_F;
    T* Q = lds + g.off_Q;
    unsigned* job_table = reinterpret_cast<unsigned*>(lds + g.off_jobs);
    {
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        for (unsigned i = tid; i < tri_all; i += NT) {
            F[i] = cF[i];
            Q[i] = cQ[i];
        }
        // (l, m) pairs: the bulk 1 <= m <= l - 2 first, then the special cases m = l, l - 1 and
        // 0 each as one block, so that the lanes of a wave mostly share one branch of entry_job
        // one word per job: m in bits 0-6, the side in bit 7, l in bits 8-15, l(l+1)/2 above
        auto pack = [](int l, int m, int side) -> unsigned {
            return (static_cast<unsigned>(l * (l + 1) / 2) << 16) | (static_cast<unsigned>(l) << 8) |
                   (static_cast<unsigned>(side) << 7) | static_cast<unsigned>(m);
        };
        // one thread per l fills that l's places (a single thread writing all of them took
        // 10 us at l_max = 32, a third of the time of a small evaluation)
        // Jobs point by point, a point's jobs in more rounds than one: in a point's last round
        // the kinds other than the bulk start with a wave of their own where the lanes allow it
        // (the host says where), and the places in between hold no job. A wave runs the branch
        // of every kind it holds, one after the other: at l_max = 32 the third of five entry
        // waves held the end of the bulk and all three other kinds, and every tile waited for it
        // (7 100 cycles against 3 300-4 900 for the other four).
        const bool spread = !SPLIT && !LIST && g.kind_at[0] != 0;
        if (spread) {
            for (unsigned i = tid; i < g.jobs_per_point; i += NT) job_table[i] = kNoJob;
            __syncthreads();
        }
        if (static_cast<int>(tid) < L - H) {
            constexpr unsigned SIDES = SPLIT ? 2u : 1u;
            const int l = L - static_cast<int>(tid);
            const unsigned levels = static_cast<unsigned>(L - H);
            auto bulk_above = [&](int from) { // sum of (l' - 2) over from < l' <= L
                return static_cast<unsigned>(L * (L + 1) / 2 - from * (from + 1) / 2 - 2 * (L - from));
            };
            const unsigned bulk_all = bulk_above(H);
            for (unsigned side = 0; side < SIDES; ++side) {
                unsigned at = side * bulk_all + bulk_above(l);
                for (int m = l - 2; m >= 1; --m) job_table[at++] = pack(l, m, static_cast<int>(side));
                const unsigned at_l = spread ? g.kind_at[0] : SIDES * bulk_all + side * levels;
                const unsigned at_l1 = spread ? g.kind_at[1] : SIDES * (bulk_all + levels) + side * levels;
                job_table[at_l + tid] = pack(l, l, static_cast<int>(side));
                job_table[at_l1 + tid] = pack(l, l - 1, static_cast<int>(side));
            }
            job_table[(spread ? g.kind_at[2] : SIDES * (bulk_all + 2 * levels)) + tid] = pack(l, 0, 0);
        }
    }

    // per point: 8 numbers (x, y, z, x^2, y^2, z^2, 1/r, x^2 + y^2), then c, s, 2(m+1)z
    // (both strides odd: lanes of the sequence waves work on different points and sequences
    // at once, and a stride with a power of two in it puts them on a few LDS banks: at l_max = 31
    // the iterates of neighbouring sequences were 528 words apart, 16 modulo the 32 banks)
    const unsigned point_stride = (8 + 3 * (L + 1)) | 1u;
    const unsigned iterate_stride = tri_all | 1u;
    // The tables are made for 2^az_shift tiles at a time (a batch), one lane per point, so that
    // the recurrences, a chain of dependent operations that few lanes share, run once per batch
    // instead of once per tile. Single tiles are made two tiles ahead (the recursions of the
    // next tile run in the same phase and read the one in between), batches one batch ahead;
    // two buffers either way, since a tile's tables are done with when its entries are
    // (TOGETHER: the entries of a tile run in that phase too, three buffers for single tiles).
    const unsigned batch_tiles = 1u << g.az_shift;
    const unsigned batch_lead = batch_tiles == 1 ? 2u : 1u;
    const unsigned batch_buffers = TOGETHER && batch_tiles == 1 ? 3u : 2u;
    auto point_data = [&](unsigned n, unsigned s) -> T* { // point s of this workgroup's n-th tile
        const unsigned slot = (((n >> g.az_shift) % batch_buffers) << g.az_shift) | (n & (batch_tiles - 1u));
        return lds + g.off_pts + (slot * S + s) * point_stride;
    };
    auto iterates = [&](unsigned n, unsigned s, unsigned which, int l) -> T* { // of this workgroup's n-th tile
        const unsigned buffer = TOGETHER ? n & 1u : 0u;
        return lds + g.off_iter + ((buffer * S + s) * ARRAYS + which) * iterate_stride + l * (l + 1) / 2;
    };

    // same XCD-contiguous walk as the closed-form kernel
    const unsigned xcd = blockIdx.x & 7u;
    const unsigned rank_in_xcd = blockIdx.x >> 3;
    const unsigned groups_per_xcd = gridDim.x >> 3;
    const unsigned xcd_first = xcd * g.tiles_per_xcd;
    unsigned xcd_last = xcd_first + g.tiles_per_xcd;
    if (xcd_last > g.n_tiles) xcd_last = g.n_tiles;
    // A workgroup takes chunks of C consecutive tiles; the chunks of an XCD's workgroups lie
    // side by side. Consecutive tiles in one workgroup share the 128-byte lines in which one
    // ends and the next begins (see flush_run); C stays small so that what the XCD writes at any
    // moment remains a compact window.
    const unsigned chunk_mask = (1u << g.chunk_shift) - 1u;

    // WHOLE == false with g.prefix_inside: l <= H of every row is written by this launch as well,
    // by wave 0, which otherwise waits at the barriers most of the time. 64 points at a time, one
    // per lane, the entries in eight slices straight from registers to HBM: the runs are 196 or
    // 392 bytes long, one per component row, so staging them would not make the stores any
    // better. The batches of 64 points are dealt to the workgroups of the launch and have
    // nothing to do with the tiles a workgroup walks; one call takes one slice of one batch.
    [[maybe_unused]] unsigned prefix_next = 0;
    [[maybe_unused]] auto prefix_slice = [&]() -> bool {
        if constexpr (!WHOLE && !VJP && H == 6) {
            const unsigned long long first =
                (static_cast<unsigned long long>(prefix_next >> 3) * gridDim.x + blockIdx.x) * 64u;
            if (first >= g.n_samples) return false;
            const unsigned slice = prefix_next & 7u;
            ++prefix_next;
            const unsigned long long i = first + lane;
            if (i < g.n_samples) {
                const Point<T> p = load_point<T, NORM>(xyz + i * 3);
                Rows<O> rows;
                rows.ny = static_cast<int>(ny);
                rows.sph = sph + i * ny;
                rows.dsph = MODE >= 1 ? dsph + i * 3 * ny : nullptr;
                rows.ddsph = nullptr;
                switch (slice) {
                case 0: closed_form_job<T, MODE, NORM, H, 0, 9>(p, rows); break;
                case 1: closed_form_job<T, MODE, NORM, H, 9, 16>(p, rows); break;
                case 2: closed_form_job<T, MODE, NORM, H, 16, 25>(p, rows); break;
                case 3: closed_form_job<T, MODE, NORM, H, 25, 31>(p, rows); break;
                case 4: closed_form_job<T, MODE, NORM, H, 31, 36>(p, rows); break;
                case 5: closed_form_job<T, MODE, NORM, H, 36, 41>(p, rows); break;
                case 6: closed_form_job<T, MODE, NORM, H, 41, 45>(p, rows); break;
                default: closed_form_job<T, MODE, NORM, H, 45, 49>(p, rows); break;
                }
            }
            return true;
        } else {
            return false;
        }
    };
    const bool prefix_wave = !WHOLE && !VJP && H == 6 && g.prefix_inside != 0 && wave == 0;

    if (xcd_first + (rank_in_xcd << g.chunk_shift) >= xcd_last) {
        // no tiles for this workgroup; its share of the batches remains
        if (prefix_wave) {
            while (prefix_slice()) {
            }
        }
        return;
    }

    // the n-th tile of this workgroup, and how many points it has (0 past the end)
    auto tile_of = [&](unsigned n) -> unsigned {
        return xcd_first + ((((n >> g.chunk_shift) * groups_per_xcd + rank_in_xcd)) << g.chunk_shift) +
               (n & chunk_mask);
    };
    auto valid_in = [&](unsigned n) -> unsigned {
        const unsigned t = tile_of(n);
        if (t >= xcd_last) return 0u;
        const unsigned long long first = static_cast<unsigned long long>(t) * S;
        const unsigned long long left = g.n_samples - first;
        return left < S ? static_cast<unsigned>(left) : S;
    };
    // lane j of wave 0 takes point j % S of tile j / S of a batch (batch_tiles * S <= 64)
    auto fetch = [&](unsigned batch, T& rx, T& ry, T& rz) {
        rx = ry = rz = 0;
        const unsigned n = (batch << g.az_shift) + lane / S;
        const unsigned s = lane % S;
        if (lane < batch_tiles * S && s < valid_in(n)) {
            const O* src = xyz + (static_cast<unsigned long long>(tile_of(n)) * S + s) * 3;
            rx = static_cast<T>(src[0]);
            ry = static_cast<T>(src[1]);
            rz = static_cast<T>(src[2]);
        }
    };
    // stage one of a batch of tiles (wave 0; lane == tid there)
    auto azimuth_stage = [&](unsigned batch, T rx, T ry, T rz) {
        const unsigned n = (batch << g.az_shift) + lane / S;
        const unsigned s = lane % S;
        if (lane < batch_tiles * S && s < valid_in(n)) {
            T* rec = point_data(n, s);
            Point<T> p;
            p.x = rx;
            p.y = ry;
            p.z = rz;
            p.x2 = p.x * p.x;
            p.y2 = p.y * p.y;
            p.z2 = p.z * p.z;
            p.ir = 0.0;
            if constexpr (NORM) {
                p.ir = 1 / root(p.x2 + p.y2 + p.z2);
                p.x *= p.ir;
                p.y *= p.ir;
                p.z *= p.ir;
                p.x2 = p.x * p.x;
                p.y2 = p.y * p.y;
                p.z2 = p.z * p.z;
            }
            rec[0] = p.x;
            rec[1] = p.y;
            rec[2] = p.z;
            rec[3] = p.x2;
            rec[4] = p.y2;
            rec[5] = p.z2;
            rec[6] = p.ir;
            rec[7] = p.x2 + p.y2;
            azimuth_job<T>(p, L, rec + 8, rec + 8 + (L + 1), rec + 8 + 2 * (L + 1));
        }
    };
    // the recursions of tile n (waves 1 .. g.sequence_waves)
    auto recursion_stage = [&](unsigned n) {
        const unsigned count = valid_in(n);
        const unsigned per_l = count * ARRAYS;
        const unsigned jobs = per_l * static_cast<unsigned>(L - H);
        for (unsigned j = tid - 64; j < jobs; j += 64 * g.sequence_waves) { // waves 1 .. sequence_waves
            const unsigned step = j / per_l;
            const unsigned rest = j - step * per_l;
            const int l = L - static_cast<int>(step); // longest recursions first
            const unsigned s = rest / ARRAYS;
            const unsigned which = rest - s * ARRAYS;
            const T* rec = point_data(n, s);
            sequence_job<T>(l, static_cast<int>(which), rec[2], rec[7], Q, rec + 8 + 2 * (L + 1),
                            iterates(n, s, which, l));
        }
    };

    // wave 0 and the sequence waves prepare the next tiles
    const unsigned apart_waves = 1 + g.sequence_waves;
    // All waves but the slice waves, the last ones, compute entries (TOGETHER: the waves in between).
    const unsigned entry_first_wave = TOGETHER ? apart_waves : 0u;
    const unsigned entry_end_wave = NT / 64 - g.slice_waves;
    const unsigned wide_first = 64 * entry_first_wave;
    const unsigned wide_lanes = 64 * (entry_end_wave - entry_first_wave);

    constexpr unsigned LINE = 128u / static_cast<unsigned>(sizeof(O)); // elements per 128-byte line
    // position within its 128-byte line of element `element` of an output array
    auto phase_of = [](const O* array, unsigned long long element) -> unsigned {
        return static_cast<unsigned>((reinterpret_cast<uintptr_t>(array) / sizeof(O) + element) % LINE);
    };

    // Where the rows of tile n start within their staging regions. WHOLE: element 0 of a region
    // stands for the start of the 128-byte line in which the tile's run begins in HBM, so the run
    // itself starts `phase` elements in. WHOLE == false: position within 16 bytes of the first
    // staged row, see row_stride. VJP: the rows never leave LDS, no position to match.
    struct Phases {
        unsigned sph, dsph, ddsph;
    };
    auto phases_of = [&](unsigned n) -> Phases {
        const unsigned long long first_point = static_cast<unsigned long long>(tile_of(n)) * S;
        Phases ph;
        ph.sph = VJP ? 0u : phase_of(sph, first_point * ny + skip) % (WHOLE ? LINE : W16);
        ph.dsph = VJP || MODE < 1 ? 0u : phase_of(dsph, first_point * 3 * ny + skip) % (WHOLE ? LINE : W16);
        ph.ddsph = WHOLE && !VJP && MODE == 2 ? phase_of(ddsph, first_point * 9 * ny) : 0u;
        return ph;
    };

    // WHOLE: the closed forms of tile n, one lane per point, into the staged rows. The
    // entries of a point are cut in slices (by l), dealt to `among` waves of which this is number
    // `who`, so that no single wave carries all of the chain rule and staging.
    auto closed_stage = [&](unsigned n, unsigned who, unsigned among) {
        if constexpr (WHOLE) {
            const unsigned valid = valid_in(n);
            if (lane < valid) {
                O* staged = row_lds;
                const Phases ph = phases_of(n);
                const T* rec = point_data(n, lane);
                Point<T> p;
                p.x = rec[0];
                p.y = rec[1];
                p.z = rec[2];
                p.x2 = rec[3];
                p.y2 = rec[4];
                p.z2 = rec[5];
                p.ir = rec[6];
                Rows<O> rows;
                rows.ny = static_cast<int>(row_stride);
                rows.sph = staged + ph.sph + lane * row_stride;
                rows.dsph = staged + g.off_dsph + ph.dsph + lane * 3 * row_stride;
                rows.ddsph = staged + g.off_ddsph + ph.ddsph + lane * 9 * row_stride;
                if constexpr (H == 6) {
                    // (Rows a multiple of 32 words long, l_max = 7, 15, 23, ...: the stores of all
                    // lanes fall on one LDS bank. Storing in rotated fours, two selects per number,
                    // paid for tiles of many points, l_max = 15 with 23 points 270 us against 298
                    // per 1.2 GB, and cost more than the conflicts from ten points down, l_max = 23,
                    // 31, 39 269, 312, 345 us against 266, 258, 269; without that code the kernel
                    // needs fewer registers, l_max = 32: 732 -> 710 us. It is gone.)
                    if (0 % among == who) closed_form_job<T, MODE, NORM, H, 0, 9>(p, rows);
                    if (1 % among == who) closed_form_job<T, MODE, NORM, H, 9, 16>(p, rows);
                    if (2 % among == who) closed_form_job<T, MODE, NORM, H, 16, 25>(p, rows);
                    if (3 % among == who) closed_form_job<T, MODE, NORM, H, 25, 31>(p, rows);
                    if (4 % among == who) closed_form_job<T, MODE, NORM, H, 31, 36>(p, rows);
                    if (5 % among == who) closed_form_job<T, MODE, NORM, H, 36, 41>(p, rows);
                    if (6 % among == who) closed_form_job<T, MODE, NORM, H, 41, 45>(p, rows);
                    if (7 % among == who) closed_form_job<T, MODE, NORM, H, 45, 49>(p, rows);
                } else {
                    // (l <= 1: four entries, the chain rule of each is most of its work)
                    if (0 % among == who) closed_form_job<T, MODE, NORM, H, 0, 1>(p, rows);
                    if (1 % among == who) closed_form_job<T, MODE, NORM, H, 1, 2>(p, rows);
                    if (2 % among == who) closed_form_job<T, MODE, NORM, H, 2, 3>(p, rows);
                    if (3 % among == who) closed_form_job<T, MODE, NORM, H, 3, 4>(p, rows);
                }
            }
        }
    };

    // the entries of tile n (the entry waves)
    auto entry_stage = [&](unsigned n) {
        const unsigned valid = valid_in(n);
        O* staged = row_lds;
        const unsigned t = tid - wide_first;
        const Phases ph = phases_of(n);
        const unsigned phase_sph = ph.sph, phase_dsph = ph.dsph, phase_ddsph = ph.ddsph;
        // what depends on the point only
        Point<T> p;
        p.x = p.y = p.z = p.x2 = p.y2 = p.z2 = p.ir = 0;
        const T* c = nullptr;
        const T* sn = nullptr;
        const T* itA = nullptr;
        const T* itB = nullptr;
        const T* itC = nullptr;
        Rows<O> rows;
        rows.ny = static_cast<int>(row_stride);
        rows.sph = rows.dsph = rows.ddsph = nullptr;
        auto take_point = [&](unsigned s) {
            const T* rec = point_data(n, s);
            p.x = rec[0];
            p.y = rec[1];
            p.z = rec[2];
            p.x2 = rec[3];
            p.y2 = rec[4];
            p.z2 = rec[5];
            p.ir = rec[6];
            c = rec + 8;
            sn = rec + 8 + (L + 1);
            itA = iterates(n, s, 0, 0);
            itB = iterates(n, s, MODE >= 1 ? 1 : 0, 0);
            itC = iterates(n, s, MODE == 2 ? 2 : 0, 0);
            // rows are addressed with the entry's index in the full row; shift the bases when
            // the staged rows start at l = H + 1
            rows.sph = staged + phase_sph + s * row_stride - skip;
            rows.dsph = staged + g.off_dsph + phase_dsph + s * 3 * row_stride - skip;
            rows.ddsph = staged + g.off_ddsph + phase_ddsph + s * 9 * row_stride - skip;
        };
        auto take_job = [&](unsigned e) {
            const unsigned packed = job_table[e];
            if constexpr (!LIST && !SPLIT) {
                if (packed == kNoJob) return;
            }
            const int m = static_cast<int>(packed & 0x7fu);
            const int side = static_cast<int>((packed >> 7) & 1u);
            const int l = static_cast<int>((packed >> 8) & 0xffu);
            const int tri = static_cast<int>(packed >> 16);
            entry_job<T, MODE, NORM, SPLIT>(l, m, tri, side, p, F + tri, c, sn, itA + tri, itB + tri,
                                            itC + tri, rows);
        };
        const unsigned per_point = g.jobs_per_point;
        if constexpr (LIST) {
            // The jobs of the tile's points as one list, dealt to the wide lanes round after
            // round: only the last round can leave lanes idle (l_max = 20: 203 jobs per point on
            // 320 lanes, seven points in five rounds instead of seven); a lane looks at every
            // job's point. (Both loops in one kernel made either slower by some 5 %.)
            // With derivatives the list is ordered by kind first (the bulk of all points, then |m| = l of all
            // points, |m| = l - 1, m = 0) and by point within a kind, so that the lanes of a wave
            // share a branch of entry_job except where two kinds meet: three places per tile
            // instead of three per point.
            const unsigned total = valid * per_point;
            if constexpr (MODE == 0) {
                // values: an entry is three multiplications, the order by kind does not pay
                // (float32 l_max = 40, 400k points: 824 us point after point, 889 us by kind)
                unsigned current = ~0u;
                for (unsigned q = t; q < total; q += wide_lanes) {
                    const unsigned s = __umulhi(q, g.magic_jobs); // exact: q * per_point < 2^32
                    if (s != current) {
                        current = s;
                        take_point(s);
                    }
                    take_job(q - s * per_point);
                }
                return;
            }
            // (read into scalar registers here: picked by index inside the loop, the members of g
            // would be copied to scratch memory and fetched from there job by job, and a wave that
            // waits for such a load also waits for the stores of its last flush)
            const unsigned b0 = __builtin_amdgcn_readfirstlane(g.kind_jobs[0]);
            const unsigned b1 = __builtin_amdgcn_readfirstlane(g.kind_jobs[1]);
            const unsigned b3 = __builtin_amdgcn_readfirstlane(g.kind_jobs[2]);
            const unsigned magic0 = __builtin_amdgcn_readfirstlane(g.kind_magic[0]);
            const unsigned magic1 = __builtin_amdgcn_readfirstlane(g.kind_magic[1]);
            const unsigned magic3 = __builtin_amdgcn_readfirstlane(g.kind_magic[2]);
            const unsigned t1 = valid * b0, t2 = t1 + valid * b1, t3 = t2 + valid * b1;
            unsigned current = ~0u;
            for (unsigned q = t; q < total; q += wide_lanes) {
                unsigned r, b, first_job, magic;
                if (q < t1) {
                    r = q, b = b0, first_job = 0, magic = magic0;
                } else if (q < t2) {
                    r = q - t1, b = b1, first_job = b0, magic = magic1;
                } else if (q < t3) {
                    r = q - t2, b = b1, first_job = b0 + b1, magic = magic1;
                } else {
                    r = q - t3, b = b3, first_job = b0 + 2 * b1, magic = magic3;
                }
                // exact: r * b < 2^32; a single job per point has no such multiplier in 32 bits
                const unsigned s = b == 1 ? r : __umulhi(r, magic);
                if (s != current) {
                    current = s;
                    take_point(s);
                }
                take_job(first_job + (r - s * b));
            }
        } else {
            // One pass takes the jobs of as many points as fit side by side in the wide lanes
            // (of one point, in several rounds, when it has more jobs than there are lanes);
            // what depends on the point only is read once per pass.
            unsigned local = 0, e_first = t;
            if (g.points_per_pass > 1) {
                local = __umulhi(t, g.magic_jobs);
                e_first = t - local * per_point;
            }
            for (unsigned s0 = 0; s0 < valid; s0 += g.points_per_pass) {
                const unsigned s = s0 + local;
                if (s >= valid || local >= g.points_per_pass) continue;
                take_point(s);
                for (unsigned e = e_first; e < per_point; e += wide_lanes) take_job(e);
            }
        }
    };

    // last stage of tile n: the staged rows to HBM, by `count` threads of which this is number
    // `ft`. (With all waves of the workgroup on one run, loads and stores alternating one by one
    // measured faster than several loads in flight per wave.)
    auto flush_stage = [&](unsigned n, unsigned ft, unsigned count) {
        const unsigned valid = valid_in(n);
        const unsigned long long first = static_cast<unsigned long long>(tile_of(n)) * S;
        const O* staged = row_lds;
        if constexpr (WHOLE) {
            // The tile's run of `len` elements of one output array starts at element `at` of that
            // array. Only whole 128-byte lines go out with vector stores. The line in which the
            // run ends is completed by the next tile: when that tile is this workgroup's next one
            // (same chunk), the unfinished part is carried over into the region the next tile is
            // staged in; at the ends of a chunk the partial lines are stored element by element.
            const bool starts = (n & chunk_mask) == 0;
            const bool ends = (n & chunk_mask) == chunk_mask || valid_in(n + 1) == 0;
            O* carry_to = row_lds;
            auto flush_run = [&](unsigned region_offset, O* array, unsigned long long at, unsigned len) {
                using V = typename Pack<O>::type;
                constexpr unsigned W = Pack<O>::width;
                O* region = row_lds + region_offset;
                const unsigned phase = phase_of(array, at);
                O* line0 = array + (at - phase); // HBM address of region element 0
                const unsigned lo = starts ? phase : 0u; // first element that holds data
                const unsigned hi = phase + len;
                const unsigned full_lo = (lo + LINE - 1u) / LINE * LINE;
                const unsigned full_hi = hi / LINE * LINE;
                // where element e of the region (counted as it lies in HBM) is staged: past the carried part of
                // the first line, row_pad elements further for every row before it (exact: e * ny < 2^32)
                auto staged_at = [&](unsigned e) -> unsigned {
                    return row_pad == 0 || e < phase ? e : e + row_pad * __umulhi(e - phase, g.magic_ny);
                };
                unsigned tail_from; // what follows the head and the whole lines
                if (full_hi > full_lo) {
                    const unsigned nvec = (full_hi - full_lo) / W;
                    V* out = reinterpret_cast<V*>(line0 + full_lo);
                    // (two or four loads in flight per lane ahead of their stores: no faster on any shape)
                    for (unsigned v = ft; v < nvec; v += count) {
                        emit<O, SPHX_STREAMING_STORES>(*reinterpret_cast<const V*>(region + staged_at(full_lo + v * W)),
                                                       out + v);
                    }
                    tail_from = full_hi;
                } else {
                    tail_from = full_lo < hi ? full_lo : hi;
                }
                // head: the part of the first line that belongs to this chunk
                const unsigned head_end = full_lo < hi ? full_lo : hi;
                if (lo + ft < head_end) line0[lo + ft] = region[staged_at(lo + ft)];
                // tail: stored if the chunk ends here, else handed to the next tile
                const unsigned tail = hi - tail_from;
                if (ft < tail) {
                    const O value = region[staged_at(tail_from + ft)];
                    if (ends) {
                        line0[tail_from + ft] = value;
                    } else if (carry_to + region_offset != region || staged_at(tail_from + ft) != ft) {
                        carry_to[region_offset + ft] = value;
                    }
                }
            };
            flush_run(0, sph, first * ny, valid * ny);
            if constexpr (MODE >= 1) flush_run(g.off_dsph, dsph, first * 3 * ny, valid * 3 * ny);
            if constexpr (MODE == 2) flush_run(g.off_ddsph, ddsph, first * 9 * ny, valid * 9 * ny);
        } else {
            // one run per (point, component) row, dealt to the waves in turn. In float64 the
            // vector stores start at a line boundary of the row (l_max = 20 gradients, 100k
            // points: 491 -> 381 us); in float32 that measured the same or 2 % worse.
            constexpr bool LINES = sizeof(O) == 8;
            const unsigned waves = count / 64;
            for (unsigned r = __builtin_amdgcn_readfirstlane(ft >> 6); r < valid * components_of(MODE); r += waves) {
                // rows [0, valid) are values, the next 3 * valid are gradients
                if (r < valid) {
                    copy_out<O, SPHX_STREAMING_STORES, false, SPHX_FLUSH_UNROLL, LINES>(
                        staged + phase_of(sph, first * ny + skip) % W16 + r * row_stride,
                        sph + (first + r) * ny + skip, nrow, nrow, 0, 0, ft & 63u, 64);
                } else {
                    const unsigned q = r - valid;
                    copy_out<O, SPHX_STREAMING_STORES, false, SPHX_FLUSH_UNROLL, LINES>(
                        staged + g.off_dsph + phase_of(dsph, first * 3 * ny + skip) % W16 + q * row_stride,
                        dsph + (first * 3 + q) * ny + skip, nrow, nrow, 0, 0, ft & 63u, 64);
                }
            }
        }
    };

    // VJP: in place of the flush. `sph` holds the upstream gradient sph_grad[N][ny] (read
    // only), `dsph` is xyz_grad[N][3]. Wave 1 + r takes gradient row r of the tile (point r / 3,
    // component r % 3): its lanes multiply the staged entries with the point's row of sph_grad
    // and a butterfly adds the lanes' sums up. With WHOLE == false the staged rows begin at
    // l = H + 1 and closed_form_vjp_kernel has already stored the sum over l <= H, so the
    // result is added to what xyz_grad holds. By `among` waves of which this is number `who`.
    auto contract_stage = [&](unsigned n, unsigned who, unsigned among) {
        if constexpr (VJP) {
            const unsigned valid = valid_in(n);
            const unsigned long long first = static_cast<unsigned long long>(tile_of(n)) * S;
            const T* staged = row_lds + g.off_dsph; // O is T here
            const T* upstream = sph;
            T* xyz_grad = dsph;
            for (unsigned r = who; r < valid * 3; r += among) {
                const unsigned s = r / 3;
                const T* row = staged + r * row_stride - skip; // indexed with the entry's index in the full row
                const T* weight = upstream + (first + s) * ny;
                T partial = 0;
#pragma unroll 4
                for (unsigned k = skip + lane; k < ny; k += 64) {
                    partial += row[k] * weight[k];
                }
                for (unsigned offset = 32; offset > 0; offset >>= 1) {
                    partial += __shfl_xor(partial, static_cast<int>(offset));
                }
                if (lane == 0) {
                    T* out = xyz_grad + first * 3 + r;
                    *out = (!WHOLE || g.vjp_accumulate) ? *out + partial : partial;
                }
            }
        }
    };

    // fill the pipeline: tables of tiles 0 and 1, iterates of tile 0
    T rx = 0, ry = 0, rz = 0;
    if (wave == 0) {
        fetch(0, rx, ry, rz);
        azimuth_stage(0, rx, ry, rz);
        fetch(1, rx, ry, rz);
    }
    __syncthreads(); // prefactor tables, job table, tables of batch 0
    if (wave == 0) {
        if (batch_lead == 2) {
            azimuth_stage(1, rx, ry, rz);
            fetch(2, rx, ry, rz);
        }
    } else if (wave < apart_waves) {
        recursion_stage(0);
    }

    // wave 0's part of tile n: the tables of a batch ahead, a slice of the rows that start at l = 7
    auto table_stage = [&](unsigned n) {
        if ((n & (batch_tiles - 1u)) == 0) {
            azimuth_stage((n >> g.az_shift) + batch_lead, rx, ry, rz);
            fetch((n >> g.az_shift) + batch_lead + 1, rx, ry, rz);
        }
        if (prefix_wave) prefix_slice();
    };
    for (unsigned n = 0; valid_in(n) != 0; ++n) {
        __syncthreads(); // iterates of tile n in place; rows of tile n-1 flushed
        // The closed-form slices go round all waves, or to the waves set aside for them when the waves that had a
        // slice on top of their jobs were what the tile waited for. Round all waves: the last wave first (the jobs
        // are dealt from lane 0 up, so that the last waves are the ones a short last round leaves idle); TOGETHER:
        // the first wave first, the waves that make tables and iterates have time to spare.
        if (g.slice_waves == 0) {
            closed_stage(n, TOGETHER ? wave : NT / 64 - 1 - wave, NT / 64);
        } else if constexpr (TOGETHER) {
            if (wave == 0 || wave >= entry_end_wave) {
                closed_stage(n, wave == 0 ? 0u : wave - entry_end_wave + 1u, g.slice_waves + 1u);
            }
        } else if (wave >= entry_end_wave) {
            closed_stage(n, wave - entry_end_wave, g.slice_waves);
        }
        if constexpr (TOGETHER) {
            if (wave == 0) {
                table_stage(n);
            } else if (wave < apart_waves) {
                recursion_stage(n + 1);
            }
        }
        if (wave >= entry_first_wave && wave < entry_end_wave) entry_stage(n);
        __syncthreads(); // rows of tile n complete, its tables and iterates done with
        if constexpr (TOGETHER) {
            if constexpr (VJP) {
                if (wave != 0) contract_stage(n, wave - 1, NT / 64 - 1); // (wave 0 has loads in flight)
            } else {
                flush_stage(n, tid, NT);
            }
        } else if (wave == 0) {
            if (g.priorities & 2u) __builtin_amdgcn_s_setprio(2);
            table_stage(n);
            __builtin_amdgcn_s_setprio(0);
        } else if (wave < apart_waves) {
            if (g.priorities & 2u) __builtin_amdgcn_s_setprio(2);
            recursion_stage(n + 1);
            __builtin_amdgcn_s_setprio(0);
        } else if constexpr (VJP) {
            contract_stage(n, wave - apart_waves, NT / 64 - apart_waves);
        } else {
            if (g.priorities & 1u) __builtin_amdgcn_s_setprio(2);
            flush_stage(n, tid - 64 * apart_waves, NT - 64 * apart_waves);
            __builtin_amdgcn_s_setprio(0);
        }
    }
    // what is left of this workgroup's share of the batches (no barrier follows)
    if (prefix_wave) {
        while (prefix_slice()) {
        }
    }
}

} // namespace sphx

#endif

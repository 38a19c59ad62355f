// pairs_kernel: derivatives beyond the closed forms, every entry lane bound to one (l, m) pair for the
// whole launch. MODE 1: values and gradients; MODE 2: second derivatives too.
#ifndef SPHX_PAIRS_KERNEL_HPP
#define SPHX_PAIRS_KERNEL_HPP

#include <hip/hip_runtime.h>

#include <cstdint>

#include "sphx_device.hpp"
#include "sphx_pairs_tiling.hpp"

namespace sphx {

// ---------------------------------------------------------------------------
// Persistent workgroups of up to sixteen waves, one per CU, that walk over tiles of `tile`
// consecutive points; a tile's rows are staged in LDS in HBM layout and flushed as whole
// 128-byte lines. A tile round has two halves, the stage (rows are filled) and the flush (rows
// go to HBM), and the waves have roles:
//
//   entry waves     stage: lane j keeps the pair (l, m >= 1) that the host's lane table gives it
//                   for the whole launch. Its prefactors, its multipliers and the positions of
//                   its entries within a row are registers; per point it reads the point's
//                   coordinates, the iterates around (l, m) and (c_{m-1}, s_{m-1}, c_m, s_m) with
//                   three 16-byte reads, one point ahead of the arithmetic, and stages the entries
//                   (l, +-m) of every array. Nothing is decoded per job: the stage is bound by
//                   the issue of vector instructions, and every one that is not arithmetic of
//                   the reference counts.
//                   Flush: these waves stream the rows out.
//   sequence waves  flush: one lane per (point, l, sequence) of the next tile, the bare Q
//                   recursions, the iterates of the two sequences of one l interleaved in LDS.
//   prep waves      stage: the closed forms of l <= 6 of the tile from a parking area into the
//                   rows, and the entries with m = 0. Flush: one lane per point of a *batch* of
//                   several tiles, one batch ahead: normalised coordinates, (c_m, s_m) pairs and
//                   2(m+1)z into the point's record, and the closed forms in slices into the
//                   parking area, one work item per tile round.
//
// While the rows are flushed the vector ALUs would idle, and while they are filled the path to
// memory would: everything that does not need the rows runs during the flush.
//
// Arithmetic: templates_core.hpp:122-152, :154-198, :201-294 and :392-426 of the reference
// through the same expressions as entry_job (sphx_device.hpp), the chain rule of
// templates.hpp:553-614 through finish(); same operations in the same order, hence the same
// numbers. With second derivatives (closed forms only to l = 1, three recursions per l, thirteen
// rows per point) the entries are entry_job itself, fed from registers, and nothing is parked: the
// prep waves evaluate the closed forms of l <= 1 straight into the rows.
// ---------------------------------------------------------------------------
extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

// (c_m, s_m) pairs and 2(m+1)z of one point; templates.hpp:451-466 (see azimuth_job)
template <typename T>
__device__ __forceinline__ void azimuth_pairs_job(const Point<T>& p, int L, T* cs, T* tmz) {
    T twoz = p.z + p.z;
    T cm = 1.0, sm = 0.0, tz = twoz;
    cs[0] = cm;
    cs[1] = sm;
    tmz[0] = tz;
    for (int m = 1; m <= L; ++m) {
        T cn = cm * p.x - sm * p.y;
        T sn = cm * p.y + sm * p.x;
        tz = tz + twoz;
        cm = cn;
        sm = sn;
        cs[2 * m] = cm;
        cs[2 * m + 1] = sm;
        tmz[m] = tz;
    }
}

// The inputs of entry_job_from (sphx_device.hpp) in registers: what a lane has read around its own m.
template <typename T> struct EntryWindow {
    T pk_;
    T c_[3], s_[3];   // at m - 2, m - 1, m
    T A_[2], B_[2];   // at m, m + 1
    T C_[3];          // at m, m + 1, m + 2
    __device__ __forceinline__ T pk() const { return pk_; }
    __device__ __forceinline__ T c(int d) const { return c_[2 + d]; }
    __device__ __forceinline__ T s(int d) const { return s_[2 + d]; }
    __device__ __forceinline__ T A(int d) const { return A_[d]; }
    __device__ __forceinline__ T B(int d) const { return B_[d]; }
    __device__ __forceinline__ T C(int d) const { return C_[d]; }
};

template <typename T> struct Pair2;
template <> struct Pair2<float> {
    typedef float type __attribute__((ext_vector_type(2)));
};
template <> struct Pair2<double> {
    typedef double type __attribute__((ext_vector_type(2)));
};

// NT: the most threads a workgroup may have. 1024 leaves a lane 128 registers; the entries with second
// derivatives need more and run in workgroups of 512.
template <typename T, int MODE, bool NORM, unsigned NT = kPairsThreads, typename O = T>
__global__ __launch_bounds__(NT, 1) void pairs_kernel(PairsTiling g, const T* __restrict__ table_F,
                                                     const T* __restrict__ table_Q, const O* __restrict__ xyz,
                                                     O* __restrict__ sph, O* __restrict__ dsph,
                                                     O* __restrict__ ddsph
#ifdef SPHX_PAIRS_CLOCKS
                                                                ,
                                                                unsigned long long* clocks
#endif
) {
    static_assert(MODE >= 0 && MODE <= 2, "values alone, with gradients, with second derivatives too");
    constexpr int H = MODE == 2 ? 1 : 6;
    constexpr unsigned NYH = (H + 1) * (H + 1);
    constexpr unsigned COMP = MODE == 2 ? 13 : (MODE == 1 ? 4 : 1); // component rows per point
    constexpr unsigned SEQS = MODE + 1;            // recursions per (point, l): Q_l^m, the Q_{l-1} and Q_{l-2} sequences
    // ... interleaved in LDS: A_m alone, (A_m, B_m) pairs, (A_m, B_m, C_m, -) fours
    constexpr unsigned IT = MODE == 2 ? 4 : (MODE == 1 ? 2 : 1);
    // work items of a batch: the records; the closed forms in eight slices, or their values in one
    constexpr unsigned ITEMS = MODE == 2 ? 1 : (MODE == 1 ? 9 : 2);
    using P2 = typename Pair2<T>::type;
    using V4 = T __attribute__((ext_vector_type(4)));

    O* row_lds = reinterpret_cast<O*>(lds_raw);
    T* lds = reinterpret_cast<T*>(lds_raw + g.tables_at);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned nthreads = blockDim.x;
    const int L = g.l_max;
    const unsigned S = g.tile;
    const unsigned ny = g.ny;
    const unsigned P = g.prep_waves, NSEQ = g.sequence_waves;
    const unsigned entry_first = P + NSEQ;
    const unsigned levels = static_cast<unsigned>(L - H);

    // the constants of the Q recursions, row l at l * q_stride (a row starts at a 16-byte boundary),
    // and the prefactors of m = 0
    T* Qt = lds + g.off_Q;
    T* F0 = lds + g.off_F0;
    const unsigned QS = g.q_stride;
    for (unsigned i = tid; i < (static_cast<unsigned>(L) + 1u) * QS; i += nthreads) {
        const unsigned l = i / QS, m = i - l * QS;
        Qt[i] = m <= l ? table_Q[l * (l + 1) / 2 + m] : static_cast<T>(0.0);
    }
    for (unsigned l = tid; l <= static_cast<unsigned>(L); l += nthreads) F0[l] = table_F[l * (l + 1) / 2];

    // ---- the walk over tiles: XCD-contiguous, chunks of consecutive tiles ----
    const unsigned xcd = blockIdx.x & 7u;
    const unsigned rank_in_xcd = blockIdx.x >> 3;
    const unsigned groups_per_xcd = gridDim.x >> 3;
    const unsigned xcd_first = xcd * g.tiles_per_xcd;
    unsigned xcd_last = xcd_first + g.tiles_per_xcd;
    if (xcd_last > g.n_tiles) xcd_last = g.n_tiles;
    const unsigned chunk_mask = (1u << g.chunk_shift) - 1u;
    if (xcd_first + (rank_in_xcd << g.chunk_shift) >= xcd_last) return; // no tile for this workgroup

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

    // records and parked closed forms: two buffers of one batch each
    const unsigned tpb = g.batch_tiles;
    auto batch_slot = [&](unsigned n) -> unsigned { // tile n's place in the two batch buffers
        const unsigned b = tpb == 1u ? n : __umulhi(n, g.magic_batch); // (2^32 / 1 is no 32-bit number)
        return (b & 1u) * tpb + (n - b * tpb);
    };
    auto record = [&](unsigned n, unsigned s) -> T* {
        return lds + g.off_pts + (batch_slot(n) * S + s) * g.point_stride;
    };
    auto parked = [&](unsigned n, unsigned s) -> T* {
        return lds + g.off_park + (batch_slot(n) * S + s) * g.park_stride;
    };
    auto iterates = [&](unsigned s) -> T* { return lds + g.off_iter + s * g.iter_stride; };

    constexpr unsigned LINE = 128u / static_cast<unsigned>(sizeof(O));
    auto phase_of = [](const O* array, unsigned long long element) -> unsigned {
        return static_cast<unsigned>((reinterpret_cast<uintptr_t>(array) / sizeof(O) + element) % LINE);
    };
    // Where the rows of tile n start within their staging regions: element 0 of a region stands for
    // the start of the 128-byte line in which the tile's run begins in HBM.
    struct Phases {
        unsigned sph, dsph, ddsph;
    };
    auto phases_of = [&](unsigned n) -> Phases {
        const unsigned long long first_point = static_cast<unsigned long long>(tile_of(n)) * S;
        Phases ph;
        ph.sph = phase_of(sph, first_point * ny);
        ph.dsph = MODE >= 1 ? phase_of(dsph, first_point * 3 * ny) : 0u;
        ph.ddsph = MODE == 2 ? phase_of(ddsph, first_point * 9 * ny) : 0u;
        return ph;
    };
    [[maybe_unused]] auto staged_rows = [&](const Phases& ph, unsigned s) -> Rows<O> {
        Rows<O> rows;
        rows.ny = static_cast<int>(ny);
        rows.sph = row_lds + ph.sph + s * ny;
        rows.dsph = MODE >= 1 ? row_lds + g.off_dsph + ph.dsph + s * 3 * ny : nullptr;
        rows.ddsph = MODE == 2 ? row_lds + g.off_ddsph + ph.ddsph + s * 9 * ny : nullptr;
        return rows;
    };

#ifdef SPHX_PAIRS_CLOCKS
    // development only: cycles of every wave of workgroup 8 in the two halves of a round and at the barriers
    unsigned long long c_work = 0, c_wait_a = 0, c_wait_b = 0, c_flush = 0, c_mark = __builtin_readcyclecounter();
    unsigned c_tiles = 0;
#define SPHX_MARK(acc)                                                \
    do {                                                              \
        const unsigned long long now_ = __builtin_readcyclecounter(); \
        acc += now_ - c_mark;                                         \
        c_mark = now_;                                                \
    } while (0)
#else
#define SPHX_MARK(acc) \
    do {               \
    } while (0)
#endif

    // Every role has a loop of its own, with the same barriers in the same order (the branches are
    // uniform over a wave): what one role keeps in registers is then no burden on the others.
    if (wave < P) {
        // =================================== prep waves ===================================
        // lane p takes point p % S of tile p / S of a batch
        T rx = 0, ry = 0, rz = 0;
        auto fetch = [&](unsigned batch) {
            rx = ry = rz = 0;
            const unsigned n = batch * tpb + lane / S;
            const unsigned s = lane % S;
            if (lane < tpb * S && s < valid_in(n)) {
                const O* src = xyz + (static_cast<unsigned long long>(tile_of(n)) * S + s) * 3;
                rx = static_cast<T>(src[0]);
                ry = static_cast<T>(src[1]);
                rz = static_cast<T>(src[2]);
            }
        };
        auto prep_item = [&](unsigned batch, unsigned item) {
            const unsigned n = batch * tpb + lane / S;
            const unsigned s = lane % S;
            if (!(lane < tpb * S && s < valid_in(n))) return;
            // (the coordinates pass through an empty asm: the slices below are alternatives, and without it
            // the compiler evaluates what they have in common, nearly all closed forms, ahead of the switch
            // and keeps it in registers that a lane does not have)
            T raw[3] = {rx, ry, rz};
            asm volatile("" : "+v"(raw[0]), "+v"(raw[1]), "+v"(raw[2]));
            const Point<T> p = load_point<T, NORM>(raw);
            if (item == 0) {
                T* rec = record(n, s);
                rec[0] = p.x;
                rec[1] = p.y;
                rec[2] = p.z;
                rec[3] = p.ir;
                rec[4] = p.x2 + p.y2;
                azimuth_pairs_job<T>(p, L, rec + 8, rec + g.tmz_at);
                return;
            }
            if constexpr (MODE == 0) {
                Rows<T> rows;
                rows.ny = static_cast<int>(NYH);
                rows.sph = parked(n, s);
                rows.dsph = rows.ddsph = nullptr;
                closed_form_job<T, MODE, NORM, H>(p, rows);
            }
            if constexpr (MODE == 1) {
                Rows<T> rows;
                rows.ny = static_cast<int>(NYH);
                rows.sph = parked(n, s);
                rows.dsph = rows.sph + NYH;
                rows.ddsph = nullptr;
                switch (item) {
                case 1: closed_form_job<T, MODE, NORM, H, 0, 9>(p, rows); break;
                case 2: closed_form_job<T, MODE, NORM, H, 9, 16>(p, rows); break;
                case 3: closed_form_job<T, MODE, NORM, H, 16, 25>(p, rows); break;
                case 4: closed_form_job<T, MODE, NORM, H, 25, 31>(p, rows); break;
                case 5: closed_form_job<T, MODE, NORM, H, 31, 36>(p, rows); break;
                case 6: closed_form_job<T, MODE, NORM, H, 36, 41>(p, rows); break;
                case 7: closed_form_job<T, MODE, NORM, H, 41, 45>(p, rows); break;
                default: closed_form_job<T, MODE, NORM, H, 45, 49>(p, rows); break;
                }
            }
        };
        const unsigned prep_lanes = 64u * P;
        // MODE 0, 1: the closed forms of tile n from the parking area into its rows: point after point, a lane
        // takes the same entries of every point
        [[maybe_unused]] auto unpark_stage = [&](unsigned n, unsigned valid, O* rows_v, O* rows_g) {
            for (unsigned r = tid; r < COMP * NYH; r += prep_lanes) {
                const unsigned comp = r / NYH;
                const unsigned k = r - comp * NYH;
                const T* from = parked(n, 0) + r;
                O* to = comp == 0 ? rows_v + k : rows_g + (comp - 1) * ny + k;
                const unsigned to_step = comp == 0 ? ny : 3 * ny;
                for (unsigned s = 0; s < valid; ++s) {
                    *to = static_cast<O>(*from);
                    from += g.park_stride;
                    to += to_step;
                }
            }
        };
        // MODE 2: the closed forms of l <= 1 are a handful of operations: one lane per point, straight into the rows
        [[maybe_unused]] auto low_stage = [&](unsigned n, unsigned valid, const Phases& ph) {
            if (tid < valid) {
                const T* rec = record(n, tid);
                Point<T> p;
                p.x = rec[0];
                p.y = rec[1];
                p.z = rec[2];
                p.ir = rec[3];
                p.x2 = p.x * p.x;
                p.y2 = p.y * p.y;
                p.z2 = p.z * p.z;
                closed_form_job<T, MODE, NORM, H>(p, staged_rows(ph, tid));
            }
        };
        // the entries with m = 0 of tile n, one lane per (point, l); templates_core.hpp:392-426
        auto axial_stage = [&](unsigned n, unsigned valid, const Phases& ph) {
            for (unsigned a = tid; a < valid * levels; a += prep_lanes) {
                const unsigned s = a / levels;
                const int l = L - static_cast<int>(a - s * levels);
                const T* rec = record(n, s);
                const T* it = iterates(s) + IT * (l * (l + 1) / 2);
                const P2 xy = *reinterpret_cast<const P2*>(rec);
                const P2 zi = *reinterpret_cast<const P2*>(rec + 2);
                Point<T> p;
                p.x = xy[0];
                p.y = xy[1];
                p.z = zi[0];
                p.ir = zi[1];
                p.x2 = p.y2 = p.z2 = 0;
                const T pk = F0[l];
                if constexpr (MODE == 0) {
                    // templates_core.hpp:393-395
                    row_lds[ph.sph + s * ny + static_cast<unsigned>(l * (l + 1))] = static_cast<O>(it[0] * pk);
                } else if constexpr (MODE == 1) {
                    const P2 it0 = *reinterpret_cast<const P2*>(it);      // Q_l^0 and the Q_{l-1} sequence at 0
                    const P2 it1 = *reinterpret_cast<const P2*>(it + IT); // ... at 1
                    Entry<T> e;
                    e.hxx = e.hxy = e.hxz = e.hyy = e.hyz = e.hzz = static_cast<T>(0.0);
                    e.v = it0[0] * pk;
                    e.gx = pk * p.x * it1[1];
                    e.gy = pk * p.y * it1[1];
                    e.gz = pk * l * it0[1];
                    e = finish<T, MODE, NORM>(p, e);
                    const unsigned k = static_cast<unsigned>(l * (l + 1));
                    O* out_v = row_lds + ph.sph + s * ny + k;
                    O* out_g = row_lds + g.off_dsph + ph.dsph + s * 3 * ny + k;
                    out_v[0] = static_cast<O>(e.v);
                    out_g[0] = static_cast<O>(e.gx);
                    out_g[ny] = static_cast<O>(e.gy);
                    out_g[2 * ny] = static_cast<O>(e.gz);
                    asm volatile("" ::"v"(it1[0])); // see pair_entries
                } else {
                    const V4 q0 = *reinterpret_cast<const V4*>(it);
                    const V4 q1 = *reinterpret_cast<const V4*>(it + IT);
                    const V4 q2 = *reinterpret_cast<const V4*>(it + 2 * IT);
                    EntryWindow<T> in;
                    in.pk_ = pk;
                    in.c_[0] = in.c_[1] = in.c_[2] = in.s_[0] = in.s_[1] = in.s_[2] = 0; // m = 0 uses neither
                    in.A_[0] = q0[0];
                    in.A_[1] = q1[0];
                    in.B_[0] = q0[1];
                    in.B_[1] = q1[1];
                    in.C_[0] = q0[2];
                    in.C_[1] = q1[2];
                    in.C_[2] = q2[2];
                    entry_job_from<T, MODE, NORM, false>(l, 0, l * (l + 1) / 2, 0, p, in, staged_rows(ph, s));
                }
            }
        };

        // the first batch (or two) in full, then one batch (or two) ahead: one work item per tile round
        const unsigned ahead = g.lookahead;
        for (unsigned b = 0; b < ahead; ++b) {
            fetch(b);
            for (unsigned item = wave; item < ITEMS; item += P) prep_item(b, item);
        }
        fetch(ahead);
        __syncthreads();
        unsigned step = 0, batch = 0;
        SPHX_MARK(c_wait_b);
        for (unsigned n = 0;; ++n) {
            const unsigned valid = valid_in(n);
            if (valid == 0) break;
            __syncthreads(); // iterates of tile n in place, rows of tile n - 1 flushed
            SPHX_MARK(c_wait_a);
            {
                const Phases ph = phases_of(n);
                if constexpr (MODE <= 1) {
                    unpark_stage(n, valid, row_lds + ph.sph, row_lds + g.off_dsph + ph.dsph);
                } else {
                    low_stage(n, valid, ph);
                }
                axial_stage(n, valid, ph);
            }
            SPHX_MARK(c_work);
            __syncthreads(); // rows of tile n complete
            SPHX_MARK(c_wait_b);
            if (g.priorities & 2u) __builtin_amdgcn_s_setprio(2);
            const unsigned item = step * P + wave;
            if (item < ITEMS) prep_item(batch + ahead, item);
            if (++step == tpb) {
                step = 0;
                ++batch;
                fetch(batch + ahead);
            }
            __builtin_amdgcn_s_setprio(0);
            SPHX_MARK(c_flush);
        }
    } else if (wave < entry_first) {
        // ================================= sequence waves =================================
        // One bare recursion per lane: start values, then blocks of four steps whose constants,
        // 2(m+1)z and the row of Q constants, come as 16-byte reads one block ahead of the arithmetic.
        // Same operations in the same order as sequence_job (sphx_device.hpp).
        const unsigned seq_tid = tid - 64u * P;
        const unsigned seq_lanes = 64u * NSEQ;
        const unsigned seq_jobs = SEQS * S * levels;
        // job j: l from l_max down, the points of a tile and their sequences side by side
        auto run_chain = [&](unsigned n, unsigned j, unsigned valid) {
            const unsigned per_l = SEQS * S;
            const unsigned step = j / per_l;
            const unsigned rest = j - step * per_l;
            const unsigned s = rest / SEQS, which = rest - s * SEQS;
            if (s >= valid) return;
            const int l = L - static_cast<int>(step);
            const T* rec = record(n, s);
            const T z = rec[2];
            const T rxy = rec[4];
            // row l for Q_l^m, row l - 1 for the Q_{l-1} sequence, row l - 2 for the Q_{l-2} sequence
            const T* row = Qt + (static_cast<unsigned>(l) - which) * QS;
            T* out = iterates(s) + IT * (l * (l + 1) / 2) + which;
            // start values (templates_core.hpp:122-123, 135, 150, 155, 167, 196 and :228-231) and the first step
            T v1, v2;
            int top = l - 2;
            if (which == 0) {
                v2 = row[l];
                v1 = -z * v2;
                out[l * IT] = v2;
                out[(l - 1) * IT] = v1;
            } else if (which == 1) {
                v2 = 0;
                v1 = row[l - 1];
                out[l * IT] = v2;
                out[(l - 1) * IT] = v1;
            } else {
                v2 = 0;
                v1 = row[l - 2];
                out[l * IT] = v2;
                out[(l - 1) * IT] = v2;
                out[(l - 2) * IT] = v1;
                top = l - 3;
            }
            if (top < 0) return;
            int base = top & ~3; // the block of four that holds the first step
            const T* pt = rec + g.tmz_at + base;
            const T* pk = row + base;
            T* po = out + IT * base;
            V4 tz = *reinterpret_cast<const V4*>(pt);
            V4 km = *reinterpret_cast<const V4*>(pk);
            // (below m = 0 the reads fetch, unused, what precedes the tables: the pairs of the record,
            // the end of the row before)
            V4 tz_next = *reinterpret_cast<const V4*>(pt - 4);
            V4 km_next = *reinterpret_cast<const V4*>(pk - 4);
#define SPHX_STEP(tzv, kmv, j)                                  \
    do {                                                        \
        const T v0 = (kmv)[j] * ((tzv)[j] * v1 + rxy * v2);     \
        po[(j) * IT] = v0;                                      \
        v2 = v1;                                                \
        v1 = v0;                                                \
    } while (0)
            switch (top & 3) {
            case 3: SPHX_STEP(tz, km, 3); [[fallthrough]];
            case 2: SPHX_STEP(tz, km, 2); [[fallthrough]];
            case 1: SPHX_STEP(tz, km, 1); [[fallthrough]];
            default: SPHX_STEP(tz, km, 0); break;
            }
            // whole blocks, two per turn: what was read ahead needs no moving
            int blocks = base >> 2;
            while (blocks >= 2) {
                pt -= 8;
                pk -= 8;
                tz = *reinterpret_cast<const V4*>(pt);
                km = *reinterpret_cast<const V4*>(pk);
                po -= 4 * IT;
                SPHX_STEP(tz_next, km_next, 3);
                SPHX_STEP(tz_next, km_next, 2);
                SPHX_STEP(tz_next, km_next, 1);
                SPHX_STEP(tz_next, km_next, 0);
                tz_next = *reinterpret_cast<const V4*>(pt - 4);
                km_next = *reinterpret_cast<const V4*>(pk - 4);
                po -= 4 * IT;
                SPHX_STEP(tz, km, 3);
                SPHX_STEP(tz, km, 2);
                SPHX_STEP(tz, km, 1);
                SPHX_STEP(tz, km, 0);
                blocks -= 2;
            }
            if (blocks == 1) {
                po -= 4 * IT;
                SPHX_STEP(tz_next, km_next, 3);
                SPHX_STEP(tz_next, km_next, 2);
                SPHX_STEP(tz_next, km_next, 1);
                SPHX_STEP(tz_next, km_next, 0);
            }
#undef SPHX_STEP
        };
        auto sequence_stage = [&](unsigned n) {
            const unsigned valid = valid_in(n);
            if (valid == 0) return;
            for (unsigned j = seq_tid; j < seq_jobs; j += seq_lanes) run_chain(n, j, valid);
        };

        __syncthreads(); // records of batch 0
        sequence_stage(0);
        SPHX_MARK(c_wait_b);
        for (unsigned n = 0; valid_in(n) != 0; ++n) {
            __syncthreads(); // iterates of tile n in place
            SPHX_MARK(c_wait_a);
            __syncthreads(); // rows of tile n complete, its iterates no longer needed
            SPHX_MARK(c_wait_b);
            if (g.priorities & 2u) __builtin_amdgcn_s_setprio(2);
            sequence_stage(n + 1);
            __builtin_amdgcn_s_setprio(0);
            SPHX_MARK(c_flush);
        }
    } else {
        // ================================== entry waves ===================================
        // MODE 1: the waves of a slot share a point, which is then the same for a whole wave (its addresses are
        // scalars). MODE 2: the table deals the lanes to the points lane by lane.
        const unsigned ew = wave - entry_first;
        const unsigned wave_slot = MODE <= 1 ? ew / g.slot_waves : 0u;
        const unsigned job = g.lane_job[(ew - wave_slot * g.slot_waves) * 64u + lane];
        const bool has_job = job != kPairsNoJob;
        const unsigned slot = MODE <= 1 ? wave_slot : (has_job ? job >> 14 : 0u);
        const unsigned slots = MODE <= 1 ? g.entry_waves / g.slot_waves : g.lane_slots;
        const int e_l = has_job ? static_cast<int>((job >> 7) & 127u) : H + 1;
        const int e_m = has_job ? static_cast<int>(job & 127u) : 1;
        const bool no_pdq = e_m >= e_l - 1; // |m| = l and l - 1: no Q_{l-1}^{m+1} term in d/dx, d/dy
        const bool no_dz = e_m == e_l;      // |m| = l: no d/dz
        const int e_tri = e_l * (e_l + 1) / 2;
        const T pkm = table_F[e_tri + e_m];
        const T fm = static_cast<T>(e_m);
        const T pk_lm = pkm * static_cast<T>(e_l + e_m);
        const unsigned k_plus = static_cast<unsigned>(e_l * (e_l + 1) + e_m);
        const unsigned k_minus = static_cast<unsigned>(e_l * (e_l + 1) - e_m);
        const unsigned o_cs = 8u + 2u * static_cast<unsigned>(e_m - 1);
        const unsigned o_it = IT * static_cast<unsigned>(e_tri + e_m);

        // what a lane reads per point: (x, y), (z, 1/r), (A_m, B_m), (A_{m+1}, B_{m+1}) with A = Q_l and B the
        // Q_{l-1} sequence, (c_{m-1}, s_{m-1}), (c_m, s_m); three 16-byte reads and no arithmetic
        struct Fetched {
            P2 xy, zi, it0, it1, q1, q0;
        };
        auto fetch_point = [&](unsigned n, unsigned s) -> Fetched {
            const T* rec = record(n, s);
            const T* it = iterates(s) + o_it;
            Fetched f;
            f.xy = *reinterpret_cast<const P2*>(rec);
            f.zi = *reinterpret_cast<const P2*>(rec + 2);
            f.it0 = *reinterpret_cast<const P2*>(it);
            f.it1 = *reinterpret_cast<const P2*>(it + IT);
            f.q1 = *reinterpret_cast<const P2*>(rec + o_cs);
            f.q0 = *reinterpret_cast<const P2*>(rec + o_cs + 2);
            return f;
        };
        // where a lane's entries of the current point go: (l, +m) and (l, -m) in the value row and in
        // the first gradient row (the other two are ny and 2 ny further on)
        struct Places {
            O *vp, *vm, *gp, *gm;
        };
        // One point's entries (l, +-m). Where the reference leaves a term out (no_pdq, no_dz) the lane
        // selects the shorter expression; every number is computed by the reference's own operations.
        auto pair_entries = [&](const Fetched& f, const Places& at) {
            Point<T> p;
            p.x = f.xy[0];
            p.y = f.xy[1];
            p.z = f.zi[0];
            p.ir = f.zi[1];
            p.x2 = p.y2 = p.z2 = 0;
            const T zero = static_cast<T>(0.0);
            const T cm1 = f.q1[0], sm1 = f.q1[1], cm = f.q0[0], sm = f.q0[1];
            auto put_entry = [&](O* v, O* gr, const Entry<T>& raw) {
                const Entry<T> e = finish<T, MODE, NORM>(p, raw);
                v[0] = static_cast<O>(e.v);
                gr[0] = static_cast<O>(e.gx);
                gr[ny] = static_cast<O>(e.gy);
                gr[2 * ny] = static_cast<O>(e.gz);
            };
            Entry<T> e;
            e.hxx = e.hxy = e.hxz = e.hyy = e.hyz = e.hzz = zero;
            const T pq0 = f.it0[0] * pkm; // Q_l^m F_l^m
            const T pqm = pq0 * fm;
            const T pdq = pkm * f.it1[1];
            const T pdqx = pdq * p.x;
            const T pdqy = pdq * p.y;
            const T pdz = pk_lm * f.it0[1];
            // templates_core.hpp:201-294; :122-152 for |m| = l, :154-198 for |m| = l - 1
            T t = pqm * cm1;
            e.v = pq0 * cm;
            e.gx = no_pdq ? t : (pdqx * cm + t);
            t = pqm * -sm1;
            e.gy = no_pdq ? t : (pdqy * cm + t);
            e.gz = no_dz ? zero : pdz * cm;
            put_entry(at.vp, at.gp, e);
            t = pqm * sm1;
            e.v = pq0 * sm;
            e.gx = no_pdq ? t : (pdqx * sm + t);
            t = pqm * cm1;
            e.gy = no_pdq ? t : (pdqy * sm + t);
            e.gz = no_dz ? zero : pdz * sm;
            put_entry(at.vm, at.gm, e);
            // (A_{m+1} comes along in a 16-byte read and is not used: without a use down here its register
            // would serve as scratch above, and the lane would wait for the read that is still in flight)
            asm volatile("" ::"v"(f.it1[0]));
        };
        auto entry_stage = [&](unsigned n) {
            const unsigned valid = valid_in(n);
            if (slot >= valid || !has_job) return;
            const Phases ph = phases_of(n);
            if constexpr (MODE == 0) {
                // values alone, templates_core.hpp:214-218 (:127-128 and :160-162 for |m| = l and l - 1): the
                // iterate, its prefactor, c_m and s_m. Four points per turn: their reads are in flight together.
                O* vp = row_lds + ph.sph + slot * ny + k_plus;
                O* vm = row_lds + ph.sph + slot * ny + k_minus;
                const unsigned step = slots * ny;
                for (unsigned s = slot; s < valid; s += 4u * slots) {
                    T a[4];
                    P2 cs[4];
#pragma unroll
                    for (unsigned u = 0; u < 4u; ++u) {
                        // (past the tile's last point: the last point once more, nothing stored)
                        const unsigned su = s + u * slots < valid ? s + u * slots : s;
                        a[u] = iterates(su)[o_it];
                        cs[u] = *reinterpret_cast<const P2*>(record(n, su) + o_cs + 2);
                    }
#pragma unroll
                    for (unsigned u = 0; u < 4u; ++u) {
                        if (s + u * slots < valid) {
                            const T pq = a[u] * pkm;
                            vp[u * step] = static_cast<O>(pq * cs[u][0]);
                            vm[u * step] = static_cast<O>(pq * cs[u][1]);
                        }
                    }
                    vp += 4u * step;
                    vm += 4u * step;
                }
                return;
            }
            if constexpr (MODE == 2) {
                // entry_job's own arithmetic on what the lane reads of the point: the iterates at m, m + 1, m + 2
                // and (c, s) at m - 2, m - 1, m
                for (unsigned s = slot; s < valid; s += slots) {
                    const T* rec = record(n, s);
                    const T* it = iterates(s) + o_it;
                    const T* cs = rec + 8u + 2u * static_cast<unsigned>(e_m);
                    const P2 xy = *reinterpret_cast<const P2*>(rec);
                    const P2 zi = *reinterpret_cast<const P2*>(rec + 2);
                    const V4 q0 = *reinterpret_cast<const V4*>(it);
                    const V4 q1 = *reinterpret_cast<const V4*>(it + IT);
                    const V4 q2 = *reinterpret_cast<const V4*>(it + 2 * IT);
                    const P2 p0 = *reinterpret_cast<const P2*>(cs);
                    const P2 p1 = *reinterpret_cast<const P2*>(cs - 2);
                    const P2 p2 = *reinterpret_cast<const P2*>(cs - 4); // (for m = 1: two spare numbers, not used)
                    Point<T> p;
                    p.x = xy[0];
                    p.y = xy[1];
                    p.z = zi[0];
                    p.ir = zi[1];
                    p.x2 = p.y2 = p.z2 = 0;
                    EntryWindow<T> in;
                    in.pk_ = pkm;
                    in.c_[0] = p2[0];
                    in.c_[1] = p1[0];
                    in.c_[2] = p0[0];
                    in.s_[0] = p2[1];
                    in.s_[1] = p1[1];
                    in.s_[2] = p0[1];
                    in.A_[0] = q0[0];
                    in.A_[1] = q1[0];
                    in.B_[0] = q0[1];
                    in.B_[1] = q1[1];
                    in.C_[0] = q0[2];
                    in.C_[1] = q1[2];
                    in.C_[2] = q2[2];
                    entry_job_from<T, MODE, NORM, false>(e_l, e_m, e_tri, 0, p, in, staged_rows(ph, s));
                }
                return;
            }
            O* rows_v = row_lds + ph.sph;
            O* rows_g = row_lds + g.off_dsph + ph.dsph;
            unsigned s = slot; // the same for the whole wave: the point's addresses are scalars
            Places at;
            at.vp = rows_v + s * ny + k_plus;
            at.vm = rows_v + s * ny + k_minus;
            at.gp = rows_g + s * 3 * ny + k_plus;
            at.gm = rows_g + s * 3 * ny + k_minus;
            auto advance = [&]() {
                at.vp += slots * ny;
                at.vm += slots * ny;
                at.gp += slots * 3 * ny;
                at.gm += slots * 3 * ny;
                s += slots;
            };
            // The reads of the next point are issued before the arithmetic of this one; two copies of the
            // body take turns, so that what was read ahead needs no moving.
            Fetched even = fetch_point(n, s), odd = even;
            for (;;) {
                bool more = s + slots < valid;
                if (more) odd = fetch_point(n, s + slots);
                pair_entries(even, at);
                if (!more) break;
                advance();
                more = s + slots < valid;
                if (more) even = fetch_point(n, s + slots);
                pair_entries(odd, at);
                if (!more) break;
                advance();
            }
        };

        // ---- flush: whole 128-byte lines only, the unfinished last line carried into the next tile ----
        const unsigned flush_tid = tid - 64u * entry_first;
        const unsigned flush_lanes = nthreads - 64u * entry_first;
        auto flush_stage = [&](unsigned n) {
            const unsigned valid = valid_in(n);
            const unsigned long long first = static_cast<unsigned long long>(tile_of(n)) * S;
            const bool starts = (n & chunk_mask) == 0;
            const bool ends = (n & chunk_mask) == chunk_mask || valid_in(n + 1) == 0;
            const unsigned ft = flush_tid, count = flush_lanes;
            // The tile's run of `len` elements of one output array starts at element `at` of that array.
            // Only whole 128-byte lines go out with vector stores. The line in which the run ends is
            // completed by the next tile: when that tile is this workgroup's next one (same chunk), the
            // unfinished part is carried over to the start of the region, where the next tile's run
            // continues it; at the ends of a chunk the partial lines are stored element by element.
            auto flush_run = [&](unsigned region_offset, O* array, unsigned long long at, unsigned len) {
                using V = typename Pack<O>::type;
                constexpr unsigned W = Pack<O>::width;
                O* region = row_lds + region_offset;
                const unsigned phase = phase_of(array, at);
                O* line0 = array + (at - phase); // HBM address of region element 0
                const unsigned lo = starts ? phase : 0u;
                const unsigned hi = phase + len;
                const unsigned full_lo = (lo + LINE - 1u) / LINE * LINE;
                const unsigned full_hi = hi / LINE * LINE;
                unsigned tail_from;
                if (full_hi > full_lo) {
                    const unsigned nvec = (full_hi - full_lo) / W;
                    const V* in = reinterpret_cast<const V*>(region + full_lo);
                    V* out = reinterpret_cast<V*>(line0 + full_lo);
                    for (unsigned v = ft; v < nvec; v += count) {
                        emit<O, true>(in[v], out + v);
                    }
                    tail_from = full_hi;
                } else {
                    tail_from = full_lo < hi ? full_lo : hi;
                }
                const unsigned head_end = full_lo < hi ? full_lo : hi;
                if (lo + ft < head_end) line0[lo + ft] = region[lo + ft];
                const unsigned tail = hi - tail_from;
                if (ft < tail) {
                    const O value = region[tail_from + ft];
                    if (ends) {
                        line0[tail_from + ft] = value;
                    } else if (tail_from != 0) {
                        region[ft] = value;
                    }
                }
            };
            flush_run(0, sph, first * ny, valid * ny);
            if constexpr (MODE >= 1) flush_run(g.off_dsph, dsph, first * 3 * ny, valid * 3 * ny);
            if constexpr (MODE == 2) flush_run(g.off_ddsph, ddsph, first * 9 * ny, valid * 9 * ny);
        };

        __syncthreads();
        SPHX_MARK(c_wait_b);
        for (unsigned n = 0; valid_in(n) != 0; ++n) {
            __syncthreads();
            SPHX_MARK(c_wait_a);
            entry_stage(n);
            SPHX_MARK(c_work);
            __syncthreads();
            SPHX_MARK(c_wait_b);
            if (g.priorities & 1u) __builtin_amdgcn_s_setprio(2);
            flush_stage(n);
            __builtin_amdgcn_s_setprio(0);
            SPHX_MARK(c_flush);
#ifdef SPHX_PAIRS_CLOCKS
            ++c_tiles;
#endif
        }
    }
#ifdef SPHX_PAIRS_CLOCKS
    if (blockIdx.x == 8 && lane == 0) {
        unsigned long long* c = clocks + wave * 5;
        c[0] = c_wait_a;
        c[1] = c_work;
        c[2] = c_wait_b;
        c[3] = c_flush;
        c[4] = c_tiles;
    }
#endif
#undef SPHX_MARK
}

} // namespace sphx

#endif

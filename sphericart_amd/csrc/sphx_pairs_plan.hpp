// Host side of pairs_kernel: tile, batch, wave roles, LDS layout and the table that gives every
// entry lane its (l, m) pair, from the shape of a call. Plain C++, no HIP: the planner can be
// compiled and tested without a device.
#ifndef SPHX_PAIRS_PLAN_HPP
#define SPHX_PAIRS_PLAN_HPP

#include <cstddef>
#include <cstring>

#include "sphx_pairs_tiling.hpp"

namespace sphx {

// What the caller may fix (0 = let the planner choose).
struct PairsChoice {
    unsigned tile = 0, batch_tiles = 0, prep_waves = 0, sequence_waves = 0, chunk_shift_plus_one = 0;
};

struct PairsLaunch {
    PairsTiling g;
    unsigned lds_bytes = 0, threads = 0, workgroups = 0;
};

// The lane table of values and gradients: the pairs (l, m >= 1) of one point in a row, l and m descending,
// over as few waves as hold them; the waves of one such group share a point. (A table that kept the lanes of a
// half-wave on different LDS banks, at the price of one more wave, measured 1-3 % slower: the stage is
// bound by instruction issue, not by LDS.) Returns the number of waves, 0 if `waves` do not hold the pairs.
inline unsigned short pairs_job(unsigned slot, int l, int m) {
    return static_cast<unsigned short>((slot << 14) | (static_cast<unsigned>(l) << 7) | static_cast<unsigned>(m));
}
inline unsigned pairs_lane_table(int l_max, int hard, unsigned waves, unsigned short* table) {
    for (unsigned i = 0; i < kPairsThreads; ++i) table[i] = static_cast<unsigned short>(kPairsNoJob);
    if (waves > kPairsThreads / 64u) waves = kPairsThreads / 64u;
    unsigned at = 0;
    for (int l = l_max; l > hard; --l) {
        if (at + static_cast<unsigned>(l) > waves * 64u) return 0;
        for (int m = l; m >= 1; --m) table[at++] = pairs_job(0, l, m);
    }
    return (at + 63u) / 64u;
}

// The lane table with second derivatives. The entries with |m| = l, |m| = l - 1 and 1 <= |m| <= l - 2 are three
// different pieces of code, and a wave runs every piece that one of its lanes needs: the table is ordered by
// kind (the bulk of all points side by side, then |m| = l, then |m| = l - 1), the bulk filled up to a whole
// wave where the lanes allow. As many points side by side (four at most) as `waves` waves hold. Returns that
// number, 0 if not even one point fits.
inline unsigned pairs_lane_table_by_kind(int l_max, int hard, unsigned waves, unsigned most_slots,
                                         unsigned short* table) {
    for (unsigned i = 0; i < kPairsThreads; ++i) table[i] = static_cast<unsigned short>(kPairsNoJob);
    if (waves > kPairsThreads / 64u) waves = kPairsThreads / 64u;
    const unsigned lanes = waves * 64u;
    unsigned bulk = 0, levels = 0;
    for (int l = hard + 1; l <= l_max; ++l) {
        bulk += l >= 2 ? static_cast<unsigned>(l - 2) : 0u;
        ++levels;
    }
    if (most_slots > 4u) most_slots = 4u;
    for (unsigned slots = most_slots; slots >= 1u; --slots) {
        if (slots * (bulk + 2u * levels) > lanes) continue;
        unsigned at = 0;
        for (unsigned s = 0; s < slots; ++s) {
            for (int l = l_max; l > hard; --l) {
                for (int m = l - 2; m >= 1; --m) table[at++] = pairs_job(s, l, m);
            }
        }
        const unsigned padded = (at + 63u) & ~63u;
        if (padded + slots * 2u * levels <= lanes) at = padded; // the other kinds start a wave of their own
        for (unsigned s = 0; s < slots; ++s) {
            for (int l = l_max; l > hard; --l) table[at++] = pairs_job(s, l, l);
        }
        for (unsigned s = 0; s < slots; ++s) {
            for (int l = l_max; l > hard; --l) {
                if (l >= 2) table[at++] = pairs_job(s, l, l - 1);
            }
        }
        return slots;
    }
    return 0;
}

// false: this shape is not for pairs_kernel (the pairs of a point do not fit the waves, or the rows of
// a tile and the tables do not fit LDS).
// `mode`: 1 values and gradients, 2 second derivatives too (in float64 in workgroups of 512 threads: the
// entries need more than the 128 registers that sixteen waves leave a lane).
inline bool plan_pairs(size_t n_samples, int l_max, int mode, size_t elem, size_t out_elem, int lds_limit, int cus,
                       const PairsChoice& want, PairsLaunch* out) {
    if (mode < 0 || mode > 2) return false;
    const int H = mode == 2 ? 1 : 6;
    const unsigned NYH = static_cast<unsigned>((H + 1) * (H + 1));
    const unsigned COMP = mode == 2 ? 13u : (mode == 1 ? 4u : 1u), SEQS = static_cast<unsigned>(mode) + 1u;
    const unsigned IT = mode == 2 ? 4u : (mode == 1 ? 2u : 1u);
    const unsigned ITEMS = mode == 2 ? 1u : (mode == 1 ? 9u : 2u);
    const unsigned WAVES = (mode == 2 && elem == 8 ? 512u : kPairsThreads) / 64u;
    if (l_max <= H || l_max > 64 || n_samples == 0) return false;
    PairsTiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    const unsigned esize = static_cast<unsigned>(elem), osize = static_cast<unsigned>(out_elem);
    const unsigned L = static_cast<unsigned>(l_max);
    const unsigned ny = (L + 1) * (L + 1);
    const unsigned tri_all = (L + 1) * (L + 2) / 2;
    const unsigned levels = L - H;

    const unsigned line = 128u / osize;
    auto align4 = [](unsigned v) { return (v + 3u) & ~3u; };
    // a point's record: x, y, z, 1/r, x^2 + y^2, three spare; the (c_m, s_m) pairs; 2(m+1)z from a multiple of
    // four numbers on, and the records a multiple of four apart (16-byte reads of four steps' constants)
    const unsigned tmz_at = align4(8u + 2u * (L + 1));
    const unsigned point_stride = align4(tmz_at + (L + 1));
    const unsigned q_stride = align4(L + 1);
    const unsigned q_elems = (L + 1) * q_stride;
    const unsigned f0_elems = align4(L + 1);
    // (with second derivatives nothing is parked)
    const unsigned park_stride = mode == 2 ? 0u : (COMP * NYH) | 1u; // odd: the lanes of a prep wave, one point each, spread over the banks
    const unsigned iter_stride = align4(IT * tri_all + 2u * IT); // up to two groups past the end are read, never used
    auto bytes_for = [&](unsigned S, unsigned tpb) {
        const unsigned rows = align4(S * ny + line) + (mode >= 1 ? align4(S * 3 * ny + line) : 0u) +
                              (mode == 2 ? align4(S * 9 * ny + line) : 0u);
        const unsigned tables = q_elems + f0_elems + 2 * tpb * S * (point_stride + park_stride) + 4u + S * iter_stride;
        return rows * osize + tables * esize;
    };

    // as many points per tile as LDS holds next to a batch of three tiles, twelve at most (1.2 GB of
    // output, l_max = 20 - 36: within 3 % of the best tile size on every shape)
    unsigned S = want.tile ? want.tile : (mode == 0 ? 64u : 12u);
    // (values alone: two work items a batch, so a batch is a single tile, of up to a wave's lanes of points)
    const unsigned least_batch = mode == 0 ? 1u : 3u;
    if (S > (mode == 0 ? 64u : 16u)) S = mode == 0 ? 64u : 16u;
    while (S > 1 && bytes_for(S, least_batch) > static_cast<unsigned>(lds_limit)) --S;
    // Values alone: an entry is three multiplications, and what a tile costs is the entry waves going through
    // its points one after the other, then the longer of the flush and the recursions of the next tile, which
    // run side by side. More sequence waves shorten the recursions and leave fewer entry waves, which then take
    // fewer points side by side. The largest tile that fits (smaller ones measured slower throughout) with the
    // number of sequence waves of the least estimated cycles: 140 per point an entry wave goes through, 80 per
    // step of a round of recursions, stores that drain at 11 bytes per cycle after the first 19 KB, and a
    // quarter of the shorter of the two that run side by side for what they take from each other (measured on
    // this kernel, MI355X; the choice is within 2 % of the best number of waves on every shape tried).
    unsigned model_sequence_waves = 0;
    if (mode == 0 && want.tile == 0) {
        const unsigned pairs = (L * (L + 1u)) / 2u - static_cast<unsigned>(H * (H + 1)) / 2u;
        const unsigned pair_waves = (pairs + 63u) / 64u;
        const unsigned most = S;
        unsigned long long best = ~0ull;
        for (unsigned s_try = most; s_try == most; --s_try) {
            for (unsigned q = 2u; q <= WAVES / 2u; ++q) {
                if (2u + q + pair_waves > WAVES) break;
                unsigned slots = (WAVES - 2u - q) / pair_waves;
                if (slots > s_try) slots = s_try;
                const unsigned long long entry = (s_try + slots - 1u) / slots * 140ull;
                const unsigned long long rounds = (s_try * levels + 64u * q - 1u) / (64u * q);
                const unsigned long long recursions = rounds * (L + 1u) * 80ull;
                const unsigned long long bytes = static_cast<unsigned long long>(s_try) * ny * osize;
                const unsigned long long flush = bytes > 19000ull ? (bytes - 19000ull) / 11ull : 0ull;
                const unsigned long long longer = recursions > flush ? recursions : flush;
                const unsigned long long shorter = recursions > flush ? flush : recursions;
                const unsigned long long per_point = (entry + longer + shorter / 4ull + 600ull) * 1000ull / s_try;
                if (per_point <= best) {
                    best = per_point;
                    S = s_try;
                    model_sequence_waves = q;
                }
            }
        }
    }
    // batches: as many tiles as a wave has lanes for and LDS holds; at least three, so that the nine work
    // items of a batch fit its tile rounds with the prep waves there are (with second derivatives a batch is
    // only the records, and eight points are enough to share their chain of dependent operations)
    unsigned tpb = want.batch_tiles ? want.batch_tiles : (mode == 2 ? (8u + S - 1u) / S : 64u / S);
    if (tpb < least_batch) tpb = least_batch;
    if (tpb * S > 64u) tpb = 64u / S;
    while (tpb > least_batch && bytes_for(S, tpb) > static_cast<unsigned>(lds_limit)) --tpb;
    if (tpb < least_batch || bytes_for(S, tpb) > static_cast<unsigned>(lds_limit)) return false;
    if (mode == 0 && want.batch_tiles == 0) tpb = 1u;
    unsigned P = want.prep_waves ? want.prep_waves : (ITEMS + tpb - 1u) / tpb;
    if (P * tpb < ITEMS) P = (ITEMS + tpb - 1u) / tpb;
    // one recursion per lane and tile where four waves suffice for that
    unsigned NSEQ = want.sequence_waves      ? want.sequence_waves
                    : model_sequence_waves != 0 ? model_sequence_waves
                                                : (S * SEQS * levels + 63u) / 64u;
    if (NSEQ < 1) NSEQ = 1;
    if (NSEQ > (mode == 0 ? WAVES / 2u : WAVES / 4u)) NSEQ = mode == 0 ? WAVES / 2u : WAVES / 4u;
    if (P + NSEQ >= WAVES) return false;
    const unsigned room = WAVES - P - NSEQ;
    // the waves that hold a point's pairs, and as many points side by side as the entry waves allow
    unsigned slot_waves = 0, lane_slots = 0, E = 0;
    if (mode <= 1) {
        slot_waves = pairs_lane_table(l_max, H, room, g.lane_job);
        if (slot_waves == 0) return false;
        unsigned slots = room / slot_waves;
        if (slots > S) slots = S;
        E = slots * slot_waves;
    } else {
        lane_slots = pairs_lane_table_by_kind(l_max, H, room, S, g.lane_job);
        if (lane_slots == 0) return false;
        for (unsigned i = 0; i < room * 64u; ++i) {
            if (g.lane_job[i] != kPairsNoJob) E = i / 64u + 1u;
        }
        slot_waves = E;
    }

    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = S;
    g.batch_tiles = tpb;
    g.magic_batch = static_cast<unsigned>(((1ull << 32) + tpb - 1) / tpb);
    g.prep_waves = P;
    g.sequence_waves = NSEQ;
    g.entry_waves = E;
    g.slot_waves = slot_waves;
    g.lane_slots = lane_slots;
    unsigned at = align4(S * ny + line);
    g.off_dsph = at;
    if (mode >= 1) at = align4(at + S * 3 * ny + line);
    g.off_ddsph = at;
    if (mode == 2) at = align4(at + S * 9 * ny + line);
    g.tables_at = at * osize;
    at = 0;
    g.off_Q = at;
    at += q_elems;
    g.off_F0 = at;
    at += f0_elems;
    g.off_pts = at;
    g.lookahead = tpb == 1u ? 2u : 1u;
    at += 2 * tpb * S * point_stride;
    g.off_park = at;
    at += 2 * tpb * S * park_stride;
    at = align4(at);
    g.off_iter = at;
    at += S * iter_stride;
    g.point_stride = point_stride;
    g.park_stride = park_stride;
    g.iter_stride = iter_stride;
    g.tmz_at = tmz_at;
    g.q_stride = q_stride;
    out->lds_bytes = g.tables_at + at * esize;
    out->threads = 64u * (P + NSEQ + E);
    if (out->lds_bytes > static_cast<unsigned>(lds_limit)) return false;

    g.n_tiles = static_cast<unsigned>((n_samples + S - 1) / S);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    // about eight points per chunk of consecutive tiles
    g.chunk_shift = want.chunk_shift_plus_one ? want.chunk_shift_plus_one - 1u : (S >= 5 ? 0u : (S >= 3 ? 1u : (S == 2 ? 2u : 3u)));
    if (g.chunk_shift > 10u) g.chunk_shift = 10u;
    const unsigned resident = (static_cast<unsigned>(cus > 0 ? cus : 8) + 7u) & ~7u;
    auto chunks_in_xcd = [&]() { return (g.tiles_per_xcd + (1u << g.chunk_shift) - 1u) >> g.chunk_shift; };
    while (g.chunk_shift > 0 && chunks_in_xcd() * 8u < resident) --g.chunk_shift;
    const unsigned need = chunks_in_xcd() * 8u;
    out->workgroups = resident < need ? resident : need;
    if (out->workgroups < 8) out->workgroups = 8;
    return true;
}

} // namespace sphx

#endif

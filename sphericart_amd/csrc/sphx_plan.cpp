// The planner: from the shape of a call to kernels, tiles and LDS layouts. Plain host C++.

#include "sphx_plan.hpp"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/sphx_launch.h"
#include "sphx_plan_shapes.hpp"

namespace sphx {

thread_local std::string t_error;

int fail(int code, const std::string& what) {
    t_error = what;
    return code;
}

static const char* const kSwitchNames[SW_COUNT] = {
    "SPHX_AZ_SHIFT", "SPHX_CHUNK_SHIFT", "SPHX_GRADIENT_LANES",
    "SPHX_GRADIENT_LANES_PARTS", "SPHX_GRADIENT_LANES_TILE", "SPHX_GRADIENT_LANES_WAVES", "SPHX_GROUP_THREADS",
    "SPHX_HESSIAN_LANES",
    "SPHX_HESSIAN_LANES_PARTS", "SPHX_HESSIAN_LANES_TILE", "SPHX_JOB_LIST",
    "SPHX_PAIRS", "SPHX_PAIRS_BATCH", "SPHX_PAIRS_CHUNK", "SPHX_PAIRS_PREP_WAVES", "SPHX_PAIRS_SEQUENCE_WAVES", "SPHX_PAIRS_TILE",
    "SPHX_PREFIX_INSIDE", "SPHX_RECURSIONS_TOGETHER", "SPHX_ROW_PAD", "SPHX_SEQUENCE_WAVES", "SPHX_SLICE_WAVES", "SPHX_SPLIT_BELOW",
    "SPHX_SPLIT_RATIO", "SPHX_SPLIT_SIDES", "SPHX_SPREAD_KINDS", "SPHX_TILE", "SPHX_TILE_LDS_BUDGET", "SPHX_TILE_POW2",
    "SPHX_TILE_SMALL_N", "SPHX_VALUES_ALONE", "SPHX_VALUES_LDS", "SPHX_VALUES_MIN_TILE", "SPHX_VALUES_MIN_WAVES",
    "SPHX_VALUES_PACK", "SPHX_VALUES_TILE_STEP", "SPHX_VALUES_WAVES", "SPHX_VJP_GROUPS_BELOW", "SPHX_VJP_LANES", "SPHX_VJP_MIN_TILE", "SPHX_VJP_STEP_FLOOR", "SPHX_VJP_TILE_STEP", "SPHX_WAVE_PRIORITIES",
};
struct Switches {
    bool set[SW_COUNT] = {};
    int value[SW_COUNT] = {};
};
static std::mutex g_switch_mutex;
static Switches g_switches;                       // guarded by g_switch_mutex
static std::atomic<unsigned> g_switch_generation{1}; // bumped whenever g_switches changes
static std::once_flag g_switch_env_once;

static void read_switches_from_environment() {
    const char* debug = std::getenv("SPHX_DEBUG_SWITCHES");
    if (!debug || !*debug || std::strcmp(debug, "0") == 0) return;
    std::lock_guard<std::mutex> lock(g_switch_mutex);
    for (int i = 0; i < SW_COUNT; ++i) {
        const char* v = std::getenv(kSwitchNames[i]);
        if (v && *v) {
            g_switches.set[i] = true;
            g_switches.value[i] = std::atoi(v);
        }
    }
    g_switch_generation.fetch_add(1);
}

// The overrides as a planning call sees them: this thread's copy, taken again when they change.
static thread_local Switches t_switches;
static thread_local unsigned t_switches_generation = 0;

int switch_or(Switch which, int fallback) {
    return t_switches.set[which] ? t_switches.value[which] : fallback;
}

unsigned refresh_switches() {
    std::call_once(g_switch_env_once, read_switches_from_environment);
    const unsigned generation = g_switch_generation.load(std::memory_order_acquire);
    if (t_switches_generation != generation) {
        std::lock_guard<std::mutex> lock(g_switch_mutex);
        t_switches = g_switches;
        t_switches_generation = g_switch_generation.load();
    }
    return t_switches_generation;
}

int set_switch(const char* name, int value) {
    // the environment first, so that what is set here wins over it
    std::call_once(g_switch_env_once, read_switches_from_environment);
    if (name != nullptr) {
        for (int i = 0; i < SW_COUNT; ++i) {
            if (std::strcmp(name, kSwitchNames[i]) == 0) {
                std::lock_guard<std::mutex> lock(g_switch_mutex);
                g_switches.set[i] = true;
                g_switches.value[i] = value;
                g_switch_generation.fetch_add(1);
                return SPHX_OK;
            }
        }
    }
    return fail(SPHX_ERR_ARGUMENT, std::string("unknown switch: ") + (name ? name : "(null)"));
}

void reset_switches() {
    std::call_once(g_switch_env_once, read_switches_from_environment);
    std::lock_guard<std::mutex> lock(g_switch_mutex);
    g_switches = Switches();
    g_switch_generation.fetch_add(1);
}

static unsigned pow2_floor(unsigned v) {
    unsigned p = 1;
    while (2 * p <= v) p *= 2;
    return p;
}

static unsigned align4(unsigned v) { return (v + 3u) & ~3u; }

static void plan_closed(size_t n_samples, int l_max, int hard, int mode, size_t elem, Launch* out) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = (l_max + 1) * (l_max + 1);
    g.tile = 64;
    g.n_tiles = static_cast<unsigned>((n_samples + 63) / 64);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    out->workgroups = g.tiles_per_xcd * 8u;
    out->threads = 64;
    const unsigned nyh = static_cast<unsigned>(hard + 1) * (hard + 1);
    const unsigned pad = closed_form_pad(hard);
    const unsigned per = 64 / closed_form_phases(static_cast<unsigned>(elem), mode, hard);
    unsigned at = align4(per * (nyh + pad));
    if (mode >= 1) at = align4(at + per * (3 * nyh + pad));
    if (mode == 2) at = align4(at + per * (9 * nyh + pad));
    out->lds_bytes = at * static_cast<unsigned>(elem);
}

// values_kernel: up to 64 points per workgroup, their rows and tables in LDS. Returns false when that does not
// fit, and the recursion kernel takes over. `with_sums`: the same layout for the lane kernels of the fused
// product, which keep no rows for HBM but the sums of their waves.
static bool plan_values(size_t n_samples, int l_max, size_t elem, int lds_limit, Launch* out,
                        bool with_sums = false) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    if (!with_sums && l_max > 63) return false; // a channel's prefactors: one per lane of a wave
    const unsigned esize = static_cast<unsigned>(elem);
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned vec = 16u / esize;
    // rows a multiple of 8 words long: one vector between them (values_kernel)
    const unsigned row_stride = (ny * (esize / 4u)) % 8u == 0 ? ny + vec : ny;
    const unsigned table_stride = (3u * static_cast<unsigned>(l_max + 1)) | 1u;
    const unsigned tri_all = static_cast<unsigned>(l_max + 1) * (l_max + 2) / 2;
    unsigned allowed = static_cast<unsigned>(switch_or(SW_VALUES_LDS, 160 * 1024));
    if (allowed > static_cast<unsigned>(lds_limit)) allowed = static_cast<unsigned>(lds_limit);
    // Fewer than 64 points per workgroup leave lanes idle, and from some tile on the recursion kernel with its
    // job list is faster: values stop at 24 points in float32 and 32 in float64. The product has far more
    // arithmetic per point to win and goes down to 8 points.
    const unsigned smallest = static_cast<unsigned>(
        with_sums ? switch_or(SW_VJP_MIN_TILE, 8) : switch_or(SW_VALUES_MIN_TILE, elem == 4 ? 24 : 32));
    // Which form of the kernel goes by the shape (sphx_plan_shapes.hpp): tiles of 64 / pack points whose waves
    // evaluate `pack` channels side by side, all lanes at work; one workgroup per CU with all of its LDS and up
    // to sixteen waves, or two with half of it each.
    const ShapeRow* shape = shape_row(with_sums ? 1 : 0, static_cast<int>(elem), l_max);
    const unsigned pack_by_shape = shape ? shape->pack : 1u;
    const int waves_by_shape = shape ? shape->waves : 0;
    const unsigned floor_by_shape = shape ? shape->floor : 32u;
    const bool alone = switch_or(SW_VALUES_ALONE, shape && shape->alone ? 1 : 0) != 0;
    const unsigned smallest_alone = !with_sums && elem == 4 && smallest < 40 && !alone ? 40 : smallest;
    // The tile goes down in steps of four points, so that as many lanes work as rows fit; the product's halves
    // from `floor` on, for the groups of lanes of vjp_groups_kernel.
    const unsigned step = static_cast<unsigned>(with_sums ? switch_or(SW_VJP_TILE_STEP, 4) : switch_or(SW_VALUES_TILE_STEP, 4));
    // Two workgroups per CU (80 KB each) overlap one's tables and flush with the other's arithmetic: preferred,
    // also with fewer lanes at work, over one workgroup with all of LDS unless the shape says otherwise.
    const unsigned half = 80u * 1024u;
    unsigned tile = 0, rows = 0, bytes = 0, sums_elems = 0;
    const unsigned step_floor = static_cast<unsigned>(switch_or(SW_VJP_STEP_FLOOR, static_cast<int>(floor_by_shape)));
    const int sum_waves = switch_or(SW_VALUES_WAVES, waves_by_shape != 0 ? waves_by_shape : 16);
    const unsigned groups_below = static_cast<unsigned>(switch_or(SW_VJP_GROUPS_BELOW, 16)); // (vjp_groups_kernel: eight waves)
    unsigned pack = with_sums ? 1u : static_cast<unsigned>(switch_or(SW_VALUES_PACK, static_cast<int>(pack_by_shape)));
    if (pack != 2 && pack != 4) pack = 1;
    auto search = [&]() {
        for (unsigned limit : {alone ? 0u : (allowed < half ? allowed : half), allowed}) {
            const unsigned least = pack > 1 ? 8u : (limit > half ? smallest_alone : smallest);
            for (unsigned t = 64 / pack; t >= least && t >= 8 && tile == 0;
                 t = step == 0 || (with_sums && t <= step_floor) ? t / 2 : t - step) {
                if (pack > 1 && t != 64 / pack) break;
                rows = (t * row_stride + vec - 1u) / vec * vec;
                // the product: the waves' sums; with fewer than 64 points also copies of the
                // prefactor tables (vjp_groups_kernel)
                // (a workgroup alone on its CU with more than 16 points: room for the sums of
                // up to sixteen waves, unless eight are asked for)
                const unsigned sums = (with_sums && limit > half && t > groups_below && sum_waves > 8 ? 16u : 8u) * 3u * 64u;
                const unsigned extra = !with_sums ? 0u : (t == 64 ? sums : sums + 2u * tri_all);
                bytes = (rows + t * table_stride + extra) * esize;
                if (bytes <= limit) {
                    tile = t;
                    sums_elems = sums;
                }
            }
        }
    };
    search();
    if (tile == 0 && pack > 1) { // (a smaller LDS than the shapes above were measured with)
        pack = 1;
        search();
    }
    if (tile == 0) return false;
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(tile);
    if ((n_samples + tile - 1) / tile > 0x7fffffffull) return false;
    g.n_tiles = static_cast<unsigned>((n_samples + tile - 1) / tile);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    g.rows_elems = row_stride;
    g.off_pts = rows;
    g.off_iter = table_stride;
    g.off_jobs = rows + tile * table_stride; // the product: the waves' sums,
    g.off_F = g.off_jobs + sums_elems;       // and (fewer than 64 points) the prefactor tables
    g.off_Q = g.off_F + tri_all;
    g.points_per_pass = with_sums ? 0u : pack; // values_kernel: channels a wave evaluates side by side
    out->workgroups = g.tiles_per_xcd * 8u;
    // one wave per l channel above the closed forms, eight at most
    // (alone on its CU: up to sixteen; twelve for one channel per wave in float32)
    // (four channels side by side: that kernel exists for up to eight waves only)
    const int most = with_sums ? (sums_elems > 8u * 3u * 64u ? 16 : 8)
                               : (bytes > half && pack != 4 ? (elem == 4 && pack == 1 ? 12 : 16) : 8);
    int waves = switch_or(SW_VALUES_WAVES, waves_by_shape != 0 && alone ? waves_by_shape : most);
    waves = waves < 1 ? 1 : (waves > most ? most : waves);
    // (the product's closed-form slices want at least four; values: one for the tables, one for
    // the closed forms)
    int want = (l_max - 6 + static_cast<int>(pack) - 1) / static_cast<int>(pack);
    // (the product: one or two channels are best with four waves, three or four channels with three, five or
    // six with four)
    if (with_sums) want = want <= 2 ? 4 : (want <= 4 ? 3 : (want <= 6 ? 4 : want));
    if (!with_sums && want < 2) want = switch_or(SW_VALUES_MIN_WAVES, 2);
    out->threads = 64u * static_cast<unsigned>(want < waves ? want : waves);
    out->lds_bytes = bytes;
    return true;
}

// gradients_lanes_kernel: 64, 32 or 16 points per workgroup with their four rows and tables in
// LDS. Returns false when too few points would be resident on a CU for it to pay.
static bool plan_gradient_lanes(size_t n_samples, int l_max, size_t elem, int lds_limit, int cus,
                                Launch* out, bool normalized = true) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    const unsigned esize = static_cast<unsigned>(elem);
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned vec = 16u / esize;
    auto stride_of = [&](unsigned block) { return (block * (esize / 4u)) % 8u == 0 ? block + vec : block; };
    const unsigned s_stride = stride_of(ny), d_stride = stride_of(3u * ny);
    // (closed forms only, l_max <= 6: no tables)
    const unsigned table_stride = l_max <= 6 ? 0u : (3u * static_cast<unsigned>(l_max + 1)) | 1u;
    const unsigned limit = static_cast<unsigned>(lds_limit);
    // Which tile: the one that keeps most points resident on a CU (tile times the workgroups that fit), a tile of
    // 16 counted at three quarters because it leaves three lanes in four idle; between equals the larger tile,
    // unless its workgroup would be alone on the CU (two overlap one another's phases). Below 32 resident points
    // (or 3 x 16) the recursion kernel is the faster one.
    // Few points (one workgroup per CU can take them all): the time of the call is the time of one workgroup, and
    // every workgroup beyond one per CU makes the waves of a CU queue for its vector ALUs with most of their lanes
    // idle. Then the tile is N / CUs, rounded up to a multiple of four.
    unsigned few = 0;
    const unsigned forced_tile = static_cast<unsigned>(switch_or(SW_GRADIENT_LANES_TILE, 0));
    if (cus > 0 && n_samples <= static_cast<size_t>(cus) * 64u) {
        few = static_cast<unsigned>((n_samples + static_cast<size_t>(cus) - 1) / static_cast<size_t>(cus));
        few = (few + 3u) & ~3u;
        if (few < 8u) few = 8u;
    }
    if (forced_tile == 1u) few = 0; // 1: the throughput rule also for few points
    unsigned tile = 0, off_d = 0, off_t = 0, bytes = 0, best = 0, best_groups = 0;
    for (unsigned t : {64u, 32u, 16u, few}) {
        if (t == 0) continue;
        const unsigned od = (t * s_stride + vec - 1u) / vec * vec;
        const unsigned ot = od + (t * d_stride + vec - 1u) / vec * vec;
        const unsigned b = (ot + t * table_stride) * esize;
        if (b > limit) continue;
        unsigned score = (limit / b) * t * (t >= 32 ? 4u : 3u);
        // l_max = 6, closed forms only: 32 points per workgroup, half the lanes idle, but twice as many workgroups in
        // different phases on a CU, and a tile of 32 rows of 49 numbers is a whole number of 128-byte lines (1M points,
        // float32: 127 us against 140 us with 64 points)
        if (l_max == 6 && t == 32) score = 1u << 28;
        if (t == few) score = 1u << 29;
        if (forced_tile == t) score = 1u << 30;
        if (score > best || (score == best && best_groups < 2)) {
            best = score;
            best_groups = limit / b;
            tile = t;
            off_d = od;
            off_t = ot;
            bytes = b;
        }
    }
    if (best < 32u * 4u) tile = 0;
    if (tile == 0 || (n_samples + tile - 1) / tile > 0x7fffffffull) return false;
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(tile);
    g.n_tiles = static_cast<unsigned>((n_samples + tile - 1) / tile);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    g.rows_elems = s_stride;
    g.off_dsph = off_d;
    g.off_ddsph = d_stride;
    g.off_pts = off_t;
    g.off_iter = table_stride;
    out->workgroups = g.tiles_per_xcd * 8u;
    // Eight waves share the closed-form slices and the channels; with one or two channels four are enough and
    // leave room for more workgroups. Closed forms only (l_max <= 6): eight, a slice each. (Six, two of them with
    // two slices, were 1-2 % ahead for normalised float32 at l_max = 6 on boxes whose clocks settle high, 122 us on
    // cfg3 either way, and are 140 us against 122 us on boxes whose clocks settle low: the wave with two slices is
    // then what a workgroup waits for.) Few points (one workgroup per CU, occupancy is no concern): eight waves shorten the longest chain
    // of work in the workgroup, and with three channels or more, or float64 tiles of up to 16 points, sixteen do,
    // two to a channel where that leaves four for the closed forms.
    const bool many = tile == few && l_max > 6 && (l_max >= 9 || (elem == 8 && tile <= 16));
    const int by_shape = l_max <= 6 ? 8 : (l_max <= 8 && tile != few ? 4 : (many ? 16 : 8));
    int waves = switch_or(SW_GRADIENT_LANES_WAVES, by_shape);
    const int most = l_max >= 6 ? 16 : 8; // (the kernels of l_max = 4, 5 exist for 512 threads)
    waves = waves < 1 ? 1 : (waves > most ? most : waves);
    out->threads = 64u * static_cast<unsigned>(waves);
    out->lds_bytes = bytes;
    // Few points, one or two channels: two waves per channel, each with half of its m (the longest chain of the
    // one workgroup a CU has is then half a channel or two slices of the closed forms, not a whole channel; cfg1
    // 10.0 -> 9.0 us). With three channels or more too few waves are left for the slices and nothing is gained.
    const unsigned channels = l_max > 6 ? static_cast<unsigned>(l_max - 6) : 0u;
    const bool halves = tile == few && channels >= 1 && (channels <= 2 ? waves >= 8 : 2u * channels + 4u <= static_cast<unsigned>(waves));
    const int parts = switch_or(SW_GRADIENT_LANES_PARTS, halves ? 2 : 1);
    g.sequence_waves = parts == 2 && 2u * channels <= static_cast<unsigned>(waves) ? 2u : 1u;
    return true;
}

// hessians_lanes_kernel: 64 or 32 points per workgroup with their thirteen rows, tables and
// iterates in LDS. Returns false when 32 points do not fit.
static bool plan_hessian_lanes(size_t n_samples, int l_max, size_t elem, int lds_limit, Launch* out,
                               bool normalized = true) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    const unsigned esize = static_cast<unsigned>(elem);
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned vec = 16u / esize;
    auto stride_of = [&](unsigned block) { return (block * (esize / 4u)) % 8u == 0 ? block + vec : block; };
    const unsigned s_stride = stride_of(ny), d_stride = stride_of(3u * ny), dd_stride = stride_of(9u * ny);
    const unsigned table_stride = (3u * static_cast<unsigned>(l_max + 1)) | 1u;
    const unsigned channels = static_cast<unsigned>(l_max - 1);
    const unsigned most = (elem == 4 ? hessian_lane_threads<float>() : hessian_lane_threads<double>()) / 64u;
    // Waves per channel, each with a part of its m: two where one or two channels would leave the workgroup with
    // one or two waves and that measured faster (l_max = 3 in float32 and for solid harmonics in float64, l_max = 2
    // in float32: 5-20 %).
    const bool shared = (l_max == 3 && (elem == 4 || !normalized)) || (l_max == 2 && elem == 4);
    unsigned parts = static_cast<unsigned>(switch_or(SW_HESSIAN_LANES_PARTS, shared ? 2 : 1));
    if (parts != 1 && parts != 2 && parts != 4) parts = 1;
    while (parts > 1 && parts > most) parts /= 2;
    const unsigned slots = channels * parts <= most ? channels : most / parts;
    const unsigned waves = slots * parts;
    const unsigned limit = static_cast<unsigned>(lds_limit);
    unsigned tile = 0, off_d = 0, off_dd = 0, off_t = 0, off_s = 0, bytes = 0, best = 0, best_groups = 0;
    const unsigned forced_tile = static_cast<unsigned>(switch_or(SW_HESSIAN_LANES_TILE, 0));
    for (unsigned t = 64; t >= 32; t /= 2) {
        const unsigned od = (t * s_stride + vec - 1u) / vec * vec;
        const unsigned odd = od + (t * d_stride + vec - 1u) / vec * vec;
        const unsigned ot = odd + (t * dd_stride + vec - 1u) / vec * vec;
        const unsigned os = ot + t * table_stride;
        const unsigned b = (os + waves * t * table_stride) * esize;
        if (b > limit) continue;
        const unsigned score = forced_tile == t ? 1u << 30 : (limit / b) * t;
        if (score > best || (score == best && best_groups < 2)) {
            best = score;
            best_groups = limit / b;
            tile = t;
            off_d = od;
            off_dd = odd;
            off_t = ot;
            off_s = os;
            bytes = b;
        }
    }
    if (tile == 0 || (n_samples + tile - 1) / tile > 0x7fffffffull) return false;
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(tile);
    g.n_tiles = static_cast<unsigned>((n_samples + tile - 1) / tile);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    g.rows_elems = s_stride;
    g.off_dsph = d_stride;
    g.off_ddsph = dd_stride;
    g.off_F = off_d;
    g.off_Q = off_dd;
    g.off_pts = off_t;
    g.off_iter = table_stride;
    g.off_jobs = off_s;
    g.jobs_per_point = table_stride;
    out->workgroups = g.tiles_per_xcd * 8u;
    g.sequence_waves = parts;
    out->threads = 64u * waves;
    out->lds_bytes = bytes;
    return true;
}

// Threads per workgroup of the recursion kernel: 512, two workgroups to a CU, or 1024, one workgroup with all of
// the CU's LDS and tiles of twice as many points. Two workgroups of 512 on a CU run their stages and their
// flushes against each other as chance has it, and a tile of one or two points leaves the entry lanes and the
// sequence lanes half idle in their last rounds: one workgroup of 1024 is 10-25 % faster with derivatives and
// up to 8 % with values alone (profiles/sweep.json was made with this rule). With few points (below 4 096) 512
// threads stay: more workgroups have a tile then. Not the fused product, which has no such kernel.
// SPHX_GROUP_THREADS = 512 or 1024 overrides the rule.
static unsigned group_threads(size_t n_samples, int mode, size_t elem, bool forward, bool normalized = true,
                              int l_max = -1) {
    // Second derivatives in float64: the entries (l, +m) and (l, -m) as one job need 163-231 registers per lane,
    // more than the 128 that sixteen waves leave. As two jobs solid harmonics need 103-113, normalised ones 128
    // when the jobs of a tile go as one list ordered by kind (plan_recursion sees to both), and sixteen waves gain
    // 5-20 % from l_max = 3 on (cfg4 538 -> 507 us); at l_max = 2 the list is three jobs a point and eight waves
    // are as fast. (A caller that passes no l_max, the path that evaluates float arrays in float64, keeps eight.)
    const bool f64_hessians = mode == 2 && elem == 8;
    if (!forward || (f64_hessians && l_max < 0)) return kRecursionThreads;
    const int want = switch_or(SW_GROUP_THREADS, 0);
    if (want == 512 || want == 1024) return static_cast<unsigned>(want);
    if (f64_hessians && l_max < 3) return kRecursionThreads;
    // (normalised: one-sided jobs are 20 % more work, which sixteen waves make up for at l_max = 3 (12 %), 4, 7 and 8
    // (7, 8, 5 %; every setting measured after 0.4 s of its own launches); nothing in it at 5, 6, 9, 10, behind from 12
    // to 24. From l_max = 25 a tile is a single point and a CU holds one workgroup either way: sixteen waves then,
    // 448 -> 345 us per 1.2 GB at l_max = 25, 368 -> 331 at 26, 360 -> 327 at 28, 319 -> 315 at 32.)
    if (f64_hessians && normalized && !(l_max == 3 || l_max == 4 || l_max == 7 || l_max == 8 || l_max >= 25)) {
        return kRecursionThreads;
    }
    return n_samples >= 4096 ? 2 * kRecursionThreads : kRecursionThreads;
}

// Tile size and LDS layout of the recursion kernel. Returns false when not even one point fits.
// `elem` is the size of the numbers the kernel computes with, `out_elem` that of the coordinates
// and the output arrays (and so of the staged rows): smaller when float arrays are evaluated in
// float64, else the same (0).
static bool plan_recursion(size_t n_samples, int l_max, int mode, bool whole, size_t elem,
                           unsigned budget, int lds_limit, int cus, Launch* out, bool* split_sides,
                           bool normalized = true, size_t out_elem = 0, unsigned threads = kRecursionThreads) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    const int hard = mode == 2 ? 1 : 6;
    const unsigned esize = static_cast<unsigned>(elem);
    const unsigned osize = out_elem == 0 ? esize : static_cast<unsigned>(out_elem);
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned nyh = static_cast<unsigned>(hard + 1) * (hard + 1);
    const unsigned nrow = whole ? ny : ny - nyh;
    const unsigned tri_all = static_cast<unsigned>(l_max + 1) * (l_max + 2) / 2;
    const unsigned arrays = mode + 1;
    unsigned jobs = 0;
    for (int l = hard + 1; l <= l_max; ++l) jobs += l + 1;
    // with the sides split every (l, m > 0) pair is two jobs; the job table is sized for that
    const unsigned jobs_split = 2 * jobs - static_cast<unsigned>(l_max - hard);
    bool may_split = mode == 2 && switch_or(SW_SPLIT_SIDES, 1) != 0;
    auto table_elems_for = [&](bool split) { return ((split ? jobs_split : jobs) * 4 + esize - 1) / esize; };
    // Which division of the work (recursion_kernel): the recursions of the next tile while this one is flushed, or
    // next to its entries (TOGETHER, float64 only). Next to the entries they are ahead where the flush would wait
    // for them: solid second derivatives at l_max = 4 .. 18 (5-11 %, cfg4 557 -> 513 us) and solid gradients up to
    // l_max = 10 (0-11 %) in calls of 32 768 points or more, and gradients from l_max = 27 on, where a recursion is a
    // long chain (10 %). Everywhere else in float64 the other division gains 2-14 %, as in all of float32.
    // (Each division measured after 0.4 s of its own launches: solid gradients l_max = 9, 10 are 6 and 15 % ahead with
    // the recursions apart, solid second derivatives at l_max = 10, 12, 14 by 6, 5, 4 %, behind by 1-3 % at the odd
    // l_max between them and at 16.)
    const bool together_by_shape =
        elem == 8 && ((!normalized && n_samples >= 32768 &&
                       (mode == 2 ? l_max >= 4 && l_max <= 18 && !(l_max == 10 || l_max == 12 || l_max == 14)
                                  : mode == 1 && l_max <= 8)) ||
                      (mode == 1 && l_max >= 27));
    const bool together = elem == 8 && switch_or(SW_RECURSIONS_TOGETHER, together_by_shape ? 1 : 0) != 0;
    g.together = together ? 1u : 0u;
    // per point: the rows, point tables twice and iterates once (together: three times, when a batch is a single tile,
    // and twice)
    // staged rows are `row_stride` apart (recursion_kernel): nrow, or a little more when the rows
    // are cut so that they keep their position within 16 bytes
    // (whole rows a multiple of 64 bytes long, l_max = 3 mod 4, would all start on one LDS bank: 16 bytes are left
    // free after each, which the flush skips; recursion_kernel, row_pad. Not below l_max = 7, where a tile can be
    // shorter than the line its end is carried in.)
    const unsigned row_pad = whole && l_max >= 7 && (ny * osize) % 64u == 0 && switch_or(SW_ROW_PAD, 1) != 0 ? 16u / osize : 0u;
    const unsigned row_stride = nrow + (whole ? row_pad : nyh % (16u / osize));
    g.row_pad = row_pad;
    g.magic_ny = magic_of(ny);
    const unsigned rows_per_point = components_of(mode) * row_stride;
    // (the records of a point and its sequences of iterates are an odd number of words apart)
    const unsigned rest_per_point = (together ? 3u : 2u) * ((8 + 3 * (l_max + 1)) | 1u) + (together ? 2u : 1u) * arrays * (tri_all | 1u);
    unsigned fixed = 0; // bytes
    const unsigned point_bytes = rows_per_point * osize + rest_per_point * esize;
    auto bytes_for = [&](unsigned S) { return S * point_bytes + fixed; };
    const unsigned limit = static_cast<unsigned>(lds_limit);
    for (;;) {
        // 24: alignment slack of the row arrays
        // + 3 lines: a staging region starts at a line boundary of its output array
        fixed = (2 * tri_all + table_elems_for(may_split) + 24) * esize + 2 * 3 * 128u;
        if (bytes_for(1) <= limit || !may_split) break;
        may_split = false; // the longer job table is what does not fit
    }
    // (One row buffer. A second one, flushed by a wave of its own while the next tile is computed, measured 20-60 %
    // slower from l_max = 20 on: a wave that flushes alone waits for its own LDS loads most of the time, and the
    // entry waves lose a wave and half the points per tile.)
    if (bytes_for(1) > limit) return false;
    unsigned S = 1;
    if (bytes_for(1) <= budget) {
        // as many points as the budget holds, a power of two or not: fewer barrier rounds per point (up to 30 %
        // faster, never more than 4 % slower than the power of two below)
        S = (budget - fixed) / point_bytes;
        if (switch_or(SW_TILE_POW2, 0) != 0) S = pow2_floor(S);
        if (S > 64) S = 64;
    }
    // Few points: with the largest tile there would be fewer tiles than workgroups that a launch keeps resident.
    // Then the tile is just large enough to give every one of them a tile (for values and gradients four points
    // at least: below that the closed forms of l <= 6 weigh too much). 500 points: 16-24 us -> 10-13 us.
    if (S > 1 && switch_or(SW_TILE_SMALL_N, 1) != 0) {
        unsigned per_cu = limit / bytes_for(S);
        per_cu = per_cu < 1 ? 1u : (per_cu > 2 ? 2u : per_cu);
        if (mode == 2 && elem == 8) per_cu = 1; // more than 128 registers per lane
        const unsigned long long resident = static_cast<unsigned long long>(cus > 0 ? cus : 1) * per_cu;
        if ((n_samples + S - 1) / S <= resident) {
            unsigned long long enough = (n_samples + resident - 1) / resident;
            const unsigned least = mode < 2 ? 4u : 1u;
            if (enough < least) enough = least;
            if (enough < S) S = static_cast<unsigned>(enough);
        }
    }
    const int forced = switch_or(SW_TILE, 0);
    if (forced > 0 && forced <= 64 && bytes_for(forced) <= limit) {
        S = static_cast<unsigned>(forced);
    }

    // Point tables for several tiles at a time (recursion_kernel, az_shift): as many tiles as
    // wave 0 has lanes for, eight at most, as long as the larger table area keeps the workgroup
    // within the budget (or within what it needs anyway).
    const unsigned point_record = (8 + 3 * static_cast<unsigned>(l_max + 1)) | 1u;
    unsigned az_shift = 0;
    {
        const unsigned allowed = bytes_for(S) > budget ? bytes_for(S) : budget;
        const int cap = switch_or(SW_AZ_SHIFT, 3);
        for (unsigned shift = cap < 0 ? 0u : (cap > 6 ? 6u : static_cast<unsigned>(cap)); shift >= 1; --shift) {
            const unsigned tiles = 1u << shift;
            if (tiles * S > 64) continue;
            const unsigned extra = (2 * tiles - (together ? 3 : 2)) * S * point_record * esize;
            if (bytes_for(S) + extra <= allowed || bytes_for(S) + extra <= budget) {
                az_shift = shift;
                break;
            }
        }
    }
    const unsigned table_slots = together && az_shift == 0 ? 3u : 2u << az_shift;

    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(S);
    g.az_shift = az_shift;
    // Waves of their own for the closed forms of l <= 6 (whole rows): with sixteen waves and float32 gradients, where
    // the tile otherwise waits for the entry waves that carry a slice on top of their jobs: three of them (l_max =
    // 9 .. 18: 1-4 % over none, one or two are 5-20 % behind). In float64 the closed forms are too much for three or
    // four waves (3-10 % behind none). At l_max = 8, where the closed forms are 49 of the 81 entries, normalised
    // harmonics take four (213 -> 203 us per 1.2 GB, each setting after 0.4 s of its own launches).
    g.slice_waves = 0;
    const bool slices_apart = threads > kRecursionThreads && mode == 1 && elem == 4;
    if (whole && mode < 2) {
        const int want = switch_or(SW_SLICE_WAVES, slices_apart && S >= 9 ? (l_max == 8 && normalized ? 4 : 3) : 0);
        g.slice_waves = want < 0 ? 0u : (want > 4 ? 4u : static_cast<unsigned>(want));
    }
    g.sequence_waves = S * arrays * static_cast<unsigned>(l_max - hard) > 64 ? 2u : 1u;
    // Split the sides when that lets the entries of a tile go through the entry waves in fewer rounds than it
    // costs, a one-sided job being about 0.6 of a two-sided one. Normalised float32 is the exception: always split,
    // because the two-sided kernel needs 152 registers per lane, so that only one workgroup of 512 threads fits on
    // a CU, and the one-sided 116. For solid harmonics in float32 both fit twice (119 and 88 registers) and the
    // rule holds; float64 with the sides always split loses 10-20 % at most l_max.
    const unsigned one_side_costs = static_cast<unsigned>(switch_or(SW_SPLIT_RATIO, elem == 4 && normalized ? 1 : 6));
    unsigned wide = 0;
    auto per_pass = [&](unsigned j) { return j >= wide ? 1u : wide / j; };
    // rounds of the entry lanes per tile: whole points side by side, or (fewer, where the
    // points leave lanes idle) the jobs of all points as one list
    auto rounds_by_point = [&](unsigned j) {
        return ((S + per_pass(j) - 1) / per_pass(j)) * ((j + wide - 1) / wide);
    };
    auto rounds = [&](unsigned j) {
        const unsigned as_list = (S * j + wide - 1) / wide;
        const unsigned by_point = rounds_by_point(j);
        return S >= 3 && per_pass(j) <= 2 && as_list < by_point ? as_list : by_point;
    };
    // rounds of the entry waves per tile, in tenths of two-sided jobs, with `waves` sequence waves
    auto entry_cost = [&](unsigned waves, bool* split) {
        // (together: wave 0 and the sequence waves compute no entries)
        wide = threads - 64 * ((together ? 1 + waves : 0) + g.slice_waves);
        // (with two or more points per tile the jobs go as a list ordered by kind, which fills the lanes without
        // splitting, and the two-sided job shares the common factors: 5-15 % faster; with one point per tile
        // splitting stays)
        *split = may_split && S < 2 && one_side_costs * rounds(jobs_split) < 10 * rounds(jobs);
        // (float64 in workgroups of 1024 threads: only the one-sided job fits a lane's 128 registers)
        if (may_split && mode == 2 && elem == 8 && threads > kRecursionThreads) *split = true;
        return *split ? one_side_costs * rounds(jobs_split) : 10 * rounds(jobs);
    };
    // The sequence waves run the recursions of the next tile while the other waves flush this one; the tile waits for
    // whichever takes longer. More of them finish the recursions sooner and leave fewer waves to keep stores in
    // flight. By measurement with two to eight of sixteen waves: gradients four in float32 (l_max = 10-16: 57-62 %
    // with two, 66-69 % with four) and three in float64; second derivatives in float32 six for normalised harmonics
    // and three for solid ones, whose entries are shorter and whose flush weighs more (l_max = 8: 72.6 % with three,
    // 65 % with six; two from l_max = 16 on); in float64 two, three at both ends of the l_max range.
    if (together) {
        // Next to the entries a sequence wave takes a wave from them. Sixteen waves: gradients as few rounds of
        // recursions as four waves would need, with as few waves as that takes; second derivatives, where the
        // entries weigh more, two, three at both ends of the l_max range; values three. Eight waves: one where it
        // saves the entry waves a round per tile and for values alone, whose recursions are a third of the work;
        // second derivatives keep two.
        const unsigned recursions = S * arrays * static_cast<unsigned>(l_max - hard);
        if (threads > kRecursionThreads) {
            if (mode == 1) {
                const unsigned least = (recursions + 255u) / 256u;
                g.sequence_waves = 2;
                while (g.sequence_waves < 4 && (recursions + 64u * g.sequence_waves - 1u) / (64u * g.sequence_waves) > least) {
                    ++g.sequence_waves;
                }
            } else if (mode == 2) {
                g.sequence_waves = l_max <= 4 || l_max >= 22 ? 3u : 2u;
            } else {
                g.sequence_waves = 3;
            }
        } else if (g.sequence_waves == 2 && mode != 2) {
            bool split_one = false, split_two = false;
            const unsigned with_one = entry_cost(1, &split_one);
            const unsigned with_two = entry_cost(2, &split_two);
            if (mode == 0 || with_one < with_two) g.sequence_waves = 1;
        }
    } else if (threads > kRecursionThreads) {
        if (mode == 1) {
            g.sequence_waves = elem == 4 ? 4 : 3;
        } else if (mode == 2 && elem == 4) {
            g.sequence_waves = normalized ? 6 : (l_max <= 15 ? 3 : 2);
        } else if (mode == 2) {
            g.sequence_waves = l_max <= 4 || l_max >= 22 ? 3u : 2u;
        } else {
            // values alone (l_max from 34 on, where no other kernel holds the rows): the recursions are a third
            // of the work and the flush is short: float32 l_max = 40 344 us with three, 310 with four, 281 with eight
            g.sequence_waves = elem == 4 ? 8 : 4;
        }
        // (the shapes at which another number was measured to be ahead, with or without the flush at raised priority)
        const PriorityRow* row = priority_row(mode, static_cast<int>(elem), normalized, l_max);
        if (row != nullptr && row->sequence_waves != 0 && n_samples >= (mode == 2 ? 8192u : 32768u)) {
            g.sequence_waves = row->sequence_waves;
        }
    } else if (mode == 0) {
        g.sequence_waves = 1;
    }
    {
        // (at least four waves flush)
        const int forced_seq = switch_or(SW_SEQUENCE_WAVES, 0);
        if (forced_seq >= 1) g.sequence_waves = static_cast<unsigned>(forced_seq);
        const unsigned most = together ? 4u : threads / 64u - 5u;
        if (g.sequence_waves > most) g.sequence_waves = most;
    }
    entry_cost(g.sequence_waves, split_sides); // leaves `wide` as it will be
    g.jobs_per_point = *split_sides ? jobs_split : jobs;
    g.magic_jobs = magic_of(g.jobs_per_point);
    {
        // the kinds of jobs in the order of the job table (recursion_kernel)
        const unsigned sides = *split_sides ? 2u : 1u;
        const unsigned levels = static_cast<unsigned>(l_max - hard);
        unsigned bulk = 0;
        for (int l = hard + 1; l <= l_max; ++l) bulk += l >= 2 ? static_cast<unsigned>(l - 2) : 0u;
        g.kind_jobs[0] = sides * bulk;
        g.kind_jobs[1] = sides * levels;
        g.kind_jobs[2] = levels;
        for (int k = 0; k < 3; ++k) g.kind_magic[k] = g.kind_jobs[k] ? magic_of(g.kind_jobs[k]) : 0u;
    }
    g.points_per_pass = per_pass(g.jobs_per_point);
    // The jobs of a tile as one list. Values: the list is point after point and costs a few instructions per job, so
    // only where it saves a round and few points go side by side anyway. With derivatives the list is ordered by
    // kind of job first (recursion_kernel), which keeps the lanes of a wave on one branch of entry_job: side by
    // side, the 77 one-sided jobs of a point at l_max = 8 with second derivatives put all seven kinds into every
    // wave and 41 % of the lanes were active on average (20-35 % faster as a list). With one or two points per tile
    // the list loses unless it saves a round, and so it does for solid second derivatives in float64 in workgroups
    // of 512 threads where the points side by side fill the lanes anyway. Second derivatives with two points per
    // tile: the list unless the sides are split.
    const int want_list = switch_or(SW_JOB_LIST, -1);
    const bool saves_a_round = (S * g.jobs_per_point + wide - 1) / wide < rounds_by_point(g.jobs_per_point);
    // lanes that points side by side would fill, in percent
    const unsigned fill = 100u * g.points_per_pass * g.jobs_per_point / wide;
    const bool cheap_jobs = mode == 2 && elem == 8 && !normalized; // no chain rule, few branches
    // (normalised second derivatives in float64 in workgroups of 1024 threads exist as a list only)
    const bool must_list = mode == 2 && elem == 8 && normalized && threads > kRecursionThreads;
    // (values in workgroups of 1024 threads: always the list, 15 % faster; solid second derivatives in float64
    // in workgroups of 1024 threads, whose sides are two jobs: always the list as well)
    const bool by_shape = mode == 0   ? (threads > kRecursionThreads ? S >= 2 : saves_a_round && S >= 3 && g.points_per_pass <= 2)
                          : mode == 1 ? S >= 3 || (saves_a_round && S >= 2)
                                      : (S >= 3 && !(cheap_jobs && fill >= 90u)) || (S == 2 && !*split_sides) ||
                                            (saves_a_round && S >= 2) ||
                                            (cheap_jobs && threads > kRecursionThreads && S >= 2);
    if (must_list || want_list == 2 || (want_list == 1 && saves_a_round) || (want_list < 0 && by_shape)) {
        g.points_per_pass = 0;
    }

    // in front of every staging region, room for the part of a 128-byte line that precedes the
    // tile's run (recursion_kernel, flush_run)
    const unsigned line = whole ? 128u / osize : 16u / osize;
    unsigned at = align4(S * row_stride + line);
    g.off_dsph = at;
    if (mode >= 1) at = align4(at + S * 3 * row_stride + line);
    g.off_ddsph = at;
    if (mode == 2) at = align4(at + S * 9 * row_stride + line);
    g.rows_elems = at;
    g.tables_at = at * osize; // a multiple of 16: `at` is one of 4
    at = 0; // from here on in numbers of the arithmetic type, counted from tables_at
    g.off_F = at;
    at += tri_all;
    g.off_Q = at;
    at += tri_all;
    g.off_pts = at;
    at += table_slots * S * point_record;
    g.off_iter = at;
    at += (together ? 2u : 1u) * S * arrays * (tri_all | 1u);
    g.off_jobs = at;
    at += table_elems_for(may_split);
    out->lds_bytes = g.tables_at + at * esize;
    out->threads = threads;
    if (out->lds_bytes > limit) return false;
    // Jobs point by point, one point per pass, with derivatives: in the last round of a point the jobs with
    // |m| = l, |m| = l - 1 and m = 0 are moved to wave boundaries of the entry lanes where the lanes of that round
    // allow it, because a wave runs the branch of every kind of job it holds one after the other and the tile waits
    // for the slowest wave. The gaps are places without a job at the end of the job table. With one workgroup of
    // 1024 threads on a CU this pays (float64 gradients l_max = 32: 290 -> 249 us per 1.2 GB); with two workgroups
    // of 512, how their stages and flushes fall against each other decides, and nothing in the kernel controls
    // that: off there (SPHX_SPREAD_KINDS).
    g.kind_at[0] = g.kind_at[1] = g.kind_at[2] = 0;
    if (mode >= 1 && !*split_sides && g.points_per_pass == 1 && switch_or(SW_SPREAD_KINDS, threads > kRecursionThreads ? 1 : 0) != 0) {
        const unsigned levels = g.kind_jobs[1], bulk = g.kind_jobs[0], jobs_now = g.jobs_per_point;
        const unsigned waves = wide / 64u;
        const unsigned base = jobs_now / wide * wide; // first job of the last round
        if (jobs_now % wide != 0 && bulk >= base && levels != 0) {
            const unsigned bulk_waves = (bulk - base + 63u) / 64u;
            const unsigned spare = bulk_waves * 64u - (bulk - base); // lanes free in the bulk's last wave
            const unsigned level_waves = (levels + 63u) / 64u;
            const unsigned after_bulk = base + bulk_waves * 64u;
            unsigned at_l = 0, at_l1 = 0, at_0 = 0;
            if (bulk_waves + 3u * level_waves <= waves) { // every kind its own waves
                at_l = after_bulk;
                at_l1 = at_l + level_waves * 64u;
                at_0 = at_l1 + level_waves * 64u;
            } else if (levels <= spare && bulk_waves + 2u * level_waves <= waves) {
                at_0 = bulk; // m = 0, the cheapest, shares the bulk's last wave
                at_l = after_bulk;
                at_l1 = at_l + level_waves * 64u;
            } else if (2u * levels <= 64u && bulk_waves + 2u <= waves) {
                at_l = after_bulk; // m = 0 shares a wave with |m| = l
                at_0 = at_l + levels;
                at_l1 = at_l + 64u;
            }
            if (at_l != 0) {
                unsigned padded = at_l + levels;
                if (at_l1 + levels > padded) padded = at_l1 + levels;
                if (at_0 + levels > padded) padded = at_0 + levels;
                const unsigned more = ((padded - jobs_now) * 4u + esize - 1u) / esize * esize; // bytes
                if (padded <= base + wide && out->lds_bytes + more <= limit) {
                    g.kind_at[0] = at_l;
                    g.kind_at[1] = at_l1;
                    g.kind_at[2] = at_0;
                    g.jobs_per_point = padded;
                    g.magic_jobs = magic_of(padded);
                    out->lds_bytes += more;
                }
            }
        }
    }

    g.n_tiles = static_cast<unsigned>((n_samples + S - 1) / S);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    // Chunks of consecutive tiles per workgroup: only where a tile is one run per array, and a run is at least a
    // line long (so that a carried part never spans two tiles). About eight points per chunk: chunks of eight tiles
    // whatever their size were as good for tiles of one or two points and 6-13 % worse for larger ones.
    g.chunk_shift = 0;
    if (whole && S * nrow * osize >= 128u) {
        const int want = switch_or(SW_CHUNK_SHIFT, S >= 5 ? 0 : (S >= 3 ? 1 : (S == 2 ? 2 : 3)));
        g.chunk_shift = want < 0 ? 0u : (want > 10 ? 10u : static_cast<unsigned>(want));
    }
    unsigned per_cu = limit / out->lds_bytes;
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 2048u / threads) per_cu = 2048u / threads; // 2048 lanes per CU
    unsigned want = (static_cast<unsigned>(cus) * per_cu + 7u) & ~7u;
    // Few points: shorter chunks, down to single tiles, until every resident workgroup has one (10 000 points at
    // l_max = 8 are 625 tiles of 16: in chunks of 8 they kept 80 workgroups busy for 41 us, as single tiles they take
    // 512 and a third of the time).
    auto chunks_in_xcd = [&]() { return (g.tiles_per_xcd + (1u << g.chunk_shift) - 1u) >> g.chunk_shift; };
    while (g.chunk_shift > 0 && chunks_in_xcd() * 8u < want) --g.chunk_shift;
    const unsigned chunks_per_xcd = chunks_in_xcd();
    unsigned need = chunks_per_xcd * 8u;
    out->workgroups = want < need ? want : need;
    if (out->workgroups < 8) out->workgroups = 8;
    return true;
}

// Wave priorities of the persistent kernels (Tiling::priorities): 1 = the flushing waves run at raised priority,
// by the table of shapes in sphx_plan_shapes.hpp, for launches of `least` tiles or more per workgroup; the kernel's
// first division of its work (together) has no waves that only flush. SPHX_WAVE_PRIORITIES overrides (2, 3: the waves
// that prepare the next tile, too).
static unsigned wave_priorities(int mode, size_t elem, bool normalized, int l_max, unsigned n_tiles,
                                unsigned workgroups, unsigned least, bool forward) {
    const PriorityRow* row = priority_row(mode, static_cast<int>(elem), normalized, l_max);
    const bool by_shape = forward && n_tiles / least >= workgroups && row != nullptr;
    return static_cast<unsigned>(switch_or(SW_WAVE_PRIORITIES, by_shape ? static_cast<int>(row->priorities) : 0));
}

// Choose kernels, tile sizes and LDS layouts. `lds_limit` / `cus` describe the device.
int make_plan(size_t n_samples, int l_max, int mode, size_t elem, int lds_limit, int cus, Plan* plan,
              bool lane_kernels, bool normalized) {
    if (l_max < 0) return fail(SPHX_ERR_ARGUMENT, "l_max must be non-negative");
    if (mode < 0 || mode > 2) return fail(SPHX_ERR_ARGUMENT, "unknown derivative selector");
    if (l_max > SPHX_TABLE_LMAX) {
        return fail(SPHX_ERR_UNSUPPORTED,
                    "l_max = " + std::to_string(l_max) + " exceeds the device prefactor tables (" +
                        std::to_string(SPHX_TABLE_LMAX) + ")");
    }
    if ((n_samples + 63) / 64 > 0x7fffffffull) {
        return fail(SPHX_ERR_UNSUPPORTED, "too many samples for one launch");
    }
    const int hard = mode == 2 ? 1 : 6;
    plan->lanes = false;
    plan->closed_only = l_max <= hard;
    plan->whole = true;
    plan->split_sides = false;
    plan->pairs = false;
    // Gradients in closed form, where the rows of a tile are so long that few single-wave workgroups of
    // closed_form_kernel share a CU: the lanes kernel instead, which cuts the closed forms in slices for six or
    // eight waves and flushes with all of them (5-25 % faster at l_max = 6, at l_max = 5 in float64 and at
    // l_max = 4 for normalised float32, at every size from 10 000 points to 2M; not below).
    const bool in_slices = l_max == 6 || (l_max == 5 && elem == 8) || (l_max == 4 && elem == 4 && normalized);
    if (plan->closed_only && lane_kernels && mode == 1 && in_slices && switch_or(SW_GRADIENT_LANES, 1) != 0 &&
        plan_gradient_lanes(n_samples, l_max, elem, lds_limit, cus, &plan->closed, normalized)) {
        plan->closed_only = false;
        plan->lanes = true;
        return SPHX_OK;
    }
    if (plan->closed_only) {
        plan_closed(n_samples, l_max, l_max, mode, elem, &plan->closed);
        return SPHX_OK;
    }
    // Values alone where the rows of few points fill LDS: pairs_kernel (below, with the derivatives), which keeps
    // the recursions of the next tile and the flush of this one side by side: 10-35 % faster than values_kernel
    // (the recursion kernel from l_max = 34) from l_max = 24 in float32 and 19 in float64. Below, a point's pairs
    // leave the entry lanes idle and values_kernel is ahead (float32 l_max = 23: 50.7 % against 44.2 %).
    if (lane_kernels && mode == 0 && l_max > hard) {
        const int pairs = switch_or(SW_PAIRS, 1);
        const bool pairs_by_shape = n_samples >= 32768 && (elem == 4 ? l_max >= 24 : l_max >= 19);
        if (pairs == 2 || (pairs == 1 && pairs_by_shape)) {
            PairsChoice want;
            want.tile = static_cast<unsigned>(switch_or(SW_PAIRS_TILE, 0));
            want.batch_tiles = static_cast<unsigned>(switch_or(SW_PAIRS_BATCH, 0));
            want.prep_waves = static_cast<unsigned>(switch_or(SW_PAIRS_PREP_WAVES, 0));
            want.sequence_waves = static_cast<unsigned>(switch_or(SW_PAIRS_SEQUENCE_WAVES, 0));
            want.chunk_shift_plus_one = static_cast<unsigned>(switch_or(SW_PAIRS_CHUNK, -1) + 1);
            if (const PriorityRow* row = priority_row(mode, static_cast<int>(elem), normalized, l_max)) {
                // (the shapes at which another number of sequence waves than the planner's estimate was measured ahead)
                if (want.sequence_waves == 0) want.sequence_waves = row->sequence_waves;
            }
            if (plan_pairs(n_samples, l_max, mode, elem, elem, lds_limit, cus, want, &plan->pairs_launch)) {
                PairsLaunch& made = plan->pairs_launch;
                made.g.priorities = wave_priorities(mode, elem, normalized, l_max, made.g.n_tiles, made.workgroups, 32u, true);
                plan->pairs = true;
                return SPHX_OK;
            }
        }
    }
    if (lane_kernels && mode == 0 && plan_values(n_samples, l_max, elem, lds_limit, &plan->closed)) {
        plan->lanes = true;
        return SPHX_OK;
    }
    // Second derivatives at small l_max: one point per lane where that was measured to be faster
    // than the recursion kernel (SPHX_HESSIAN_LANES: 0 never, 2 wherever the rows fit).
    const int hessian_lanes = switch_or(SW_HESSIAN_LANES, 1);
    // (Since the recursion kernel takes its jobs as a list ordered by kind it wins from l_max = 4 on; the lanes keep
    // l_max <= 3 in float32 and, for calls too small for workgroups of 1024 threads, solid l_max = 3 in float64.)
    const bool hessian_lanes_pay = elem == 4 ? l_max <= 3 : (l_max == 3 && !normalized && n_samples < 32768);
    if (lane_kernels && mode == 2 && (hessian_lanes == 2 || (hessian_lanes == 1 && hessian_lanes_pay)) &&
        plan_hessian_lanes(n_samples, l_max, elem, lds_limit, &plan->closed, normalized)) {
        plan->lanes = true;
        return SPHX_OK;
    }
    // Derivatives where the rows of few points fill LDS: pairs_kernel, whose entry lanes keep one (l, m) pair for
    // the whole launch and whose other work runs while the rows are flushed. Gradients: up to 15 % faster than the
    // recursion kernel from l_max = 20 in float32 and 17 in float64 (cfg5 700 -> 570-620 us); below, a point's
    // pairs leave most of the entry lanes idle. Second derivatives in float64: ahead by 3-9 % at l_max = 20 and,
    // for solid harmonics, from 24 on, for normalised ones by 4, 14 and 12 % at l_max = 19, 21, 23 (and level at 22,
    // 8 % behind at 24), behind by 2-25 % elsewhere; in float32 the recursion
    // kernel's job list by kind fills sixteen waves better. SPHX_PAIRS: 0 never, 2 wherever it fits.
    {
        const int pairs = switch_or(SW_PAIRS, 1);
        // (second derivatives: thirteen rows per point, 8 192 points are as many tiles as 32 768 with gradients)
        const bool pairs_by_shape =
            mode == 1 ? n_samples >= 32768 && (elem == 4 ? l_max >= 20 : l_max >= 17)
                      : n_samples >= 8192 && elem == 8 &&
                            (l_max == 20 || (!normalized && l_max >= 24) ||
                             (normalized && (l_max == 19 || l_max == 21 || l_max == 23)));
        if (lane_kernels && mode >= 1 && l_max > hard && (pairs == 2 || (pairs == 1 && pairs_by_shape))) {
            PairsChoice want;
            want.tile = static_cast<unsigned>(switch_or(SW_PAIRS_TILE, 0));
            want.batch_tiles = static_cast<unsigned>(switch_or(SW_PAIRS_BATCH, 0));
            want.prep_waves = static_cast<unsigned>(switch_or(SW_PAIRS_PREP_WAVES, 0));
            want.sequence_waves = static_cast<unsigned>(switch_or(SW_PAIRS_SEQUENCE_WAVES, 0));
            want.chunk_shift_plus_one = static_cast<unsigned>(switch_or(SW_PAIRS_CHUNK, -1) + 1);
            if (const PriorityRow* row = priority_row(mode, static_cast<int>(elem), normalized, l_max)) {
                // (the shapes at which another number of sequence waves than the planner's estimate was measured ahead)
                if (want.sequence_waves == 0) want.sequence_waves = row->sequence_waves;
            }
            if (plan_pairs(n_samples, l_max, mode, elem, elem, lds_limit, cus, want, &plan->pairs_launch)) {
                PairsLaunch& made = plan->pairs_launch;
                made.g.priorities = wave_priorities(mode, elem, normalized, l_max, made.g.n_tiles, made.workgroups, 32u, true);
                plan->pairs = true;
                return SPHX_OK;
            }
        }
    }
    // Gradients just above the closed forms: the lanes kernel (one point per lane, the channels dealt to the
    // waves) up to l_max = 13 in float32 and wherever its tiles fit in float64; from there the recursion kernel with
    // its jobs as a list ordered by kind is ahead. Where the recursion kernel runs in workgroups of 1024 threads
    // (calls of 32 768 points or more) it is ahead from l_max = 8 on (3-20 %): the lanes keep l_max = 7; at
    // 20 000 points from l_max = 10 on (6-30 %).
    // SPHX_GRADIENT_LANES: 0 never, 2 wherever the rows fit.
    const int gradient_lanes = switch_or(SW_GRADIENT_LANES, 1);
    const bool large_groups = group_threads(n_samples, mode, elem, lane_kernels) > kRecursionThreads && n_samples >= 32768;
    // (float64, normalised, l_max = 7: the recursion kernel is 8 % ahead there, 203 against 219 us per 1.2 GB)
    const bool lanes_by_shape = large_groups ? l_max <= (elem == 8 && normalized ? 6 : 7)
                                             : (n_samples >= 16384 ? l_max <= 9 : elem == 8 || l_max <= 13);
    if (lane_kernels && mode == 1 && gradient_lanes != 0 && (gradient_lanes == 2 || lanes_by_shape) &&
        plan_gradient_lanes(n_samples, l_max, elem, lds_limit, cus, &plan->closed)) {
        plan->lanes = true;
        return SPHX_OK;
    }
    // LDS a workgroup of the recursion kernel may take: half a CU's, so that two share the CU. A workgroup that is
    // alone on its CU anyway (1024 threads, or second derivatives in float64, which need more than 128 registers
    // per lane) takes all of it: 10-30 % faster.
    unsigned threads = group_threads(n_samples, mode, elem, lane_kernels, normalized, l_max);
    const int whole_cu = (mode == 2 && elem == 8) || threads > kRecursionThreads ? lds_limit : 80 * 1024;
    const unsigned budget = static_cast<unsigned>(switch_or(SW_TILE_LDS_BUDGET, whole_cu));
    bool fits = plan_recursion(n_samples, l_max, mode, true, elem, budget, lds_limit, cus, &plan->rec,
                               &plan->split_sides, normalized, 0, threads);
    if (fits && mode == 2 && elem == 8 && threads > kRecursionThreads && !plan->split_sides) {
        // (the sides could not be split, an override or a job table that does not fit: eight waves then)
        threads = kRecursionThreads;
        fits = plan_recursion(n_samples, l_max, mode, true, elem, budget, lds_limit, cus, &plan->rec,
                              &plan->split_sides, normalized, 0, threads);
    }
    // With few points per tile the one-lane-per-point closed forms of l <= 6 would leave most of the lanes idle for
    // some two thousand instructions per tile: then the recursion kernel stages l >= 7 only and its wave 0, which
    // mostly waits, writes l <= 6 straight from registers, 64 points at a time (prefix_inside). The price is rows
    // cut in two, each part a run of its own in HBM, which costs the more the shorter the rows are. By measurement
    // (2.5 GB of output, hundreds of calls in a row: in short bursts the last-level cache merges the parts and the
    // cut rows look 10-30 % better than they are) float32 gradients are cut below three points per tile, float64
    // gradients below five, values below eight.
    const int split_below = switch_or(SW_SPLIT_BELOW, mode == 0 ? 8 : (elem == 4 ? 3 : 5));
    const bool cut = plan->rec.g.tile < split_below;
    if (mode < 2 && (!fits || cut)) {
        Launch upper;
        if (plan_recursion(n_samples, l_max, mode, false, elem, budget, lds_limit, cus, &upper,
                           &plan->split_sides, true, 0, threads)) {
            plan->whole = false;
            plan->rec = upper;
            plan->rec.g.prefix_inside = lane_kernels && switch_or(SW_PREFIX_INSIDE, 1) != 0 ? 1u : 0u;
            plan_closed(n_samples, l_max, hard, mode, elem, &plan->closed);
            fits = true;
        }
    }
    if (fits && !lane_kernels && plan->rec.g.points_per_pass == 0) {
        // the fused product has no job-list variant of the kernel: whole points side by side
        const Tiling& g = plan->rec.g;
        const unsigned wide = plan->rec.threads - 64 * ((g.together ? 1 + g.sequence_waves : 0) + g.slice_waves);
        plan->rec.g.points_per_pass = g.jobs_per_point >= wide ? 1u : wide / g.jobs_per_point;
    }
    if (!fits) {
        return fail(SPHX_ERR_UNSUPPORTED,
                    "l_max = " + std::to_string(l_max) +
                        " with this many derivatives needs more LDS for the rows of one point than "
                        "the device offers (" + std::to_string(lds_limit) + " bytes)");
    }
    plan->rec.g.priorities = wave_priorities(mode, elem, normalized, l_max, plan->rec.g.n_tiles, plan->rec.workgroups, 4u,
                                             lane_kernels && plan->whole && plan->rec.g.together == 0);
    return SPHX_OK;
}

// float arrays evaluated in float64 inside the recursion kernel (its O = float, T = double
// variants): which shapes that covers, and the launch. Below the closed-form limit there is no
// recursion kernel to run; the caller then evaluates into a float64 workspace and narrows.
bool make_wide_plan(size_t n_samples, int l_max, int mode, int lds_limit, int cus, Plan* plan, bool normalized) {
    const int hard = mode == 2 ? 1 : 6;
    if (l_max <= hard || l_max > SPHX_TABLE_LMAX || (n_samples + 63) / 64 > 0x7fffffffull) return false;
    plan->lanes = false;
    plan->closed_only = false;
    plan->whole = true;
    plan->split_sides = false;
    plan->pairs = false;
    const unsigned threads = group_threads(n_samples, mode, 8, true);
    const int whole_cu = mode == 2 || threads > kRecursionThreads ? lds_limit : 80 * 1024; // as for float64 arrays (make_plan)
    const unsigned budget = static_cast<unsigned>(switch_or(SW_TILE_LDS_BUDGET, whole_cu));
    bool fits = plan_recursion(n_samples, l_max, mode, true, 8, budget, lds_limit, cus, &plan->rec,
                               &plan->split_sides, normalized, 4, threads);
    // rows cut at l = 7 where few points fit, by the rule for float rows (make_plan)
    const int split_below = switch_or(SW_SPLIT_BELOW, mode == 0 ? 8 : 3);
    if (mode < 2 && (!fits || plan->rec.g.tile < split_below)) {
        Launch upper;
        if (plan_recursion(n_samples, l_max, mode, false, 8, budget, lds_limit, cus, &upper,
                           &plan->split_sides, normalized, 4, threads)) {
            plan->whole = false;
            plan->rec = upper;
            plan->rec.g.prefix_inside = 1u;
            fits = true;
        }
    }
    return fits;
}

int make_vjp_plan(size_t n_samples, int l_max, size_t elem, int lds_limit, int cus, VjpPlan* out) {
    out->use_lanes = out->lane_groups = false;
    if (l_max > 6 && switch_or(SW_VJP_LANES, 1) != 0) {
        out->use_lanes = plan_values(n_samples, l_max, elem, lds_limit, &out->lanes, true);
        // groups of lanes with channels of their own pay off from tiles of 16 points down (20-25 % at l_max = 24);
        // with tiles of 32 the kernel that takes its prefactors from the scalar unit is ahead
        out->lane_groups = out->use_lanes && out->lanes.g.tile <= switch_or(SW_VJP_GROUPS_BELOW, 16);
    }
    if (out->use_lanes) return SPHX_OK;
    // the closed-form or the recursion kernels with the contraction in place of the flush
    return make_plan(n_samples, l_max, 1, elem, lds_limit, cus, &out->plan, false, true);
}

std::string describe(const Plan& plan, int l_max, int mode, bool is_f64, bool normalized) {
    const std::string t = is_f64 ? "double" : "float";
    const std::string head = t + ", " + std::to_string(mode) + ", " + (normalized ? "true" : "false");
    auto geometry = [](const Launch& l) {
        return " [" + std::to_string(l.g.tile) + " points per tile, " + std::to_string(l.threads) + " threads, " +
               std::to_string(l.lds_bytes) + " B LDS, " + std::to_string(l.workgroups) + " workgroups]";
    };
    std::string text;
    if (plan.pairs) {
        const PairsLaunch& l = plan.pairs_launch;
        text = "pairs_kernel<" + head + "> [" + std::to_string(l.g.tile) + " points per tile, " +
               std::to_string(l.threads) + " threads, " + std::to_string(l.lds_bytes) + " B LDS, " +
               std::to_string(l.workgroups) + " workgroups]" +
               ((l.g.priorities & 1u) != 0 ? " (flush at raised priority)" : "");
    } else if (plan.closed_only) {
        text = "closed_form_kernel<" + head + ", " + std::to_string(l_max) + ", false>" + geometry(plan.closed);
    } else if (plan.lanes) {
        const char* names[3] = {"values_kernel", "gradients_lanes_kernel", "hessians_lanes_kernel"};
        text = std::string(names[mode]) + "<" + t + ", " + (normalized ? "true" : "false") +
               (mode == 0 ? ", " + std::to_string(plan.closed.g.points_per_pass) : std::string()) + ">" +
               geometry(plan.closed);
    } else {
        if (!plan.whole && plan.rec.g.prefix_inside == 0) {
            text = "closed_form_kernel<" + head + ", 6, true>" + geometry(plan.closed) + " + ";
        }
        text += "recursion_kernel<" + head + ", " + (plan.whole ? "true" : "false") + ", " +
                (plan.split_sides ? "true" : "false") + ", false, " +
                (plan.rec.g.points_per_pass == 0 ? "true" : "false") + ">" + geometry(plan.rec) +
                (plan.rec.g.together != 0 ? " (recursions next to the entries)" : "") +
                ((plan.rec.g.priorities & 1u) != 0 ? " (flush at raised priority)" : "");
    }
    return text;
}

} // namespace sphx

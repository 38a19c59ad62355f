// The planner: from the shape of a call to kernels, tiles and LDS layouts. Plain host C++.

#include "sphx_plan.hpp"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/sphx_launch.h"

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
    "SPHX_HESSIAN_LANES_PARTS", "SPHX_JOB_LIST",
    "SPHX_PAIRS", "SPHX_PAIRS_BATCH", "SPHX_PAIRS_CHUNK", "SPHX_PAIRS_PREP_WAVES", "SPHX_PAIRS_SEQUENCE_WAVES", "SPHX_PAIRS_TILE",
    "SPHX_PREFIX_INSIDE", "SPHX_SEQUENCE_WAVES", "SPHX_SLICE_WAVES", "SPHX_SPLIT_BELOW",
    "SPHX_SPLIT_RATIO", "SPHX_SPLIT_SIDES", "SPHX_SPREAD_KINDS", "SPHX_TILE", "SPHX_TILE_LDS_BUDGET", "SPHX_TILE_POW2",
    "SPHX_TILE_SMALL_N", "SPHX_VALUES_ALONE", "SPHX_VALUES_LDS", "SPHX_VALUES_MIN_TILE", "SPHX_VALUES_MIN_WAVES",
    "SPHX_VALUES_PACK", "SPHX_VALUES_TILE_STEP", "SPHX_VALUES_WAVES", "SPHX_VJP_GROUPS_BELOW", "SPHX_VJP_LANES", "SPHX_VJP_MIN_TILE", "SPHX_VJP_STEP_FLOOR", "SPHX_VJP_TILE_STEP",
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

// values_kernel: up to 64 points per workgroup, their rows and tables in LDS. Returns false
// when that does not fit, and the recursion kernel takes over.
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
    // Fewer than 64 points per workgroup leave lanes idle, and from some tile on the recursion
    // kernel with its job list is faster. Values, 1 GB of output, us, values kernel against
    // recursion kernel: float32 with two workgroups per CU l_max = 24 (28 points) 306 against 397,
    // l_max = 26 (24 points) 338 against 392; with one workgroup per CU l_max = 28 (44 points) 355
    // against 393, l_max = 29 (40) 370 against 390, l_max = 30 (38) 419 against 391; float64
    // l_max = 22 (32 points) 297 against 305, l_max = 23 (30) 319 against 302.
    // The product keeps no rows for HBM in LDS and has far more arithmetic per point to win:
    // it goes down to 8 points (l_max = 24 float64, 200k points: 830 us with 16 points per
    // workgroup against 1 456 us through the recursion kernel).
    const unsigned smallest = static_cast<unsigned>(
        with_sums ? switch_or(SW_VJP_MIN_TILE, 8) : switch_or(SW_VALUES_MIN_TILE, elem == 4 ? 24 : 32));
    // Between tiles of 24-44 points, with lanes idle, and the recursion kernel lie two more forms
    // of the values kernel: one workgroup per CU with all of its LDS, up to 64 points and up to
    // sixteen waves, and tiles of 32 or 16 points whose waves evaluate two or four channels side
    // by side, all lanes at work. Which is fastest goes by the shape, not by a rule (row lengths,
    // channels per wave and workgroups per CU all change with l_max). 1 GB of values, us, in the
    // order: tile that fits half of LDS / one workgroup with all of LDS / two channels, 32 points,
    // in half of LDS / the same with all of LDS / four channels, 16 points / recursion kernel.
    // float32:
    //   l_max 18 216 263 216 224 249 412    l_max 19 248 285 291 290 289 418    l_max 20 238 270 250 250 279 403
    //   l_max 21 254 262 248 252 268 397    l_max 22 271 260 238 239 260 389    l_max 23 319 288   - 427 341 425
    //   l_max 24 285 287   - 373 296 398    l_max 25 319 295   - 366 286 397    l_max 26 317 300   - 350 275 393
    //   l_max 27   - 333   - 359 393 419    l_max 28   - 317   - 334 354 393    l_max 29   - 329   - 326 342 389
    //   l_max 30   - 357   - 317 332 391    l_max 31   - 360   - 324 348 389    l_max 32   - 368   - 300 313 378
    //   l_max 33   - 365   - 297 305 386    l_max 34   - 404   - 418   - 383
    // float64:
    //   l_max 13 220 243   - 282 310 313    l_max 14 224 212   - 239 309 310    l_max 15 258 225   - 257 326 347
    //   l_max 16   - 228   - 360 335 322    l_max 20   - 252   - 299 363 313    l_max 21   - 273   - 303 365 296
    //   l_max 22   - 273   - 281 328 303    l_max 23   - 326   -   - 582 301
    // (Sixteen waves for a workgroup alone on its CU: float64 l_max = 16-21 239, 255, 248, 268, 272, 291 us
    // with eight, 228, 236, 228, 259, 252, 273 with up to sixteen; float32 l_max = 27, 28 340, 327 with
    // eight, 337, 326 with sixteen, 333, 317 with twelve.)
    unsigned pack_by_shape = 1;
    bool alone_by_shape = false;
    if (!with_sums && elem == 4) {
        if (l_max == 21 || l_max == 22 || (l_max >= 29 && l_max <= 33)) pack_by_shape = 2;
        if (l_max == 25 || l_max == 26) pack_by_shape = 4;
        alone_by_shape = l_max == 23;
    } else if (!with_sums) {
        alone_by_shape = l_max == 14 || l_max == 15;
    }
    // The product: tiles go down in steps of four points to 32 and halve from there, to 16 and 8
    // points with groups of lanes (vjp_groups_kernel). One workgroup with all of LDS is faster on
    // some shapes, with a number of waves that goes by the shape as well (the channels and the
    // eight closed-form slices share the waves; more than eight waves need twice the room for
    // their sums, which can cost points). 200k points (400k to l_max = 16), us, tiles in half of LDS /
    // one workgroup per CU with 8 / with up to 12 waves, float64:
    //   l_max 13 257 261 261    l_max 14 498 287 286    l_max 15 519 328 324    l_max 16 538 383 360
    //   l_max 17 289 228 214    l_max 18 299 261 240    l_max 19 315 290 272    l_max 20 330 336 316
    //   l_max 21 588 375 620    l_max 22 613 556 557    l_max 23 627 588 589    l_max 24 640 610 610
    //   l_max 25 660 649 650    l_max 26 675 689 690    l_max 29 804 804 804
    // float32 (l_max = 21, 31 with 16 waves 162, 423):
    //   l_max 19 144 153 135    l_max 20 155 168 154    l_max 21 181 178 172    l_max 22 211 168 185
    //   l_max 23 216 212 201    l_max 24 222 244 224    l_max 25 335 274 255    l_max 26 340 294 276
    //   l_max 27 348 289 313    l_max 28 356 318 342    l_max 29 385 404 370    l_max 30 397 381 422
    //   l_max 31 477 436 442    l_max 32 500 470 645    l_max 33 510 675 676    l_max 34 518 694 695
    //   l_max 35 789 725 726    l_max 36 807 748 748    l_max 37 820 773 773    l_max 40 874 852 851
    // (Tiles that halved all the way: float64 l_max = 10, 15, 16, 17 153, 405, 459, 259 us against 139, 340,
    // 393, 230 with the same number of waves; float32 l_max = 15, 17, 18 166, 118, 135 against 153, 97, 114.)
    // (On some shapes the steps of four go on below 32 points, to tiles of 28, 24 and 20 for the
    // lanes kernel, before the groups of lanes take over. With that, one workgroup per CU with 8 /
    // 12 waves against the best of the above: float64 l_max = 21 375 364 against 375, l_max = 22 444
    // 405 against 559, l_max = 23 468 464 against 589, l_max = 24 565 564 against 611, l_max = 25 598
    // 602 against 649, l_max = 26 719 661 against 677; float32 l_max = 35 692 642 against 725,
    // l_max = 36 678 667 against 749, l_max = 37 718 792 against 773, l_max = 43 866 868 against 909.)
    int waves_by_shape = 0;
    unsigned floor_by_shape = 32;
    if (with_sums && elem == 8) {
        if (l_max >= 14 && l_max <= 26) waves_by_shape = l_max == 25 ? 8 : 12;
        if (l_max >= 21 && l_max <= 26) floor_by_shape = 16;
    } else if (with_sums) {
        if (l_max == 19 || l_max == 23 || l_max == 25 || l_max == 26 || l_max == 29 || l_max == 35 || l_max == 36) {
            waves_by_shape = 12;
        }
        if (l_max == 21 || l_max == 31) waves_by_shape = 16;
        if (l_max == 22 || l_max == 27 || l_max == 28 || l_max == 30 || l_max == 32 || (l_max >= 37 && l_max <= 40) ||
            l_max == 43) {
            waves_by_shape = 8;
        }
        if ((l_max >= 35 && l_max <= 37) || l_max == 43) floor_by_shape = 16;
    }
    if (waves_by_shape != 0) alone_by_shape = true;
    const bool alone = switch_or(SW_VALUES_ALONE, alone_by_shape ? 1 : 0) != 0;
    const unsigned smallest_alone = !with_sums && elem == 4 && smallest < 40 && !alone ? 40 : smallest;
    // Values: the tile goes down in steps of 4 points, so that as many lanes work as rows fit
    // (l_max = 16: 60 points where halving leaves 32, 202 against 278 us in float32, 240 against
    // 352 in float64; steps of 1 or 2 gain nothing more and some odd sizes lose). The product halves.
    // (the product: the same above 32 points, halves from there down, for the groups of lanes of
    // vjp_groups_kernel)
    const unsigned step = static_cast<unsigned>(with_sums ? switch_or(SW_VJP_TILE_STEP, 4) : switch_or(SW_VALUES_TILE_STEP, 4));
    // Two workgroups per CU (80 KB each) overlap one's tables and flush with the other's
    // arithmetic: preferred, also with fewer lanes at work, over one workgroup with all of LDS
    // (l_max = 16 float32, 500k points, 32 points against 64: 142 against 164 us; l_max = 12
    // float64: 115 against 146).
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
    // the product, 0.8 GB of sph_grad, us: l_max = 9, 10 (three and four channels) 266, 310 with
    // four waves, 207, 282 with three (float64 279, 333 against 233, 304); l_max = 12 350 with six,
    // 316 with four (float64 385 against 321); one or two channels are best with four
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
    // Which tile: the one that keeps most points resident on a CU (tile times the workgroups
    // that fit), a tile of 16 counted at three quarters because it leaves three lanes in four
    // idle; between equals the larger tile, unless its workgroup would be alone on the CU (two
    // overlap one another's phases). Measured, 500k points, float32: l_max = 7 105 us with
    // 2 x 64 points against 119 with 4 x 32; l_max = 9 173 us with 2 x 32 against 186 with 64;
    // l_max = 13 357 us with 3 x 16 against 433 with 32; l_max = 15 579 us with 32 against 651
    // with 2 x 16. Below 32 resident points (or 3 x 16) the recursion kernel is the faster one
    // (l_max = 18: 1 038 us against 1 236).
    // Few points (one workgroup per CU can take them all): the time of the call is the time of
    // one workgroup, and every workgroup beyond one per CU makes the waves of a CU queue for its
    // vector ALUs with most of their lanes idle. Then the tile is N / CUs, rounded up to a
    // multiple of four: cfg1 (10 000 points, float64 l_max = 8) 11.8 us with 632 tiles of 16,
    // 16.1 us with 320 tiles of 32 (one per CU at a time: two rounds), see below for tiles of 40.
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
        // l_max = 6, closed forms only: 32 points per workgroup, half the lanes idle, but twice as
        // many workgroups in different phases on a CU (1M points, float32: 127 us against 140 us
        // with 64 points; a tile of 32 rows of 49 numbers is a whole number of 128-byte lines,
        // tiles of 24, 28, 36, 40, 48 points took 143-164 us)
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
    // Eight waves share the closed-form slices and the channels; with one or two channels four
    // are enough and leave room for more workgroups (1.5 GB of output: float64 l_max = 8 469 us
    // with eight waves, 345 with four; float32 l_max = 7, 8 286, 274 against 273, 261; from three
    // channels on eight waves are faster, l_max = 12: 357 against 411).
    // (few points: one workgroup per CU, occupancy is no concern and eight waves shorten the
    // longest chain of work in the workgroup)
    // (closed forms only, l_max <= 6: eight; six for normalised float32 at l_max = 6, 127 us
    // against 130 us with eight and 136-138 us with four or five)
    // (few points, three channels or more, or float64 tiles of up to 16 points: sixteen waves, two
    // to a channel where that leaves four for the closed forms; 10 000 points, us, eight waves
    // against sixteen: float32 l_max = 10 9.5 against 8.6, l_max = 12 11.8 against 10.9; float64
    // l_max = 8 with 2 000 points 8.0 against 6.2; one or two channels at 40 points per tile gain
    // nothing, float64 l_max = 8 9.2 against 9.1, l_max = 7 7.9 against 8.3)
    const bool many = tile == few && l_max > 6 && (l_max >= 9 || (elem == 8 && tile <= 16));
    const int by_shape = l_max <= 6 ? (l_max == 6 && elem == 4 && normalized && tile != few ? 6 : 8)
                                    : (l_max <= 8 && tile != few ? 4 : (many ? 16 : 8));
    int waves = switch_or(SW_GRADIENT_LANES_WAVES, by_shape);
    const int most = l_max >= 6 ? 16 : 8; // (the kernels of l_max = 4, 5 exist for 512 threads)
    waves = waves < 1 ? 1 : (waves > most ? most : waves);
    out->threads = 64u * static_cast<unsigned>(waves);
    out->lds_bytes = bytes;
    // Few points, one or two channels: two waves per channel, each with half of its m (the longest
    // chain of the one workgroup a CU has is then half a channel or two slices of the closed
    // forms, not a whole channel). Measured on one device, one wave per channel against two, us:
    // float64 10 000 points l_max = 8 10.0 against 9.0, l_max = 7 8.7 against 7.8; float32
    // l_max = 8 7.6 against 6.7, 2 000 points 7.0 against 5.6. With three channels two waves are
    // left for the eight slices and nothing is gained (float64 l_max = 9 10.2 against 10.5), with
    // four channels none (l_max = 10: 9.5 against 9.1 in float32, 9.9 against 10.2 in float64).
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
    // Waves per channel, each with a part of its m: two where one or two channels would leave the
    // workgroup with one or two waves (80 MB of output, us, one against two: float32 l_max = 3
    // 99 against 83, solid 80 against 70, 20 000 points 10.9 against 9.1; l_max = 2 74 against 70,
    // solid 58 against 61; float64 l_max = 3 solid 85 against 73, normalised 105 against 151).
    const bool shared = (l_max == 3 && (elem == 4 || !normalized)) || (l_max == 2 && elem == 4 && normalized);
    unsigned parts = static_cast<unsigned>(switch_or(SW_HESSIAN_LANES_PARTS, shared ? 2 : 1));
    if (parts != 1 && parts != 2 && parts != 4) parts = 1;
    while (parts > 1 && parts > most) parts /= 2;
    const unsigned slots = channels * parts <= most ? channels : most / parts;
    const unsigned waves = slots * parts;
    const unsigned limit = static_cast<unsigned>(lds_limit);
    unsigned tile = 0, off_d = 0, off_dd = 0, off_t = 0, off_s = 0, bytes = 0, best = 0, best_groups = 0;
    for (unsigned t = 64; t >= 32; t /= 2) {
        const unsigned od = (t * s_stride + vec - 1u) / vec * vec;
        const unsigned odd = od + (t * d_stride + vec - 1u) / vec * vec;
        const unsigned ot = odd + (t * dd_stride + vec - 1u) / vec * vec;
        const unsigned os = ot + t * table_stride;
        const unsigned b = (os + waves * t * table_stride) * esize;
        if (b > limit) continue;
        const unsigned score = (limit / b) * t;
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

// Threads per workgroup of the recursion kernel: 512, two workgroups to a CU, or 1024, one
// workgroup with all of the CU's LDS and tiles of twice as many points (not the fused product,
// and not second derivatives in float64, whose entry jobs need more than the 128 registers a
// lane of sixteen waves has). Two workgroups of 512 on a CU run their stages and
// their flushes against each other as chance has it, and a tile of one or two points leaves the
// entry lanes and the sequence lanes half idle in their last rounds; one workgroup of 1024
// measured, 1.2 GB of output, us, 512 against 1024: gradients float32 l_max = 14, 20, 24, 28,
// 32, 36 283, 306, 323, 329, 331, 342 against 245, 249, 259, 253, 267, 268 (l_max = 40 288
// against 290); float64 l_max = 12, 16, 20, 24, 32 303, 307, 320, 271, 266 against 239, 233,
// 252, 248, 249; second derivatives float32 l_max = 4, 8, 12, 16, 20, 24 252, 262, 271, 258,
// 334, 361 against 231, 239, 238, 238, 245, 266; solid harmonics alike; values, whose entries
// are three multiplications, gain less: float32 l_max = 24, 32, 40 405, 383, 378 against 396,
// 377, 376, float64 l_max = 24, 28, 32 317, 322, 335 against 292, 305, 297. With few points
// (below 4 096) 512 threads stay: more workgroups have a tile then.
// SPHX_GROUP_THREADS = 512 or 1024 overrides the rule.
static unsigned group_threads(size_t n_samples, int mode, size_t elem, bool forward, bool normalized = true,
                              int l_max = -1) {
    // Second derivatives in float64: the entries (l, +m) and (l, -m) as one job need 169-237 registers per lane.
    // As two jobs, solid harmonics need 121, which sixteen waves allow (normalised 181: those keep eight waves).
    // 1.2 GB of output, us, 512 threads against 1024 with the two sides as two jobs in one list: l_max = 4, 5, 6, 8,
    // 10, 12, 14, 16, 18, 20, 22 251, 244, 247, 259, 253, 216, 225, 227, 220, 226, 231 against 201, 204, 205, 204,
    // 208, 211, 205, 215, 206, 221, 216; cfg4 538 against 507; l_max = 3 305 against 243. At l_max = 2 the list is
    // three jobs a point: 219 against 227.
    const bool solid_f64_hessians = mode == 2 && elem == 8 && !normalized;
    const bool exists = forward && (mode <= 1 || (mode == 2 && elem == 4) || solid_f64_hessians);
    if (!exists) return kRecursionThreads;
    const int want = switch_or(SW_GROUP_THREADS, 0);
    if (want == 512 || want == 1024) return static_cast<unsigned>(want);
    if (solid_f64_hessians && l_max < 3) return kRecursionThreads;
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
    // per point: the rows in every row buffer, point tables three times, iterates twice
    // staged rows are `row_stride` apart (recursion_kernel): nrow, or a little more when the rows
    // are cut so that they keep their position within 16 bytes
    const unsigned row_stride = nrow + (whole ? 0u : nyh % (16u / osize));
    const unsigned rows_per_point = components_of(mode) * row_stride;
    // (the records of a point and its sequences of iterates are an odd number of words apart)
    const unsigned rest_per_point = 3 * ((8 + 3 * (l_max + 1)) | 1u) + 2 * arrays * (tri_all | 1u);
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
    // (One row buffer. A second one, flushed by a wave of its own while the next tile is computed,
    // was built and measured: it once paid where a single buffer holds one or two points (second
    // derivatives l_max = 16, float64: 770 us against 810 us), but a wave that flushes alone waits
    // for its own LDS loads most of the time and the entry waves lose a wave and half the points
    // per tile. 400 MB of output, us, two buffers against one: second derivatives float32
    // l_max = 20, 22, 28 157, 122, 167 against 121, 100, 105 (solid 109, 96 against 88, 79);
    // float64 l_max = 20, 22 149, 134 against 126, 105. Its loop is no longer in the kernel,
    // which is 1-4 % faster without it.)
    if (bytes_for(1) > limit) return false;
    unsigned S = 1;
    if (bytes_for(1) <= budget) {
        // as many points as the budget holds, a power of two or not: fewer barrier rounds per
        // point (2 GB of output, gradients, float64 l_max = 13: 824 us with 4 points per tile,
        // 611 with 7; l_max = 14: 705 with 4, 602 with 6; float32 l_max = 21: 639 with 4, 603
        // with 6; second derivatives, float64 l_max = 12: 783 with 2, 547 with 3; never more
        // than 4 % slower than the power of two below)
        S = (budget - fixed) / point_bytes;
        if (switch_or(SW_TILE_POW2, 0) != 0) S = pow2_floor(S);
        if (S > 64) S = 64;
    }
    // Few points: with the largest tile there would be fewer tiles than workgroups that a launch
    // keeps resident. Then the tile is just large enough to give every one of them a tile (for
    // values and gradients four points at least: below that the closed forms of l <= 6 weigh
    // too much). 500 points, us: second derivatives float64 l_max = 6 16.1 -> 10.2, l_max = 16
    // 16.6 -> 12.6, float32 l_max = 12 17.5 -> 11.2; gradients float32 l_max = 20 23.9 -> 12.7.
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
            const unsigned extra = (2 * tiles - 3) * S * point_record * esize;
            if (bytes_for(S) + extra <= allowed || bytes_for(S) + extra <= budget) {
                az_shift = shift;
                break;
            }
        }
    }
    const unsigned table_slots = az_shift == 0 ? 3u : 2u << az_shift;

    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(S);
    g.az_shift = az_shift;
    // Waves of their own for the closed forms of l <= 6 (whole rows): with sixteen waves and
    // float32 gradients, where the tile otherwise waits for the entry waves that carry a slice on
    // top of their jobs; one of them up to eight points per tile, two from nine on, three from 28
    // on (l_max = 8, 9, 10, 12, 13 with two 224, 226, 226, 233, 244 us, with three 209, 216, 222,
    // 231, 241). 1.2 GB of
    // output, us, three sequence waves and the slices on all waves against two sequence waves and
    // one / two slice waves: l_max = 14, 18, 24, 28, 32, 36, 40 252, 253, 263, 256, 270, 270, 296
    // against 250, 241, 253, 248, 254, 260, 275 / 237, 237, 248, 254, 255, 262, 271. In float64 the
    // closed forms are too much for two or three waves (l_max = 16: 258 against 340 / 300 us).
    g.slice_waves = 0;
    const bool slices_apart = threads > kRecursionThreads && mode == 1 && elem == 4;
    if (whole && mode < 2) {
        const int want = switch_or(SW_SLICE_WAVES, slices_apart ? (S >= 28 ? 3 : (S >= 9 ? 2 : 1)) : 0);
        g.slice_waves = want < 0 ? 0u : (want > 4 ? 4u : static_cast<unsigned>(want));
    }
    g.sequence_waves = S * arrays * static_cast<unsigned>(l_max - hard) > 64 ? 2u : 1u;
    // Split the sides when that lets the entries of a tile go through the entry waves in fewer
    // rounds than it costs, a one-sided job being about 0.6 of a two-sided one. Normalised
    // float32 is the exception: always split, because the two-sided kernel needs 152 registers
    // per lane, so that only one workgroup fits on a CU, and the one-sided 116 (1.5 GB of
    // output, l_max = 5, 16 points per tile: 895 against 652 us; l_max = 10, 8 points: 826
    // against 598; l_max = 12, 4 points: 1 005 against 642; l_max = 15, 4 points: 780 against
    // 460). For solid harmonics in float32 both fit twice (119 and 88 registers) and the rule
    // holds (l_max = 10: 319 us by the rule, 404 always split; l_max = 12: 327 against 399);
    // float64 with the sides always split loses 10-20 % at most l_max.
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
        wide = threads - 64 * (1 + waves + g.slice_waves);
        // (with two or more points per tile the jobs go as a list ordered by kind, which fills the
        // lanes without splitting, and the two-sided job shares the common factors: 400 MB of
        // output, us, split against not, normalised float32 l_max = 4, 8, 16, 20 110, 115, 108,
        // 121 -> 104, 100, 96, 113; solid l_max = 6, 12 94, 92 -> 83, 83; with one point per tile
        // splitting stays, l_max = 24, 28 117, 104 against 184, 166)
        *split = may_split && S < 2 && one_side_costs * rounds(jobs_split) < 10 * rounds(jobs);
        // (float64 in workgroups of 1024 threads: only the one-sided job fits a lane's 128 registers)
        if (may_split && mode == 2 && elem == 8 && threads > kRecursionThreads) *split = true;
        return *split ? one_side_costs * rounds(jobs_split) : 10 * rounds(jobs);
    };
    // A second sequence wave takes a wave from the entries. One is enough where it saves the
    // entry waves a round per tile, and for values alone, whose recursions are a third of the
    // work (1.5 GB of output, one against two: gradients float32 l_max = 18, 19 437, 449 against
    // 545, 595 us; float64 l_max = 15, 16, 18 475, 423, 428 against 522, 460, 494; second
    // derivatives float32 l_max = 10, 13 496, 490 against 637, 637; values float32 l_max = 40,
    // 48 468, 428 against 527, 477; with equal rounds two are faster by 2-3 % with derivatives).
    // Second derivatives in float64 follow no such rule (l_max = 6, 8, 10: 555, 437, 505 against
    // 449, 558, 445) and keep two.
    if (threads > kRecursionThreads) {
        // Sixteen waves: the tile is larger, the recursions of a tile more, and the tile waits for
        // them if they need many rounds. Measured with two, three and four sequence waves (1.2 GB
        // of output, us): gradients float32 l_max = 12, 16, 20, 24, 28, 32 249, 257, 252, 265, 255,
        // 272 / 238, 245, 249, 259, 253, 267 / 244, 248, 264, 272, 269, 281: three. Float64
        // l_max = 9, 12, 16, 18, 20, 32 223, 244, 244, 248, 270, 251 / 218, 245, 240, 234, 252, 257 /
        // 239, 239, 233, 239, 257, 253: as few rounds of recursions as four waves would need, with
        // as few waves as that takes. Second derivatives, float32, l_max = 4, 8, 12, 16, 20, 24 240,
        // 239, 240, 238, 245, 276 / 231, 248, 247, 246, 250, 266: the entries weigh more there, two,
        // three at both ends.
        const unsigned recursions = S * arrays * static_cast<unsigned>(l_max - hard);
        if (mode == 1 && elem == 4) {
            g.sequence_waves = g.slice_waves != 0 ? 2 : 3; // (two with slice waves, see above)
        } else if (mode == 1) {
            const unsigned least = (recursions + 255u) / 256u;
            g.sequence_waves = 2;
            while (g.sequence_waves < 4 && (recursions + 64u * g.sequence_waves - 1u) / (64u * g.sequence_waves) > least) {
                ++g.sequence_waves;
            }
        } else if (mode == 2) {
            g.sequence_waves = l_max <= 4 || l_max >= 22 ? 3u : 2u;
        } else {
            // values, two against three: float32 l_max = 24, 28, 32, 40, 48 381, 436, 373, 420, 355
            // against 396, 392, 377, 376, 366; float64 l_max = 24, 28, 32 295, 326, 293 against
            // 292, 305, 297
            g.sequence_waves = 3;
        }
    } else if (g.sequence_waves == 2 && !(mode == 2 && elem == 8)) {
        bool split_one = false, split_two = false;
        const unsigned with_one = entry_cost(1, &split_one);
        const unsigned with_two = entry_cost(2, &split_two);
        if (mode == 0 || with_one < with_two) g.sequence_waves = 1;
    }
    {
        const int forced_seq = switch_or(SW_SEQUENCE_WAVES, 0);
        if (forced_seq >= 1 && forced_seq <= 4) g.sequence_waves = static_cast<unsigned>(forced_seq);
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
    // The jobs of a tile as one list. Values: the list is point after point and costs a few
    // instructions per job, so only where it saves a round and few points go side by side anyway
    // (float32 l_max = 40, 48: 527, 477 -> 468, 428 us). With derivatives the list is ordered by
    // kind of job first (recursion_kernel), which keeps the lanes of a wave on one branch of
    // entry_job: side by side, the 77 one-sided jobs of a point at l_max = 8 with second
    // derivatives put all seven kinds into every wave and 41 % of the lanes were active on
    // average. 400 MB of output, us, points side by side against the list: second derivatives
    // float32 l_max = 6, 8, 10, 12 (22, 14, 9, 6 points per tile) 164, 157, 138, 144 -> 115, 117,
    // 117, 115 (solid 108, 97, 97, 97 -> 98, 84, 89, 93); float64 l_max = 4, 8, 12, 16 146, 165,
    // 135, 123 -> 106, 104, 99, 96; gradients float32 l_max = 18, 24, 26 124, 123, 116 -> 109, 116,
    // 108, float64 l_max = 12, 13, 14 122, 127, 127 -> 107, 111, 115. With one or two points per
    // tile the list loses unless it saves a round (float32 gradients l_max = 32, 40: 113, 101 ->
    // 117, 119; l_max = 36, five rounds instead of six, 111 -> 108, solid 127 -> 112), and so it
    // does for solid second derivatives in float64 where the points side by side fill the lanes
    // anyway (cfg4, four points, 94 % of the lanes: 535 -> 559 us; l_max = 15, 83 %: 98 -> 84 us).
    // Second derivatives with two points per tile: the list unless the sides are split (float64
    // l_max = 20, 22 156, 138 -> 126, 105 us; solid float32 l_max = 22 83 -> 79; float32 with split
    // sides 100 -> 108).
    const int want_list = switch_or(SW_JOB_LIST, -1);
    const bool saves_a_round = (S * g.jobs_per_point + wide - 1) / wide < rounds_by_point(g.jobs_per_point);
    // lanes that points side by side would fill, in percent
    const unsigned fill = 100u * g.points_per_pass * g.jobs_per_point / wide;
    const bool cheap_jobs = mode == 2 && elem == 8 && !normalized; // no chain rule, few branches
    // (values in workgroups of 1024 threads: always the list, us per 1.2 GB without and with:
    // float32 l_max = 26 475, 391; float64 l_max = 26, 36 353, 307 and 351, 299; the same elsewhere)
    const bool by_shape = mode == 0   ? (threads > kRecursionThreads ? S >= 2 : saves_a_round && S >= 3 && g.points_per_pass <= 2)
                          : mode == 1 ? S >= 3 || (saves_a_round && S >= 2)
                                      : (S >= 3 && !(cheap_jobs && fill >= 90u)) || (S == 2 && !*split_sides) ||
                                            (saves_a_round && S >= 2) ||
                                            (cheap_jobs && threads > kRecursionThreads && S >= 2);
    if (want_list == 2 || (want_list == 1 && saves_a_round) || (want_list < 0 && by_shape)) {
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
    at += 2 * S * arrays * (tri_all | 1u);
    g.off_jobs = at;
    at += table_elems_for(may_split);
    out->lds_bytes = g.tables_at + at * esize;
    out->threads = threads;
    if (out->lds_bytes > limit) return false;
    // Jobs point by point, one point per pass, with derivatives: in the last round of a point the
    // jobs with |m| = l, |m| = l - 1 and m = 0 are moved to wave boundaries of the entry lanes where
    // the lanes of that round allow it, because a wave runs the branch of every kind of job it
    // holds one after the other and the tile waits for the slowest wave. Float32 l_max = 32, 533
    // jobs on 320 lanes: the second round was 135 bulk jobs, then 26 + 26 + 26, all three in the
    // third wave together with the end of the bulk; moved, m = 0 follows the bulk and the other two
    // start the fourth and fifth wave. The gaps are places without a job at the end of the job
    // table. With one workgroup of 1024 threads on a CU this pays (float64 gradients l_max = 32,
    // two points per tile: 290 -> 249 us per 1.2 GB). With two workgroups of 512 the slowest wave of
    // a tile of cfg5 went from 7 400 to 5 900 cycles and a launch from 979 to 926 us for the first
    // few launches after a pause, but from 896 to 947 us in a long series of launches, and builds
    // of the kernel that differ in a few scalar instructions moved either number by 5 %: how the
    // stages and flushes of the two workgroups of a CU fall against each other decides there,
    // and nothing in the kernel controls that. Off for 512 threads (SPHX_SPREAD_KINDS).
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
    // Chunks of consecutive tiles per workgroup: only where a tile is one run per array, and a
    // run is at least a line long (so that a carried part never spans two tiles). About eight
    // points per chunk: chunks of eight tiles whatever their size were as good for tiles of one
    // or two points and worse for larger ones (second derivatives, float64, 1.5 GB of output:
    // l_max = 16, 4 points per tile, 446 us in chunks of eight tiles, 394 in chunks of two;
    // l_max = 8, 14 points, 632 against 561 for single tiles; cfg4 562 against 528).
    g.chunk_shift = 0;
    if (whole && S * nrow * osize >= 128u) {
        const int want = switch_or(SW_CHUNK_SHIFT, S >= 5 ? 0 : (S >= 3 ? 1 : (S == 2 ? 2 : 3)));
        g.chunk_shift = want < 0 ? 0u : (want > 10 ? 10u : static_cast<unsigned>(want));
    }
    unsigned per_cu = limit / out->lds_bytes;
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 2048u / threads) per_cu = 2048u / threads; // 2048 lanes per CU
    unsigned want = (static_cast<unsigned>(cus) * per_cu + 7u) & ~7u;
    // Few points: shorter chunks, down to single tiles, until every resident workgroup has one
    // (10 000 points at l_max = 8 are 625 tiles of 16: in chunks of 8 they kept 80 workgroups
    // busy for 41 us, as single tiles they take 512 and a third of the time).
    auto chunks_in_xcd = [&]() { return (g.tiles_per_xcd + (1u << g.chunk_shift) - 1u) >> g.chunk_shift; };
    while (g.chunk_shift > 0 && chunks_in_xcd() * 8u < want) --g.chunk_shift;
    const unsigned chunks_per_xcd = chunks_in_xcd();
    unsigned need = chunks_per_xcd * 8u;
    out->workgroups = want < need ? want : need;
    if (out->workgroups < 8) out->workgroups = 8;
    return true;
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
    // Gradients in closed form, where the rows of a tile are so long that few single-wave
    // workgroups of closed_form_kernel share a CU: the lanes kernel instead, which cuts the closed
    // forms in slices for six or eight waves and flushes with all of them. Measured, us, against
    // closed_form_kernel: l_max = 6 float32 1M points 127 against 134 (solid 133 against 134), 300k
    // 43 against 49, 100k 17 against 23, 10k 5.0 against 6.8; float64 500k 125 against 148 (solid
    // 131 against 152), 100k 29 against 42; l_max = 5 float64 680k 135 against 149; l_max = 4
    // float32 2M 131 against 141, 100k 8.7 against 11.3. Not below: l_max = 3 float32 100k 8.0
    // against 7.3, l_max = 4 float64 1M 139 against 132, l_max = 5 float32 140 against 142.
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
    // the recursions of the next tile and the flush of this one side by side. 1.2 GB of output, us, against
    // values_kernel (the recursion kernel from l_max = 34): float32 l_max = 22, 24, 26, 28, 30, 32, 34, 36 262,
    // 254, 242, 252, 231, 219, 236, 243 against 262, 296, 293, 319, 318, 306, 379, 381; float64 l_max = 20, 24,
    // 28, 32, 36 220, 222, 224, 215, 223 against 266, 301, 312, 298, 303; below (float32 l_max = 20 264 against
    // 257, float64 l_max = 18 293 against 247) a point's pairs leave the entry lanes idle.
    if (lane_kernels && mode == 0 && l_max > hard) {
        const int pairs = switch_or(SW_PAIRS, 1);
        const bool pairs_by_shape = n_samples >= 32768 && (elem == 4 ? l_max >= 23 : l_max >= 20);
        if (pairs == 2 || (pairs == 1 && pairs_by_shape)) {
            PairsChoice want;
            want.tile = static_cast<unsigned>(switch_or(SW_PAIRS_TILE, 0));
            want.batch_tiles = static_cast<unsigned>(switch_or(SW_PAIRS_BATCH, 0));
            want.prep_waves = static_cast<unsigned>(switch_or(SW_PAIRS_PREP_WAVES, 0));
            want.sequence_waves = static_cast<unsigned>(switch_or(SW_PAIRS_SEQUENCE_WAVES, 0));
            want.chunk_shift_plus_one = static_cast<unsigned>(switch_or(SW_PAIRS_CHUNK, -1) + 1);
            if (plan_pairs(n_samples, l_max, mode, elem, elem, lds_limit, cus, want, &plan->pairs_launch)) {
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
    // (Since the recursion kernel takes its jobs as a list ordered by kind it wins from l_max = 4
    // on; 400 MB of output, us, lanes against recursion: float32 l_max = 2 87, 99 (solid 72, 82),
    // l_max = 3 104, 108 (solid 89, 100), l_max = 4 147, 107 (solid 113, 87), l_max = 5 130, 112
    // (solid 99, 86); float64 l_max = 3 129, 114 (solid 91, 102), l_max = 5 163, 107; 20 000 points
    // float32 l_max = 3 9.0, 11.2, l_max = 4 17.9, 13.5.)
    // (Solid harmonics in float64, l_max = 3, 1.2 GB of output: 259 us against 243 in workgroups of 1024 threads.)
    const bool hessian_lanes_pay = elem == 4 ? l_max <= 3 : (l_max == 3 && !normalized && n_samples < 32768);
    if (lane_kernels && mode == 2 && (hessian_lanes == 2 || (hessian_lanes == 1 && hessian_lanes_pay)) &&
        plan_hessian_lanes(n_samples, l_max, elem, lds_limit, &plan->closed, normalized)) {
        plan->lanes = true;
        return SPHX_OK;
    }
    // (float32 from l_max = 14 on the recursion kernel with its jobs as a list ordered by kind is
    // ahead: 600 MB of output, lanes against recursion, l_max = 13 151, 150 us; 14 169, 153; 15 189,
    // 171; 16 174, 154; solid 14 152, 144; 16 160, 144. SPHX_GRADIENT_LANES=2: lanes wherever they fit.)
    // (With workgroups of 1024 threads the recursion kernel is ahead earlier when there are points
    // enough for them: 1.2 GB of output, us, lanes against recursion, float32 l_max = 8 214, 206; 9
    // 256, 217; 10 241, 227; 11 256, 286; 12 306, 238; 13 301, 246; float64 l_max = 7 224, 507; 8
    // 246, 214; 9 307, 218; 10 293, 226; 11 309, 292. The lanes keep l_max <= 8 and 11 in float32,
    // l_max = 7 in float64, and every call of fewer than 32 768 points (50 000 points, lanes against
    // recursion: float64 l_max = 9 54, 43 us, float32 l_max = 12 42, 38 us; 20 000 points 25, 22 and 21, 24).)
    // Derivatives where the rows of few points fill LDS: pairs_kernel, whose entry lanes keep one (l, m) pair for
    // the whole launch and whose other work runs while the rows are flushed. 1.2 GB of output, us, pairs_kernel
    // against recursion_kernel. Gradients: float32 l_max = 16, 20, 24, 28, 32, 36 299, 274, 267, 269, 253, 262
    // against 289, 286, 291, 288, 285, 286; float64 l_max = 14, 16, 20, 24, 28, 32, 36 289, 280, 265, 251, 268, 268,
    // 248 against 283, 289, 288, 290, 285, 285, 274; cfg5 (l_max = 32, 200 000 points) 570-620 against 700. Below,
    // a point's pairs leave most of the entry lanes idle and it loses (float32 l_max = 12: 383 against 277).
    // Second derivatives: float64 l_max = 12, 16, 20, 24 287, 299, 296, 318 against 290, 290, 333, 352; float32
    // l_max = 12, 16, 20, 24 350, 303, 318, 307 against 289, 285, 294, 304 (the recursion kernel's job list by
    // kind fills sixteen waves better). SPHX_PAIRS: 0 never, 2 wherever it fits.
    {
        const int pairs = switch_or(SW_PAIRS, 1);
        const bool pairs_by_shape = n_samples >= 32768 && (mode == 1 ? (elem == 4 ? l_max >= 20 : l_max >= 16)
                                                                     : (elem == 8 && l_max >= 20));
        if (lane_kernels && mode >= 1 && l_max > hard && (pairs == 2 || (pairs == 1 && pairs_by_shape))) {
            PairsChoice want;
            want.tile = static_cast<unsigned>(switch_or(SW_PAIRS_TILE, 0));
            want.batch_tiles = static_cast<unsigned>(switch_or(SW_PAIRS_BATCH, 0));
            want.prep_waves = static_cast<unsigned>(switch_or(SW_PAIRS_PREP_WAVES, 0));
            want.sequence_waves = static_cast<unsigned>(switch_or(SW_PAIRS_SEQUENCE_WAVES, 0));
            want.chunk_shift_plus_one = static_cast<unsigned>(switch_or(SW_PAIRS_CHUNK, -1) + 1);
            if (plan_pairs(n_samples, l_max, mode, elem, elem, lds_limit, cus, want, &plan->pairs_launch)) {
                plan->pairs = true;
                return SPHX_OK;
            }
        }
    }
    const int gradient_lanes = switch_or(SW_GRADIENT_LANES, 1);
    const bool large_groups = group_threads(n_samples, mode, elem, lane_kernels) > kRecursionThreads && n_samples >= 32768;
    const bool lanes_by_shape = large_groups ? (elem == 4 ? l_max <= 8 || l_max == 11 : l_max <= 7)
                                             : elem == 8 || l_max <= 13;
    if (lane_kernels && mode == 1 && gradient_lanes != 0 && (gradient_lanes == 2 || lanes_by_shape) &&
        plan_gradient_lanes(n_samples, l_max, elem, lds_limit, cus, &plan->closed)) {
        plan->lanes = true;
        return SPHX_OK;
    }
    // LDS a workgroup of the recursion kernel may take: half a CU's, so that two share the CU.
    // With second derivatives in float64 the kernel needs more than 128 registers per lane,
    // one workgroup of 512 threads is all a CU holds, and half of LDS would lie idle: there
    // the tile takes all of it (1.5 GB of output, l_max = 6: 694 -> 473 us, l_max = 10: 582 ->
    // 479, l_max = 12: 545 -> 468; solid harmonics l_max = 4-12: 10-20 % less, l_max = 16, 100k
    // points: 580 -> 560).
    const unsigned threads = group_threads(n_samples, mode, elem, lane_kernels, normalized, l_max);
    const int whole_cu = (mode == 2 && elem == 8) || threads > kRecursionThreads ? lds_limit : 80 * 1024;
    const unsigned budget = static_cast<unsigned>(switch_or(SW_TILE_LDS_BUDGET, whole_cu));
    bool fits = plan_recursion(n_samples, l_max, mode, true, elem, budget, lds_limit, cus, &plan->rec,
                               &plan->split_sides, normalized, 0, threads);
    // With few points per tile the one-lane-per-point closed forms of l <= 6 would leave most of
    // the lanes idle for some two thousand instructions per tile: then the recursion kernel
    // stages l >= 7 only and its wave 0, which mostly waits, writes l <= 6 straight from
    // registers, 64 points at a time (prefix_inside). The price is rows cut in two, each part a
    // run of its own in HBM, which costs the more the shorter the rows are. Measured with 2.5 GB
    // of output and 400 calls in a row (in bursts of 60 calls, or with a few hundred MB of
    // output, the last-level cache merges the parts and the cut rows look 10-30 % better than
    // they are), whole against cut, us. Gradients, float32: l_max = 17 (8 points per tile) 764
    // against 1 014; l_max = 19, 20, 22 (4) 1 196, 1 121, 922 against 992, 988, 817; l_max = 24
    // (4) 707 against 741; l_max = 28, 32 (2) 881, 781 against 883, 636. Gradients, float64:
    // l_max = 12 (8) 737 against 1 084; l_max = 13, 14, 16, 18 (4) 1 029, 878, 775, 812 against
    // 1 049, 1 059, 918, 848; l_max = 20, 24 (2) 995, 706 against 886, 626. Values: float32
    // l_max = 36, 40 (4) 1 004, 977 against 885, 865; float64 l_max = 24, 28 (4) 924, 856
    // against 741, 749.
    // (With the job-list variant of the kernel the whole rows gained more than the cut ones:
    // float32 gradients, 1.5 GB of output, whole against cut: l_max = 19-22 (5-7 points per tile)
    // 393, 407, 373, 399 us against 431, 451, 419, 424; l_max = 28, 30 (3) 396, 371 against 532,
    // 510; l_max = 32 (2) 462 against 389. Float32 gradients are therefore cut below three
    // points per tile only; values below eight, float64 gradients below four as before.)
    // (Since the float64 rows go out in whole lines, copy_out<LINES>, the cut rows gained 20 %
    // there: l_max = 20, 100k points 491 -> 376 us, and with four points per tile they now win as
    // well, l_max = 18: 291 us cut against 328 whole; with five, l_max = 16: 580 against 481.)
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
        const unsigned wide = plan->rec.threads - 64 * (1 + g.sequence_waves + g.slice_waves);
        plan->rec.g.points_per_pass = g.jobs_per_point >= wide ? 1u : wide / g.jobs_per_point;
    }
    if (!fits) {
        return fail(SPHX_ERR_UNSUPPORTED,
                    "l_max = " + std::to_string(l_max) +
                        " with this many derivatives needs more LDS for the rows of one point than "
                        "the device offers (" + std::to_string(lds_limit) + " bytes)");
    }
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
        // groups of lanes with channels of their own pay off from tiles of 16 points down
        // (200k points, float32 l_max = 24: 225 against 279 us; float64 l_max = 24: 665
        // against 866; with tiles of 32 the scalar-unit kernel is ahead, float64 l_max = 12:
        // 329 against 397)
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
               std::to_string(l.workgroups) + " workgroups]";
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
                (plan.rec.g.points_per_pass == 0 ? "true" : "false") + ">" + geometry(plan.rec);
    }
    return text;
}

} // namespace sphx

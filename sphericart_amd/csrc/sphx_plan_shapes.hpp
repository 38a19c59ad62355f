// The planner's choices that go by the shape of a call and not by a rule: which of several forms of a kernel is
// fastest changes from one l_max to the next (row lengths, channels per wave and workgroups per CU all change
// with it), so the measured winner is written down here, one row per range of l_max, next to the figures of
// the sweep that decided it. Everything else in sphx_plan.cpp follows from LDS sizes and lane counts.
// Plain C++.
#ifndef SPHX_PLAN_SHAPES_HPP
#define SPHX_PLAN_SHAPES_HPP

namespace sphx {

// values_kernel (kind 0) and the lane kernels of the fused product (kind 1) on an MI355X.
//   pack    values: channels a wave evaluates side by side (1, 2, 4); tiles of 64 / pack points
//   alone   one workgroup per CU with all of its LDS instead of two with half each
//   waves   the product, alone on its CU: waves of the workgroup (0: as many as there are channels)
//   floor   the product: tiles shrink in steps of four points down to this size and halve from there
struct ShapeRow {
    int kind, elem, l_from, l_to;
    unsigned pack;
    bool alone;
    int waves;
    unsigned floor;
    const char* measured;
};

constexpr ShapeRow kShapeRows[] = {
    // values, float32. 1 GB of values, us, in the order: tile that fits half of LDS / one workgroup with all of
    // LDS / two channels in half of LDS / the same with all of LDS / four channels / recursion kernel
    {0, 4, 21, 21, 2, false, 0, 32, "254 262 248 252 268 397"},
    {0, 4, 22, 22, 2, false, 0, 32, "271 260 238 239 260 389"},
    {0, 4, 23, 23, 1, true, 0, 32, "319 288 - 427 341 425"},
    {0, 4, 25, 25, 4, false, 0, 32, "319 295 - 366 286 397"},
    {0, 4, 26, 26, 4, false, 0, 32, "317 300 - 350 275 393"},
    {0, 4, 29, 29, 2, false, 0, 32, "- 329 - 326 342 389"},
    {0, 4, 30, 30, 2, false, 0, 32, "- 357 - 317 332 391"},
    {0, 4, 31, 31, 2, false, 0, 32, "- 360 - 324 348 389"},
    {0, 4, 32, 32, 2, false, 0, 32, "- 368 - 300 313 378"},
    {0, 4, 33, 33, 2, false, 0, 32, "- 365 - 297 305 386"},
    // values, float64, the same columns
    {0, 8, 14, 14, 1, true, 0, 32, "224 212 - 239 309 310"},
    {0, 8, 15, 15, 1, true, 0, 32, "258 225 - 257 326 347"},
    // the product, float64. 200 000 points (400 000 to l_max = 16), us: tiles in half of LDS / one workgroup per
    // CU with 8 / with up to 12 waves; from l_max = 21 with tiles of 28, 24, 20 points before they halve
    {1, 8, 14, 14, 1, true, 12, 32, "498 287 286"},
    {1, 8, 15, 15, 1, true, 12, 32, "519 328 324"},
    {1, 8, 16, 16, 1, true, 12, 32, "538 383 360"},
    {1, 8, 17, 17, 1, true, 12, 32, "289 228 214"},
    {1, 8, 18, 18, 1, true, 12, 32, "299 261 240"},
    {1, 8, 19, 19, 1, true, 12, 32, "315 290 272"},
    {1, 8, 20, 20, 1, true, 12, 32, "330 336 316"},
    {1, 8, 21, 21, 1, true, 12, 16, "588 375 364"},
    {1, 8, 22, 22, 1, true, 12, 16, "613 444 405"},
    {1, 8, 23, 23, 1, true, 12, 16, "627 468 464"},
    {1, 8, 24, 24, 1, true, 12, 16, "640 565 564"},
    {1, 8, 25, 25, 1, true, 8, 16, "660 598 602"},
    {1, 8, 26, 26, 1, true, 12, 16, "675 719 661"},
    // the product, float32, the same columns (l_max = 21, 31: sixteen waves 162, 423)
    {1, 4, 19, 19, 1, true, 12, 32, "144 153 135"},
    {1, 4, 21, 21, 1, true, 16, 32, "181 178 172"},
    {1, 4, 22, 22, 1, true, 8, 32, "211 168 185"},
    {1, 4, 23, 23, 1, true, 12, 32, "216 212 201"},
    {1, 4, 25, 25, 1, true, 12, 32, "335 274 255"},
    {1, 4, 26, 26, 1, true, 12, 32, "340 294 276"},
    {1, 4, 27, 27, 1, true, 8, 32, "348 289 313"},
    {1, 4, 28, 28, 1, true, 8, 32, "356 318 342"},
    {1, 4, 29, 29, 1, true, 12, 32, "385 404 370"},
    {1, 4, 30, 30, 1, true, 8, 32, "397 381 422"},
    {1, 4, 31, 31, 1, true, 16, 32, "477 436 442"},
    {1, 4, 32, 32, 1, true, 8, 32, "500 470 645"},
    {1, 4, 35, 35, 1, true, 12, 16, "789 692 642"},
    {1, 4, 36, 36, 1, true, 12, 16, "807 678 667"},
    {1, 4, 37, 37, 1, true, 8, 16, "820 718 792"},
    {1, 4, 38, 40, 1, true, 8, 32, "874 852 851 (l_max = 40)"},
    {1, 4, 43, 43, 1, true, 8, 16, "909 866 868"},
};

// The row for a shape, or nullptr: then one channel per wave, two workgroups per CU where they fit.
inline const ShapeRow* shape_row(int kind, int elem, int l_max) {
    for (const ShapeRow& row : kShapeRows) {
        if (row.kind == kind && row.elem == elem && l_max >= row.l_from && l_max <= row.l_to) return &row;
    }
    return nullptr;
}

// recursion_kernel and pairs_kernel: the shapes at which the waves that flush a tile run at raised priority
// (s_setprio) while other waves prepare the next tile. The flush and the preparation end at the same barrier;
// whichever of them a tile waits for gains or loses by it, and which one that is changes from one l_max to the
// next with the tile and the rounds of the sequence lanes. Measured at 1.2 GB of output after 0.3 s of the same
// launches (settled clocks; `python -m sphericart_amd.tune` is the measurement), on two boxes: percent gained on either
// box (the same sign on both at nearly every l_max, and the same in short bursts on two other boxes; the rows are
// the shapes that gained 3 % or more on both, elsewhere the priority costs up to 10 %). The gain holds from
// 50 000 points up in pairs_kernel (2 to 13 % at 50 000, 100 000, 200 000 and 400 000 points) and from 50 000
// down to 20 000 in recursion_kernel (1 to 11 %); the planner asks for 32 and 4 tiles per workgroup. Whether the
// priority is 1, 2 or 3 makes no difference.
struct PriorityRow {
    int mode, elem;
    bool normalized;
    int l_from, l_to;
    unsigned priorities;     // 1: the flushing waves at raised priority
    unsigned sequence_waves; // recursion_kernel: this many instead of the planner's rule (0: the rule)
    const char* measured;
};

constexpr PriorityRow kFlushPriorityRows[] = {
    // gradients, float32
    {1, 4, true, 31, 31, 1, 0, "+4 / +8 (l_max = 32, cfg5: between -3 and +6 from run to run at 50 000 to 800 000 points, left alone)"},
    {1, 4, true, 34, 35, 1, 0, "+8 / +8, +14 / +14"},
    {1, 4, false, 11, 14, 1, 0, "+10 / +8, +7 / +7, +5 / +5, +6 / +5"},
    {1, 4, false, 16, 16, 1, 0, "+5 / +5"},
    {1, 4, false, 23, 23, 1, 0, "+5 / +6"},
    {1, 4, false, 29, 29, 1, 0, "+12 / +10"},
    {1, 4, false, 33, 34, 1, 0, "+14 / +12, +10 / +9"},
    // gradients, float64
    {1, 8, true, 23, 24, 1, 0, "+5 / +7, +8 / +5"},
    {1, 8, true, 31, 32, 1, 0, "+7 / +6, +9 / +10"},
    {1, 8, false, 19, 19, 1, 0, "+11 / +11"},
    {1, 8, false, 21, 21, 1, 0, "+13 / +12"},
    {1, 8, false, 25, 25, 1, 0, "+8 / +8"},
    {1, 8, false, 30, 31, 1, 0, "+12 / +14, +6 / +4"},
    // second derivatives, float32, solid (normalised: 0 to +3 at l_max = 5-28 on both boxes, -1 to -2 on a third)
    {2, 4, false, 5, 6, 1, 0, "+13 / +13, +11 / +12"},
    {2, 4, false, 8, 8, 1, 0, "+11 / +9"},
    {2, 4, false, 10, 14, 1, 0, "+14 / +14, +10 / +12, +10 / +8, +4 / +3, +7 / +6"},
    {2, 4, false, 27, 28, 1, 0, "+6 / +5, +12 / +12"},
    // second derivatives, float64, solid
    {2, 8, false, 19, 19, 1, 0, "+5 / +5"},
    {2, 8, false, 22, 22, 1, 0, "+5 / +5"},
    {2, 8, false, 24, 24, 1, 0, "+6 / +5"},
    // With another number of sequence waves than the rule's (four for gradients in float32, three in float64, three or
    // two for solid second derivatives in float32). Every setting measured after 0.4 s of its own launches, median
    // of three turns, us per 1.2 GB: the rule without priority / this row, on one box, then on another.
    {1, 4, false, 8, 8, 1, 3, "221 / 197, 222 / 195"},
    {1, 4, false, 9, 9, 0, 2, "221 / 205, 222 / 205"},
    {1, 4, false, 10, 10, 1, 3, "230 / 202, 231 / 200"},
    {1, 8, false, 11, 11, 1, 4, "211 / 204, 210 / 203"},
    {1, 8, false, 13, 13, 1, 4, "217 / 209, 216 / 207"},
    {1, 8, false, 15, 16, 1, 4, "218 / 208 and 220 / 212, 216 / 205 and 219 / 213"},
    {2, 4, false, 4, 4, 0, 8, "215 / 199, 217 / 199"},
    {2, 4, false, 18, 19, 1, 4, "214 / 206 and 216 / 207, 211 / 205 and 215 / 206"},
    {2, 4, false, 21, 21, 1, 4, "219 / 207, 218 / 206"},
    {2, 8, false, 23, 23, 1, 2, "240 / 217, 239 / 218 (the rule: three)"},
    // pairs_kernel with gradients, where the planner's estimate gives four sequence waves in float32 and two or three in
    // float64: the rule with the priority where a row above had it / this row; one turn, then the median of three
    {1, 4, false, 30, 30, 0, 3, "223 / 214, 223 / 211"},
    {1, 4, false, 31, 31, 0, 3, "233 / 205, 233 / 204"},
    {1, 4, false, 32, 32, 1, 3, "220 / 204, 217 / 205"},
    {1, 4, false, 35, 35, 0, 3, "240 / 210, 241 / 211"},
    {1, 8, false, 20, 20, 1, 2, "225 / 204, 225 / 204"},
    {1, 8, false, 23, 23, 1, 2, "239 / 221, 237 / 225"},
    {1, 8, false, 26, 27, 1, 4, "228 / 205 and 239 / 230, 229 / 206 and 240 / 231"},
    {1, 8, false, 28, 29, 1, 2, "227 / 208 and 244 / 225, 227 / 208 and 244 / 228"},
};

inline const PriorityRow* priority_row(int mode, int elem, bool normalized, int l_max) {
    for (const PriorityRow& row : kFlushPriorityRows) {
        if (row.mode == mode && row.elem == elem && row.normalized == normalized && l_max >= row.l_from &&
            l_max <= row.l_to) {
            return &row;
        }
    }
    return nullptr;
}

} // namespace sphx

#endif

// Arguments of the decode / verify-window launches, as the launchers resolve them from the C ABI's parameters.
#pragma once
#include <type_traits>

#include "pkv_common.hpp"

namespace pkv {

struct AttendArgs {
    const uint8_t* q;
    const uint8_t* kp;
    const uint8_t* vp;
    const float* ks;
    const float* vs;
    const float* hm;
    const int32_t* tables;
    const int32_t* rows;
    const int32_t* starts;
    const int32_t* counts;
    const int64_t* firsts;
    const int32_t* offsets;
    float* po;
    float* pm;
    float* pl;
    void* out;
    float* lse;
    const float* sinks;
    unsigned* ticket;      // two zeroed counters of the unit-pulling launches: next unit, workgroups done
    int64_t q_st, q_sh, o_st, o_sh, tab_stride;
    int tab_width, n_rows, columns, hq, hkv, g, page, page_shift, parts, piece, sliding, out_dtype, tiles, max_keys, heads_per_wave, units_x, units_y;
    float sscale, k_mult, v_mult;
};

}   // namespace pkv

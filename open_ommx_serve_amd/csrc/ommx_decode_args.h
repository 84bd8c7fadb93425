// Argument block and small helpers shared by the decode kernels.
#pragma once
#include "ommx_common.h"

namespace ommx {

struct DecodeArgs {
    const uint16_t* q; int64_t q_sb, q_sh;
    const uint8_t* k_base; const int8_t* k_scale; const uint16_t* k_zp;
    const uint16_t* k_ms; const uint16_t* k_mc;
    const uint8_t* k_obmp;           // index plane: 4-byte bitmaps, or 7-bit position streams (idx_repr 1)
    const uint8_t* k_oval;
    const uint8_t* v_main; const int8_t* v_scale; const uint16_t* v_zp;
    const void* rt; int64_t rt_s; const void* rg; int64_t rg_s; int i64;
    const int32_t* seq;
    float* al; int64_t al_b, al_h, al_s;
    int B, Hq, Hkv, ps, kout, S;
    float sm_scale, cap;
    int off, gbase;
    int idx_repr;                    // 0 flat bitmap, 1 relidx7
    int scale_bf16;                  // k_scale / v_scale hold bf16 steps instead of int8 exponents
    int gt, gc;                      // tokens per K group, channels per V vector (16, 32, 64 or 128)
    int v_bf16;                      // v_main holds bf16 rows [P,ps,H,D] instead of INT2 codes
    // Extents of the planes the tables index: a page id outside [0, n_pages) or a group slot outside
    // [0, n_gslots) is clamped into range (no access leaves the planes) and OMMX_ERR_TABLE_RANGE is
    // OR-ed into *err (may be NULL).  0 = extent not given: ids are used as they are.
    int n_pages, n_gslots;
    int32_t* err;
    // set by the launcher of the serving-recipe kernel only: head_dim is 64 and Hkv counts PAIRS of kv
    // heads (the planes of two neighbouring 64-channel heads read like one 128-channel head)
    int half;
};

// 7-bit position streams (pack.py:128-164): position s of a frame at bits [7s, 7s+7)
__host__ __device__ constexpr int relidx7_bytes(int k) { return (7 * k + 7) / 8; }

__device__ __forceinline__ int64_t table_at(const void* t, int64_t i, int i64) {
    return i64 ? static_cast<const int64_t*>(t)[i] : static_cast<const int32_t*>(t)[i];
}

// Page id / group slot as read from a table, held inside the plane; `bad` collects whether any was not.
__host__ __device__ __forceinline__ int clamp_id(int id, int n, bool& bad) {
    if (n > 0) {
        const uint32_t u = static_cast<uint32_t>(id), top = static_cast<uint32_t>(n - 1);
        bad |= u > top;                       // negative ids are huge as unsigned: one comparison
        id = static_cast<int>(u < top ? u : top);
    }
    return id;
}
__device__ __forceinline__ void report_table_range(int32_t* err, bool bad) {
    if (__any(bad) && err && (threadIdx.x & 63) == 0) atomicOr(err, OMMX_ERR_TABLE_RANGE);
}

__device__ __forceinline__ float apply_cap(float x, float cap) {
    // cap * tanh(x / cap) written as the reference does: cap * (2*sigmoid(2x/cap) - 1)
    if (cap > 0.0f) x = cap * (2.0f / (1.0f + __expf(-2.0f * x / cap)) - 1.0f);
    return x;
}


struct CombineArgs {
    const float* al; int64_t al_b, al_h, al_s;
    const uint16_t* q; int64_t q_sb, q_sh;
    const uint16_t* kt; const uint16_t* vt;
    int64_t kt_b, kt_t, kt_h, vt_b, vt_t, vt_h;
    const int32_t* tail; const int32_t* seq;
    float* o; int64_t o_b, o_h;
    float* lse; int64_t lse_b;
    int B, Hq, Hkv, S;
    float sm_scale, cap;
    int gt;                          // tokens per K group: the splits are rounded to it
    int T;                           // rows every request's tail buffer holds (0: not told): rows below it
                                     // may be read before b_tail_len has arrived
};

int launch_decode_ref(const DecodeArgs& a, int D, int R, hipStream_t st);
int launch_combine(const CombineArgs& a, int D, hipStream_t st);

}  // namespace ommx

// Argument block and arithmetic helpers shared by the store kernels (tuned 32x32 recipe kernel
// and the kernel for every other group size).  Every fp32 operation is a single IEEE rounding
// in the reference packer's order; the including files are compiled with -ffp-contract=off.
#pragma once
#include "ommx_common.h"

namespace ommx {

struct StoreArgs {
    const void* K;
    const void* V;
    int64_t k_ts, k_hs, v_ts, v_hs;
    const int32_t* src_rows;
    const int32_t* dst_pages;
    const int32_t* dst_groups;
    const float* table;
    uint8_t* k_base;
    int8_t* k_scale;
    uint16_t* k_zp;
    uint16_t* k_ms;
    uint16_t* k_mc;
    uint8_t* k_obmp;        // index plane: bitmaps [G,H,D,4], or 7-bit streams [G,H,D,ceil(7k/8)]
    uint8_t* k_oval;
    uint8_t* v_main;
    int8_t* v_scale;
    uint16_t* v_zp;
    int32_t* err;
    int H, D, ps, kout;
    int v_vec;              // V rows allow 16-byte loads
    int idx_repr;           // 0 flat bitmap (codec.py:330-372), 1 relidx7 (pack.py:128-164)
    int select_abs;         // 0 signed top + bottom tails (pack.py:436-445), 1 largest |w| (pack.py:446-448)
    int scale_mode;         // 0 power of two, int8 exponent plane; 1 power of two, bf16 plane;
                            // 2 bf16((max - min) / 3) as it comes, bf16 plane (pack.py:459-463, 586-590)
    int gt, gc;             // tokens per K vector, channels per V vector (32 and 32 in the tuned kernel)
    int v_bf16;             // V is kept as bf16 rows [pages, ps, H, D]; v_scale = 1, v_zp = 0 (pack.py:596-602)
};


template <bool F32>
__device__ __forceinline__ float load_elem(const void* base, int64_t idx) {
    if (F32) return static_cast<const float*>(base)[idx];
    return bf16_to_f32(static_cast<const uint16_t*>(base)[idx]);
}

// rint(log2(x)) for x >= 1e-12 through the threshold table: the exponent of x's binade,
// plus one when x has reached that binade's rounding point.
__device__ __forceinline__ int pow2_round_exp(float x, const float* __restrict__ table) {
    const uint32_t kb = (__float_as_uint(x) >> 23) & 0xFFu;
    return static_cast<int>(kb) - 127 + (x >= table[kb] ? 1 : 0);
}

__device__ __forceinline__ float exp2_int(int e) {   // exact 2^e, e in [-126,127]
    return __uint_as_float(static_cast<uint32_t>(e + 127) << 23);
}

// FP4 code of m: sign bit and the number of magnitude thresholds fthr[1..7] (ascending) that |m| has
// reached.
__device__ __forceinline__ uint32_t fp4_encode(float m, const float* __restrict__ fthr) {
    const float a = fabsf(m);
    uint32_t idx = 0;
#pragma unroll
    for (int j = 1; j <= 7; ++j) idx += (a >= fthr[j]) ? 1u : 0u;
    return ((m < 0.0f) ? 8u : 0u) | idx;
}
// The same with the seven thresholds in (scalar) registers t[1..7]: three compares down the sorted
// thresholds instead of seven.
__device__ __forceinline__ uint32_t fp4_encode_sorted(float m, const float (&t)[8]) {
    const float a = fabsf(m);
    const bool c4 = a >= t[4];
    const bool c2 = a >= (c4 ? t[6] : t[2]);
    const float lo = c4 ? t[5] : t[1], hi = c4 ? t[7] : t[3];
    const bool c1 = a >= (c2 ? hi : lo);
    return ((m < 0.0f) ? 8u : 0u) | (c4 ? 4u : 0u) | (c2 ? 2u : 0u) | (c1 ? 1u : 0u);
}

// x / 2^e is computed as x * 2^-e: 2^-e is exact for e in [-126,126], the product and the
// quotient are then the same real number, so they round alike, denormal results included.
// The quantisation step of one vector from raw = max(range, 1e-8) / 3 (pack.py:459-463).
struct Step {
    float scale;            // the step as the packer uses it (after its bf16 round trip)
    float inv;              // exact inverse when inv_ok
    bool inv_ok;
    int e;                  // exponent (power-of-two modes)
    uint16_t bits;          // the step as bf16
    bool in_range;
};
__device__ __forceinline__ Step make_step(float raw, int mode, const float* tab) {
    Step s;
    if (mode == 2) {
        s.bits = f32_to_bf16_rne(raw);
        s.scale = bf16_to_f32(s.bits);
        s.inv = 0.0f; s.inv_ok = false; s.e = 0; s.in_range = true;
        return s;
    }
    s.e = pow2_round_exp(fmaxf(raw, 1e-12f), tab);
    s.in_range = s.e >= -126 && s.e <= 127;
    s.scale = exp2_int(s.e);
    s.inv_ok = s.e >= -126 && s.e <= 126;
    s.inv = exp2_int(s.inv_ok ? -s.e : 0);
    s.bits = static_cast<uint16_t>((s.e + 127) << 7);
    return s;
}

// INT2 code clamp(rint(x / 2^e), 0, 3) of a finite x.  v_cvt_pk_u8_f32 rounds to nearest even
// and saturates below at 0; the upper clamp commutes with the rounding.
__device__ __forceinline__ uint32_t int2_code(float x, float scale, float inv_scale, bool inv_ok) {
    if (inv_ok) return __builtin_amdgcn_cvt_pk_u8_f32(fminf(x * inv_scale, 3.0f), 0u, 0u);
    const float c = fminf(fmaxf(rintf(__fdiv_rn(x, scale)), 0.0f), 3.0f);
    return static_cast<uint32_t>(static_cast<int>(c));
}

// The same code from w, 2^-e and c = -zp * 2^-e in one fused multiply-add.  (w - zp) * 2^-e as the
// reference computes it is fl(w - zp) scaled exactly; the fused form rounds the exact (w - zp) * 2^-e
// once, and scaling by a power of two commutes with rounding while nothing under- or overflows: an
// underflowing quotient gives code 0 and an overflowing one code 3 either way.  The caller checks
// that c is finite (a huge zero point over a tiny step would make it infinite).
__device__ __forceinline__ uint32_t int2_code_fused(float w, float inv_scale, float c) {
    return __builtin_amdgcn_cvt_pk_u8_f32(fminf(__builtin_fmaf(w, inv_scale, c), 3.0f), 0u, 0u);
}

int launch_store_generic(const StoreArgs& a, int T, int in_dtype, hipStream_t st);

}  // namespace ommx

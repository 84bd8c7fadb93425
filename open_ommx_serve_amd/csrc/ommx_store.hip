// Quantize-on-store kernel: bf16/fp32 K,V rows -> the ten OMMX planes, bit-exact with
// the reference packer (ommx_gpu_serve/attention/pack.py:419-623; codec.py:45-65,
// 330-372).  Compiled with -ffp-contract=off: every fp32 operation below is a single
// IEEE rounding in the order the reference performs it.
//
// One workgroup packs one (32-token group, kv head).  It has D threads and does two jobs:
//   K: thread d owns the vector "channel d over the 32 tokens": outlier selection,
//      min/max of the rest, power-of-two scale, INT2 codes, FP4 map and nibbles.
//   V: thread x owns the vector "token x/(D/32), channels 32*(x%(D/32))..+31".
// The K codes of 4 neighbouring channels share a byte of k_base, so they are transposed
// through LDS and written as 8-byte pieces of the token-major rows.
#include <limits.h>

#include "ommx_store_common.h"

namespace ommx {

// Order-preserving integer image of a bf16 value held as fp32 bits, low 16 bits cleared.
// -0 must have been turned into +0 before (they tie in the reference's sorts).
__device__ __forceinline__ int ordered_bits(float x) {
    const int b = __float_as_int(x);
    return (b ^ ((b >> 31) & 0x7FFFFFFF)) & static_cast<int>(0xFFFF0000u);
}
// The same for a value whose low 16 bits are zero (a bf16 widened to fp32): nothing to clear.
__device__ __forceinline__ int ordered_bits_bf16(float x) {
    const int b = __float_as_int(x);
    return b ^ ((b >> 31) & 0x7FFF0000);
}
__device__ __forceinline__ float from_ordered_bits(int k) {
    const int s = k & static_cast<int>(0xFFFF0000u);
    // the image is its own inverse: the sign bit stays, the others flip under a set sign
    return __int_as_float(s ^ ((s >> 31) & 0x7FFF0000));
}
__device__ __forceinline__ int med3_i32(int a, int b, int c) {
    return max(min(a, b), min(max(a, b), c));          // v_med3_i32
}

// IDXT: index plane known at compile time (0 bitmap, 1 relidx7) or read from the arguments (2)
template <bool F32, bool FAST6, int IDXT>
// (six waves per SIMD for the tuned bitmask instantiation, which fits their 80 registers without spilling)
__global__ void __launch_bounds__(256, (FAST6 && IDXT == 0) ? 6 : 1) store_pack_kernel(StoreArgs a) {
    static_assert(!(F32 && FAST6), "the tuned path reads bf16 input");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // head_dim 128 is compiled in for the tuned instantiations (their launch checks it): row offsets
    // of the code tile become instruction immediates
    const int D = FAST6 ? 128 : a.D;
    uint8_t* s_codes = smem;                       // [32][D] one code per byte
    uint8_t* s_oval = smem + 32 * D;               // [D][nval] nibble bytes, packed as in memory
    uint8_t* s_oidx = smem + 36 * D;               // [D][nidx] position stream bytes (relidx7 only)
    const int g = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int NGV = D >> 5;
    const int kout = a.kout, kt = (kout + 1) >> 1, kb = kout - kt;
    const int nval = (kout + 1) >> 1;              // nibble bytes per frame
    const int64_t gs = a.dst_groups ? a.dst_groups[g] : g;
    const float* __restrict__ tab = a.table;
    // the tuned instantiation serves the serving recipe only: its variants are compile-time there
    const int scale_mode = FAST6 ? 0 : a.scale_mode;
    const bool select_abs = FAST6 ? false : a.select_abs != 0;
    const int idx_repr = IDXT == 2 ? a.idx_repr : IDXT;
    int err = 0;

    // ------------------------------------------------------------------ K vector
    {
        const int d = tid;
        float w[32];
        bool fin = true;
        if (a.src_rows) {
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const int64_t row = a.src_rows[g * 32 + i];
                w[i] = load_elem<F32>(a.K, row * a.k_ts + (int64_t)h * a.k_hs + d);
            }
        } else {
            // consecutive rows: the row address is the same for the whole workgroup (scalar registers,
            // advanced by one stride per row); the thread adds its channel as one 32-bit offset shared by
            // the 32 loads
            typedef const __attribute__((address_space(1))) char* gptr;      // a global-memory address
            uint64_t row = reinterpret_cast<uint64_t>(a.K) +
                           static_cast<uint64_t>(((int64_t)g * 32 * a.k_ts + (int64_t)h * a.k_hs) * (F32 ? 4 : 2));
            const uint64_t stride = static_cast<uint64_t>(a.k_ts * (F32 ? 4 : 2));
            const uint32_t off = static_cast<uint32_t>(d) * (F32 ? 4u : 2u);
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                if (F32) w[i] = *reinterpret_cast<const __attribute__((address_space(1))) float*>(reinterpret_cast<gptr>(row) + off);
                else w[i] = bf16_to_f32(*reinterpret_cast<const __attribute__((address_space(1))) uint16_t*>(reinterpret_cast<gptr>(row) + off));
                row += stride;
                asm volatile("" : "+s"(row));        // keeps the row address a scalar of its own: folded into one
                                                     // vector expression it costs four vector instructions a load
            }
        }
        if (!FAST6) {
#pragma unroll
            for (int i = 0; i < 32; ++i) fin = fin && is_finite_f32(w[i]);
        }

        uint32_t top = 0, bot = 0;
        int key_hi[3] = {0, 0, 0}, key_lo[3] = {0, 0, 0};    // FAST6: sorted keys of the chosen lanes
        int t4 = INT_MIN, b4 = INT_MAX;                      // FAST6: keys of the fourth largest / smallest lane
        auto select_generic = [&]() {
            if (select_abs) {
                // the kout largest magnitudes, ties to the lower index (stable descending sort
                // of |w|, pack.py:446-448)
                top = bot = 0;
                for (int r = 0; r < kout; ++r) {
                    float best = 0.0f; int bi = -1;
    #pragma unroll
                    for (int i = 0; i < 32; ++i) {
                        const bool free_lane = !((top >> i) & 1u);
                        if (free_lane && (bi < 0 || fabsf(w[i]) > best)) { best = fabsf(w[i]); bi = i; }
                    }
                    if (bi >= 0) top |= 1u << bi;
                }
                return;
            }
            // signed select (pack.py:436-445): kt largest, ties to the lower index ...
            top = 0;
            for (int r = 0; r < kt; ++r) {
                float best = 0.0f; int bi = -1;
    #pragma unroll
                for (int i = 0; i < 32; ++i) {
                    const bool free_lane = !((top >> i) & 1u);
                    if (free_lane && (bi < 0 || w[i] > best)) { best = w[i]; bi = i; }
                }
                if (bi >= 0) top |= 1u << bi;
            }
            // ... then kb smallest of the vector with chosen lanes replaced by +1e9.
            bot = 0;
            for (int r = 0; r < kb; ++r) {
                float best = 0.0f; int bi = -1;
    #pragma unroll
                for (int i = 0; i < 32; ++i) {
                    const float v = ((top >> i) & 1u) ? 1e9f : w[i];
                    const bool free_lane = !((bot >> i) & 1u);
                    if (free_lane && (bi < 0 || v < best)) { best = v; bi = i; }
                }
                if (bi >= 0) bot |= 1u << bi;
            }
        };
        bool fast_done = false, ranks_clean = false;
        if (FAST6) {
            // bf16 inputs leave 16 free bits under the value: key = ordered value bits | tie
            // breaker.  Largest three: tie breaker 31-i with max (equal values: lower index
            // first, the stable descending sort).  Smallest three: tie breaker i with min.
            // One pass each through a three-deep max / median network.
            // (a fourth rank on either side: the largest and the smallest of the lanes that stay)
            int t1 = INT_MIN, t2 = INT_MIN, t3 = INT_MIN;
            int b1 = INT_MAX, b2 = INT_MAX, b3 = INT_MAX;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const int ob = ordered_bits_bf16(w[i] + 0.0f);                   // FAST6 is a bf16-input instantiation
                const int kt_i = ob | (31 - i), kb_i = ob | i;
                const int n4 = med3_i32(t3, t4, kt_i), n3 = med3_i32(t2, t3, kt_i), n2 = med3_i32(t1, t2, kt_i);
                t1 = max(t1, kt_i); t2 = n2; t3 = n3; t4 = n4;
                const int m4 = med3_i32(b3, b4, kb_i), m3 = med3_i32(b2, b3, kb_i), m2 = med3_i32(b1, b2, kb_i);
                b1 = min(b1, kb_i); b2 = m2; b3 = m3; b4 = m4;
            }
            // (the fourth ranks are pinned here: left to the compiler, their two chains of 32 steps
            // move down into the one branch that reads them, and all 64 keys stay live until then)
            asm volatile("" : "+v"(t4), "+v"(b4));
            top = (1u << (31 - (t1 & 31))) | (1u << (31 - (t2 & 31))) | (1u << (31 - (t3 & 31)));
            bot = (1u << (b1 & 31)) | (1u << (b2 & 31)) | (1u << (b3 & 31));
            key_hi[0] = t1; key_hi[1] = t2; key_hi[2] = t3;
            key_lo[0] = b1; key_lo[1] = b2; key_lo[2] = b3;
            // The reference takes the smallest three of the vector with the top lanes moved
            // to +1e9.  That is the same set unless a top lane is among the overall smallest
            // three (heavy ties): then the bottom ranks are taken again with those lanes at +1e9.
            // (A pass with three running values, not the general selection below: that one
            // keeps two 32-element arrays in registers and would set this kernel's register
            // count.)
            ranks_clean = (top & bot) == 0u;
            if (!ranks_clean) {
                b1 = INT_MAX; b2 = INT_MAX; b3 = INT_MAX;
#pragma unroll
                for (int i = 0; i < 32; ++i) {
                    float wi = w[i];
                    asm volatile("" : "+v"(wi));      // formed again here: 32 keys kept from the first pass would cost 32 registers
                    // (the reference's own sentinel, so that a vector it refuses is refused here too)
                    const int kb_i = ordered_bits(((top >> i) & 1u) ? 1e9f : wi + 0.0f) | i;
                    const int m3 = med3_i32(b2, b3, kb_i), m2 = med3_i32(b1, b2, kb_i);
                    b1 = min(b1, kb_i); b2 = m2; b3 = m3;
                }
                bot = (1u << (b1 & 31)) | (1u << (b2 & 31)) | (1u << (b3 & 31));
                key_lo[0] = b1; key_lo[1] = b2; key_lo[2] = b3;
            }
            fast_done = true;
        }
        if (!fast_done) select_generic();
        const uint32_t om = top | bot;
        if (FAST6 && fast_done) {
            // NaN / Inf sort to the ends of the ordered keys: the largest and the smallest
            // chosen value tell whether the whole vector is finite
            fin = is_finite_f32(from_ordered_bits(key_hi[0])) && is_finite_f32(from_ordered_bits(key_lo[0]));
        } else if (FAST6) {
#pragma unroll
            for (int i = 0; i < 32; ++i) fin = fin && is_finite_f32(w[i]);
        }
        if (!fin) err |= OMMX_ERR_NONFINITE_K;
        if (__popc(om) != kout) err |= OMMX_ERR_UNDERFILLED;

        // affine base over the non-outlier lanes (pack.py:455-465)
        float mn = 1e9f, mx = -1e9f, omn = 1e9f, omx = -1e9f;
        // With three lanes taken from either end, what stays starts at the fourth rank, and the
        // outliers span the first ranks: no pass over the vector.  (With equal values around
        // the fourth rank its VALUE is still the extreme of the lanes that stay.)  A zero
        // minimum, or zero at both outlier ends, goes the long way: which sign a zero result
        // takes depends on the lanes, not on the ranks.
        bool ranks_do = false;
        if (FAST6 && ranks_clean) {
            mn = from_ordered_bits(b4);
            mx = from_ordered_bits(t4);
            omn = from_ordered_bits(key_lo[0]);
            omx = from_ordered_bits(key_hi[0]);
            ranks_do = mn != 0.0f && (omn != 0.0f || omx != 0.0f);
        }
        if (!ranks_do) {
            mn = 1e9f; mx = -1e9f; omn = 1e9f; omx = -1e9f;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const bool o = (om >> i) & 1u;
                mn = fminf(mn, o ? 1e9f : w[i]);
                mx = fmaxf(mx, o ? -1e9f : w[i]);
                omn = fminf(omn, o ? w[i] : 1e9f);
                omx = fmaxf(omx, o ? w[i] : -1e9f);
            }
        }
        if (mn > 1e8f) mn = 0.0f;
        if (mx < -1e8f) mx = 0.0f;
        if (omn > 1e8f) omn = 0.0f;
        if (omx < -1e8f) omx = 0.0f;
        const float raw = __fdiv_rn(fmaxf(mx - mn, 1e-8f), 3.0f);
        const Step st = make_step(raw, scale_mode, tab);
        if (!st.in_range) err |= OMMX_ERR_EXP_RANGE;
        if (st.e > 15) err |= OMMX_NOTE_WIDE_STEP;      // beyond the f16 operands of the matrix-core decode
        const float scale = st.scale;
        const uint16_t zp_b = f32_to_bf16_rne(mn);
        const float zp = bf16_to_f32(zp_b);

        // dedicated FP4 map over the outlier lanes (pack.py:486-498); without map planes the
        // outliers share the base scale and zero point instead (pack.py:502-506)
        const bool own_map = FAST6 ? true : a.k_ms != nullptr;
        uint16_t mc_b = 0, ms_b = 0;
        float mc = 0.0f, ms = 0.0f;
        if (kout > 0 && own_map) {
            mc_b = f32_to_bf16_rne(__fdiv_rn(omx + omn, 2.0f));
            // `12.0 / o_range` with a Python scalar on the left is torch's reciprocal-then-multiply
            // (Tensor.__rtruediv__): two roundings, which differ from one division once in some 1e5
            // vectors after the bf16 rounding (pack.py:492)
            ms_b = f32_to_bf16_rne(__fmul_rn(__fdiv_rn(1.0f, fmaxf(omx - omn, 1e-8f)), 12.0f));
            mc = bf16_to_f32(mc_b);
            ms = bf16_to_f32(ms_b);
        }

        const bool inv_ok = st.inv_ok;
        const float inv_scale = st.inv;
        // the value whose FP4 code is stored: (w - centre) * map_scale, or (w - zp) / scale
        // (a division by a power of two: the same rounding as the exact inverse multiply)
        auto fp4_input = [&](float wv) {
            if (own_map) return (wv - mc) * ms;
            return inv_ok ? (wv - zp) * inv_scale : __fdiv_rn(wv - zp, scale);
        };
        uint32_t nib = 0;
        bool mfin = true;
        if (FAST6 && fast_done) {
            const float zc = -zp * inv_scale;
            if (inv_ok && fabsf(zc) < INFINITY) {      // one branch per vector, not one per element
#pragma unroll
                for (int i = 0; i < 32; ++i)
                    s_codes[i * D + d] = static_cast<uint8_t>(int2_code_fused(w[i], inv_scale, zc));
            } else if (inv_ok) {
#pragma unroll
                for (int i = 0; i < 32; ++i)
                    s_codes[i * D + d] = static_cast<uint8_t>(int2_code(w[i] - zp, scale, inv_scale, true));
            } else {
#pragma unroll
                for (int i = 0; i < 32; ++i)
                    s_codes[i * D + d] = static_cast<uint8_t>(int2_code(w[i] - zp, scale, inv_scale, false));
            }
            // |(w - mc) * ms| is largest at the extreme lanes, which are outliers: they decide
            // whether every mapped value is finite (codec.py:55-57 checks all of them)
            float thr[8];      // the FP4 boundaries, the same for every thread: scalar registers
#pragma unroll
            for (int j2 = 1; j2 < 8; ++j2)
                thr[j2] = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(tab[256 + j2])));
            thr[0] = 0.0f;
#pragma unroll
            for (int r = 0; r < 6; ++r) {
                const int key = r < 3 ? key_hi[r] : key_lo[r - 3];
                const int pos = r < 3 ? 31 - (key & 31) : (key & 31);
                const float mapped = fp4_input(from_ordered_bits(key));
                mfin = mfin && is_finite_f32(mapped);
                const int slot = __popc(om & ((1u << pos) - 1u));
                nib |= fp4_encode_sorted(mapped, thr) << (4 * slot);
            }
        } else {
            int slot = 0;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                s_codes[i * D + d] = static_cast<uint8_t>(int2_code(w[i] - zp, scale, inv_scale, inv_ok));
                if (kout > 0) {
                    const float mapped = fp4_input(w[i]);
                    mfin = mfin && is_finite_f32(mapped);
                    if ((om >> i) & 1u) {
                        nib |= fp4_encode(mapped, tab + 256) << (4 * slot);
                        ++slot;
                    }
                }
            }
        }
        if (!mfin) err |= OMMX_ERR_NONFINITE_K;

        const int64_t gidx = (gs * a.H + h) * D + d;
        if (scale_mode == 0) a.k_scale[gidx] = static_cast<int8_t>(st.e);
        else reinterpret_cast<uint16_t*>(a.k_scale)[gidx] = st.bits;
        a.k_zp[gidx] = zp_b;
        if (kout > 0) {
            if (own_map) {
                a.k_ms[gidx] = ms_b;
                a.k_mc[gidx] = mc_b;
            }
            if (idx_repr == 0) {
                reinterpret_cast<uint32_t*>(a.k_obmp)[gidx] = om;  // byte p>>3, bit p&7
            } else {               // ascending positions, 7 bits each, least significant first
                uint64_t stream = 0;
                uint32_t m = om;
                for (int s = 0; s < kout; ++s) {
                    stream |= static_cast<uint64_t>(__ffs(m) - 1) << (7 * s);
                    m &= m - 1;
                }
                const int nidx = (7 * kout + 7) / 8;
                for (int b = 0; b < nidx; ++b)
                    s_oidx[d * nidx + b] = static_cast<uint8_t>(stream >> (8 * b));
            }
            for (int b = 0; b < nval; ++b) s_oval[d * nval + b] = static_cast<uint8_t>(nib >> (8 * b));
        }
    }
    __syncthreads();

    // nibble plane: D frames of nval bytes, contiguous in memory
    if (kout > 0) {
        const int64_t obase = (gs * a.H + h) * (int64_t)D * nval;
        // (D is a multiple of 32 and the plane is 8-byte aligned: whole dwords)
        for (int w = tid; w < D * nval / 4; w += D)
            reinterpret_cast<uint32_t*>(a.k_oval + obase)[w] = reinterpret_cast<const uint32_t*>(s_oval)[w];
        if (idx_repr != 0) {     // D frames of nidx bytes, contiguous in memory
            const int nidx = (7 * kout + 7) / 8;
            const int64_t ibase = (gs * a.H + h) * (int64_t)D * nidx;
            for (int w = tid; w < D * nidx / 4; w += D)
                reinterpret_cast<uint32_t*>(a.k_obmp + ibase)[w] = reinterpret_cast<const uint32_t*>(s_oidx)[w];
        }
    }

    // ------------------------------------------------- k_base rows and the V vector
    {
        const int t = tid / NGV, j = tid % NGV;           // token in group, 32-channel slice
        const int tok = g * 32 + t;
        const int lp = tok / a.ps;
        const int64_t page = a.dst_pages ? a.dst_pages[lp] : lp;
        const int64_t prow = page * a.ps + (tok % a.ps);  // physical token row

        // 32 code bytes -> 64 bits: four codes of a dword fold into its low byte
        uint64_t kb8 = 0;
        const uint4* cr = reinterpret_cast<const uint4*>(s_codes + t * D + 32 * j);
#pragma unroll
        for (int q4 = 0; q4 < 2; ++q4) {
            const uint4 u = cr[q4];
            const uint32_t uw[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int k = 0; k < 4; ++k)      // bytes (c0, c1, c2, c3) . (1, 4, 16, 64): one dot product per byte of the row
                kb8 |= static_cast<uint64_t>(__builtin_amdgcn_udot4(uw[k], 0x40100401u, 0u, false)) << (8 * (4 * q4 + k));
        }
        reinterpret_cast<uint64_t*>(a.k_base)[(prow * a.H + h) * NGV + j] = kb8;

        const int64_t row = a.src_rows ? a.src_rows[tok] : tok;
        const int64_t vbase = row * a.v_ts + (int64_t)h * a.v_hs + 32 * j;
        float v[32];
        bool fin = true;
        // finite <=> exponent field not all ones: the largest exponent field of the vector decides
        if (!F32 && a.v_vec) {                    // 64 contiguous bytes: four 16-byte loads
            typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
            u16x2 e2 = {0, 0};                    // largest exponent field of the even / of the odd channels
            const uint4* vp = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.V) + vbase);
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const uint4 u = vp[q4];
                const uint32_t uw[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v[8 * q4 + 2 * k] = __uint_as_float(uw[k] << 16);
                    v[8 * q4 + 2 * k + 1] = __uint_as_float(uw[k] & 0xFFFF0000u);
                    e2 = __builtin_elementwise_max(e2, __builtin_bit_cast(u16x2, uw[k] & 0x7F807F80u));
                }
            }
            fin = e2[0] != 0x7F80 && e2[1] != 0x7F80;
        } else {
            uint32_t emax = 0;
#pragma unroll
            for (int c = 0; c < 32; ++c) {
                v[c] = load_elem<F32>(a.V, vbase + c);
                emax = max(emax, __float_as_uint(v[c]) & 0x7F800000u);
            }
            fin = emax != 0x7F800000u;
        }
        float mn = 0.0f, mx = 0.0f;
#pragma unroll
        for (int c = 0; c < 32; ++c) {
            mn = c == 0 ? v[c] : fminf(mn, v[c]);
            mx = c == 0 ? v[c] : fmaxf(mx, v[c]);
        }
        if (!fin) err |= OMMX_ERR_NONFINITE_V;
        const float raw = __fdiv_rn(fmaxf(mx - mn, 1e-8f), 3.0f);
        const Step st = make_step(raw, scale_mode, tab);
        if (!st.in_range) err |= OMMX_ERR_EXP_RANGE;
        if (st.e > 15) err |= OMMX_NOTE_WIDE_STEP;
        const float scale = st.scale;
        const uint16_t zp_b = f32_to_bf16_rne(mn);
        const float zp = bf16_to_f32(zp_b);
        const bool inv_ok = st.inv_ok;
        const float inv_scale = st.inv;
        uint64_t vb8 = 0;
        const float zc = -zp * inv_scale;
        if (inv_ok && fabsf(zc) < INFINITY) {
#pragma unroll
            for (int c4 = 0; c4 < 8; ++c4) {
                uint32_t four = 0u;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    four = __builtin_amdgcn_cvt_pk_u8_f32(fminf(__builtin_fmaf(v[4 * c4 + k], inv_scale, zc), 3.0f), k, four);
                vb8 |= static_cast<uint64_t>(__builtin_amdgcn_udot4(four, 0x40100401u, 0u, false)) << (8 * c4);
            }
        } else if (inv_ok) {
#pragma unroll
            for (int c = 0; c < 32; ++c)
                vb8 |= static_cast<uint64_t>(int2_code(v[c] - zp, scale, inv_scale, true)) << (2 * c);
        } else {
#pragma unroll
            for (int c = 0; c < 32; ++c)
                vb8 |= static_cast<uint64_t>(int2_code(v[c] - zp, scale, inv_scale, false)) << (2 * c);
        }
        const int64_t vidx = (prow * a.H + h) * NGV + j;
        reinterpret_cast<uint64_t*>(a.v_main)[vidx] = vb8;
        if (scale_mode == 0) a.v_scale[vidx] = static_cast<int8_t>(st.e);
        else reinterpret_cast<uint16_t*>(a.v_scale)[vidx] = st.bits;
        a.v_zp[vidx] = zp_b;
    }
    if (err && a.err) atomicOr(a.err, err);
}

}  // namespace ommx

extern "C" void ommx_store_default_table(float* t) {
    // first float strictly above sqrt(2)*2^k: exact rint(log2(x)) switches there
    for (int kb = 0; kb < 256; ++kb) {
        const double b = 1.4142135623730951 * __builtin_ldexp(1.0, kb - 127);
        float c = static_cast<float>(b);
        if (static_cast<double>(c) < b) c = __builtin_nextafterf(c, __builtin_inff());
        t[kb] = (kb == 0 || kb == 255) ? __builtin_inff() : c;
    }
    // FP4 level boundaries: geometric means of neighbouring magnitudes (the zero level
    // counts as 1e-8), a tie staying with the lower level
    const double lv[8] = {1e-8, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0};
    t[256] = 0.0f;
    for (int j = 1; j < 8; ++j) {
        const double b = __builtin_sqrt(lv[j - 1] * lv[j]);
        float c = static_cast<float>(b);
        if (static_cast<double>(c) <= b) c = __builtin_nextafterf(c, __builtin_inff());
        t[256 + j] = c;
    }
}

extern "C" int ommx_store_pack(const void* K, const void* V, int in_dtype,
                               int64_t k_ts, int64_t k_hs, int64_t v_ts, int64_t v_hs,
                               const int32_t* src_rows, int T, int H, int D, int page_size,
                               int k_outliers, int index_repr, int select_abs, int scale_mode,
                               int group_tokens, int group_channels, int v_bf16,
                               const int32_t* dst_pages,
                               const int32_t* dst_groups, const float* table,
                               uint8_t* k_base, void* k_scale, uint16_t* k_zp,
                               uint16_t* k_ms, uint16_t* k_mc, uint8_t* k_index,
                               uint8_t* k_oval, uint8_t* v_main, void* v_scale,
                               uint16_t* v_zp, int32_t* err_flag, void* stream) {
    using namespace ommx;
    const int gt = group_tokens, gc = group_channels;
    if (!(gt == 16 || gt == 32 || gt == 64 || gt == 128) || !(gc == 16 || gc == 32 || gc == 64 || gc == 128)) {
        set_error("ommx_store_pack: group_tokens and group_channels must be 16, 32, 64 or 128");
        return -1;
    }
    if (T < 0 || T % gt || page_size <= 0 || T % page_size) {
        set_error("ommx_store_pack: T must be a multiple of group_tokens and of page_size");
        return -1;
    }
    if (D < 32 || D > 256 || D % 32 || D % gc || H <= 0) {
        set_error("ommx_store_pack: head_dim must be a multiple of 32 and of group_channels in [32,256]");
        return -1;
    }
    if (k_outliers < 0 || k_outliers > 16 || k_outliers > gt) {
        set_error("ommx_store_pack: outliers_per_vector must be in [0, min(16, group_tokens)]");
        return -1;
    }
    if (index_repr != 0 && index_repr != 1) { set_error("ommx_store_pack: index_repr"); return -1; }
    if (scale_mode < 0 || scale_mode > 2) { set_error("ommx_store_pack: scale_mode"); return -1; }
    if (in_dtype != 0 && in_dtype != 1) { set_error("ommx_store_pack: in_dtype"); return -1; }
    if (!K || !V || !table || !k_base || !k_scale || !k_zp || !v_main || !v_scale || !v_zp ||
        (k_outliers > 0 && (!k_index || !k_oval)) || (!k_ms != !k_mc)) {
        set_error("ommx_store_pack: null plane or input pointer");
        return -1;
    }
    if (T == 0) return 0;
    StoreArgs a{K, V, k_ts, k_hs, v_ts, v_hs, src_rows, dst_pages, dst_groups, table,
                k_base, static_cast<int8_t*>(k_scale), k_zp, k_ms, k_mc, k_index, k_oval, v_main,
                static_cast<int8_t*>(v_scale), v_zp,
                err_flag, H, D, page_size, k_outliers,
                (reinterpret_cast<uintptr_t>(V) % 16 == 0 && v_ts % 8 == 0 && v_hs % 8 == 0) ? 1 : 0,
                index_repr, select_abs ? 1 : 0, scale_mode, gt, gc, v_bf16 ? 1 : 0};
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (gt != 32 || gc != 32 || k_outliers > 8 || 32 % page_size || v_bf16) {   // everything but the 32x32 recipe
        if (launch_store_generic(a, T, in_dtype, st) != 0) {
            set_error("ommx_store_pack: no kernel for this recipe");
            return -1;
        }
        if (hipGetLastError() != hipSuccess) { set_error("ommx_store_pack: launch failed"); return -2; }
        return 0;
    }
    const dim3 grid(T / 32, H), block(D);
    const size_t shm = 32 * (size_t)D + 4 * (size_t)D + (index_repr ? 8 * (size_t)D : 0);
    const bool tuned = k_outliers == 6 && !select_abs && scale_mode == 0 && k_ms && D == 128;   // the serving recipe
    if (in_dtype == 1)
        hipLaunchKernelGGL((store_pack_kernel<true, false, 2>), grid, block, shm, st, a);
    else if (tuned && index_repr == 0)
        hipLaunchKernelGGL((store_pack_kernel<false, true, 0>), grid, block, shm, st, a);
    else if (tuned)
        hipLaunchKernelGGL((store_pack_kernel<false, true, 1>), grid, block, shm, st, a);
    else
        hipLaunchKernelGGL((store_pack_kernel<false, false, 2>), grid, block, shm, st, a);
    if (hipGetLastError() != hipSuccess) { set_error("ommx_store_pack: launch failed"); return -2; }
    return 0;
}

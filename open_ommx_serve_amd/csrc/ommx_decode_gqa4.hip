// Split-KV decode kernel for gfx950, serving shape: head_dim 128, 1, 2, 4 or 8 q heads per kv head,
// 6 outliers per K vector of 32 tokens (either index plane, either outlier map), INT2 V with
// 32-channel vectors, int8 exponents; in a general form (GEN) also 1..8 outliers on the bitmap
// plane and head_dim 64 with 1, 2 or 4 q heads per kv head.  Same operator as
// ommx_gpu_serve/attention/paged_decode.py:1255-2284; the other shapes of the matrix-core path
// (longer groups, no outliers) stay on the kernel in ommx_decode.hip.
//
// A wavefront owns one kv head (and its q heads) of one split and walks it 64 tokens at a time;
// a workgroup is 4 waves = 4 neighbouring kv heads.  Measured on MI355X this operator is bound
// by how many instructions a SIMD can issue (vector ALU first, LDS second, a 16-byte LDS access
// taking four issue slots), so the kernel is built for few instructions per token and to keep
// THREE waves per SIMD resident: at most 168 vector registers, no scratch memory, 13.4 KB of LDS
// per wave.  What that takes, against the kernel in ommx_decode.hip:
//   * P.V runs transposed (rows = V channels, columns = q heads), the V step 2^e sits in the
//     exponent field of the V operand, and the four column replicas of the q heads each take
//     every fourth channel block, so the output accumulator is 8 registers instead of 32;
//   * the softmax denominator comes out of the same matrix instruction that sums p*2^e and
//     p*zp (a row of ones), the running maximum is refreshed only when a logit exceeds it by
//     more than 2^8 (any bound that keeps exp2 in range serves an online softmax);
//   * the V staging area of LDS is the K staging area of the same step, reused once QK is done.
// With 8 q heads per kv head (NH = 8) the sixteen matrix rows / columns are two replicas of the
// heads instead of four: a lane then keeps four heads of one token of either group, the output
// takes four accumulators, and two workgroups fit a compute unit (190 registers, 14.1 KB of LDS
// per wave); everything up to the logits is the same code.
// Arithmetic: exact 16-bit operands, fp32 accumulation, as in ommx_decode.hip.
//   A (QK)   q * 2^(10-2m) as f16 in pair order, m = 1..4 fixed per channel pair; this one operand
//            set serves the base codes, the outlier tile and the bias columns.
//   K base   B = (1 + code*2^(2m-10)) * 2^e as f16: the 2-bit code is dropped into mantissa bits
//            [2m+1:2m] of a per-(group, channel) pattern that carries the exponent, one and-or per
//            channel pair.  The constant terms sum q*zp and sum A*2^e come from one small "bias"
//            MFMA per 64 tokens (zero points are staged divided by the channel's 2^(10-2m), exact).
//   outliers a channel-major pass (one lane = two channels) reads the stored 2-bit code of every
//            outlier position back from the staged K rows (the base MFMA takes every position as
//            stored; nothing is cleared there) and scatters
//            (outlier - zp - code*2^e) / 2^(10-2m) as f16 into a [32 tokens][128 channels] tile
//            that is the B operand of an f16 MFMA against the same A.  Entries whose f16 rounding
//            could show on a logit add their rounding residual times q through LDS float atomics.
//   P.V      A = (1 + code/4 | 1 + code/16) * 2^e_v as f16 for 8 tokens of one channel, B = p (f16).
#include <type_traits>

#include "ommx_decode_util.h"

namespace ommx {

namespace {

using namespace decode_util;

#ifndef OMMX_GQA4_WAVES
#define OMMX_GQA4_WAVES 3          // waves per SIMD the register budget is set for
#endif
constexpr int D = 128;
// ---- per-wave LDS map (bytes) ------------------------------------------------------------
constexpr int TILE_ROW = 272;                       // bytes per row of the outlier tile (256 used)
constexpr int KT_ROW = 40;                          // bytes per staged K code row (32 used): 16 rows read as b64 spread over all banks
constexpr int VT_COL = 68;                          // dwords per V dword column (64 used)
constexpr int PT_ROW = 72;                          // halfwords per row of the f16 [row][64 tokens] arrays
constexpr int OFF_TILE = 0;                         // [32 tokens][TILE_ROW] f16 outlier deltas of one group
constexpr int OFF_KT = OFF_TILE + 32 * TILE_ROW;    // [64 tokens][KT_ROW] K code rows
constexpr int OFF_MAG = OFF_KT + 64 * KT_ROW;       // [2 groups][128] f16 2^e, channels (p, p+8) adjacent
constexpr int OFF_ZPP = OFF_MAG + 512;              // same order, f16 zero points over the A scale
// after QK the same bytes hold what P.V needs
constexpr int OFF_VT = OFF_KT;                      // [8 dword columns][VT_COL] V code dwords
constexpr int OFF_PT = OFF_VT + 8 * VT_COL * 4;     // [NH heads][PT_ROW] f16 softmax weights
// what follows the weights depends on the number of q heads per kv head (NH = 4 or 8)
template <int NH>
struct LdsMap {
    static constexpr int OFF_VZ = OFF_PT + NH * PT_ROW * 2;    // [4 channel groups][PT_ROW] f16 V zero points
    static constexpr int OFF_VS = OFF_VZ + 4 * PT_ROW * 2;     // [4 channel groups][PT_ROW] f16 2^e_v
    static constexpr int OFF_STAGE_END = (OFF_VS + 4 * PT_ROW * 2 > OFF_ZPP + 512) ? OFF_VS + 4 * PT_ROW * 2 : OFF_ZPP + 512;
    static constexpr int OFF_LC = OFF_STAGE_END;               // [32 tokens][NH heads] f32 logit corrections of one group
    static constexpr int OFF_ZERO = OFF_LC + 32 * NH * 4;      // 128 B of zeros, never written again
    static constexpr int OFF_ONES = OFF_ZERO + 128;            // 128 B of f16 1.0, never written again
    static constexpr int LDS_WAVE = OFF_ONES + 128;            // 13376 (4 heads) / 14464 (8 heads)
    static_assert(OFF_KT % 16 == 0 && OFF_PT % 16 == 0 && OFF_VZ % 16 == 0 && OFF_LC % 16 == 0, "b128 alignment");
};
static_assert(3 * 4 * LdsMap<4>::LDS_WAVE <= 160 * 1024, "4 heads: three workgroups per compute unit");
static_assert(2 * 4 * LdsMap<8>::LDS_WAVE <= 160 * 1024, "8 heads: two workgroups per compute unit");

// One f16 carries 11 bits: rounding an outlier delta d costs up to |d| * 2^-11, i.e. up to
// |d| * max|q| * 2^-11 * sm_scale on a logit.  A delta with |d| * max|q| >= BIG_DELTA * 16
// (at most 1.4e-3 on a logit at sm_scale = 128^-0.5) gets its residual added exactly; smaller
// ones stay below that and average a quarter of it.  The bound is held at other sm_scale values
// (head_dim 64: 64^-0.5) by dividing the threshold by sm_scale / 128^-0.5; the general form, with
// up to 8 entries per vector, takes three quarters of it, and half with fewer than 6 outlier slots (more
// large values then stay in the base codes, the steps grow, and so do the entries).
constexpr float BIG_DELTA = 2.0f;
constexpr float BIG_DELTA_SM_SCALE = 0.08838834764831845f;
// the running maximum of the online softmax is refreshed when a logit (base 2) exceeds it by this
constexpr float MAX_SLACK = 8.0f;
// The base operand (1 + code*2^(2m-10)) * 2^e carries a constant A*2^e per channel, up to 2^8 times
// the signal, which the bias MFMA takes out again: two large sums that cancel in fp32.  From steps
// of 2^EXACT_STEP_EXP on (values a hundred or more wide inside one vector) that shows on the logits, and
// the step's two groups take the operand code*2^(2m-10+e) instead (one packed subtraction more per operand
// register, exact: both terms share the exponent) and drops the 2^e bias column.
constexpr int EXACT_STEP_EXP = 5;
// f16 operands: steps above 2^15 do not fit (K or V values beyond some 1e5); such a step is held at 2^15
// and OMMX_ERR_VALUE_RANGE is reported
constexpr int MAX_STEP_EXP = 15;

// K pair p of a code dword: channels p (low half) and p+8 (high half) as f16 with the 2-bit
// code at mantissa bits [2m+1:2m], m = k_pos(p) in 1..4, where the element reads
// (1 + code * 2^(2m-10)) * 2^e; the A operand of that channel carries q * 2^(10-2m).  Four
// positions, so that only pairs 0 (up two bits) and 5..7 (down six) need a shift.
__host__ __device__ constexpr int k_pos(int p) { return p == 0 ? 1 : (p <= 4 ? p : p - 3); }
template <int P>
__device__ __forceinline__ uint32_t k_pair(uint32_t w, uint32_t w_up2, uint32_t w_dn6, uint32_t magic) {
    const uint32_t sh = P == 0 ? w_up2 : (P <= 4 ? w : w_dn6);
    return (sh & (0x00030003u << (2 * k_pos(P)))) | magic;
}
// V channel y of a merged dword (token a in the low 16 bits, token b in the high 16 bits) as
// f16 (1 + c/16) * 2^e (even y, code at mantissa bits [7:6]) or (1 + c/4) * 2^e (odd y, bits
// [9:8]); `step` holds the f16 2^e of the two tokens.
template <int Y>
__device__ __forceinline__ uint32_t v_pair(uint32_t m, uint32_t step) {
    const uint32_t sh = Y <= 1 ? (m << 6) : Y <= 3 ? (m << 2) : Y <= 5 ? (m >> 2) : (m >> 6);
    return (sh & ((Y & 1) ? 0x03000300u : 0x00C000C0u)) | step;
}
__device__ __forceinline__ uint32_t pk_u16(uint32_t lo, uint32_t hi) { return (lo & 0xFFFFu) | (hi << 16); }

// IDX: 0 = outlier positions from 32-bit bitmaps, 1 = from 7-bit position streams.
// OWN_MAP: outliers decode through their own (map_scale, centre) pair; false = through the
// base scale and zero point.  PARTIAL: the kv head serves 1 or 2 q heads (spare head slots repeat
// the last head and are not written).  ORDER: 0 one request, 1 up to 64 requests served longest
// first, 2 up to 256 (radix select); see ommx_decode.hip.
// NH: q heads per kv head the matrix rows and columns are laid out for, 4 or 8.
// GEN: the general form of the recipe: 1..8 outliers per vector (a.kout, bitmap plane only), and
// head_dim 64 (a.half): the planes of two neighbouring 64-channel kv heads read exactly like one
// 128-channel head, so a wave takes the pair as one head whose q heads are those of both, each
// zero on the other one's channels, and writes each q head only its own half of the output.
template <int IDX, bool OWN_MAP, bool PARTIAL, int ORDER, int NH = 4, bool GEN = false, int KSLOTS = 6>
__global__ void __launch_bounds__(256, (NH == 8 || (GEN && KSLOTS == 8)) ? 2 : OMMX_GQA4_WAVES) decode_gqa4_kernel(DecodeArgs a) {
    static_assert(NH == 4 || (NH == 8 && !PARTIAL), "4 heads (or fewer, PARTIAL) or exactly 8");
    static_assert(!GEN || IDX == 0, "the general form reads bitmaps");
    // outlier slots walked per vector: the general form walks 4 or 8 whatever a.kout is (loads and
    // arithmetic of all slots go out together; only the writes of the slots beyond a.kout are skipped)
    constexpr int KMAX = GEN ? KSLOTS : 6;
    static_assert(KMAX == 4 || KMAX == 6 || KMAX == 8, "outlier slots");
    const int kout = GEN ? a.kout : 6;
    const bool half = GEN && a.half;
    using Lds = LdsMap<NH>;
    constexpr int OFF_VZ = Lds::OFF_VZ, OFF_VS = Lds::OFF_VS, OFF_LC = Lds::OFF_LC, OFF_ZERO = Lds::OFF_ZERO,
                  OFF_ONES = Lds::OFF_ONES, LDS_WAVE = Lds::LDS_WAVE;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem_all[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // uniform: keeps the plane pointers scalar
    uint8_t* const sm = smem_all + wave * LDS_WAVE;
    const uint32_t sm_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) uint8_t*)sm));
    const int j = lane & 15, kq = lane >> 4;
    const int Hkv = a.Hkv;
    const int waves = blockDim.x >> 6;
    const int kvh = blockIdx.y * waves + wave;
    const int heads = PARTIAL ? a.Hq / Hkv : NH;
    const int qh0 = kvh * heads;
    const int r_half = max(heads >> 1, 1);            // head_dim 64: q heads per kv head of the pair
    const int Dout = half ? 64 : D;                   // channels of an output state
    const int sp = blockIdx.x;
    int b = ORDER == 0 ? 0 : static_cast<int>(blockIdx.z), L;      // ORDER 0 is launched for one request only
    if (ORDER >= 1 && a.B > 1 && a.B <= 64) {
        const int my_len = lane < a.B ? a.seq[lane] : 0;
        const uint32_t key = (static_cast<uint32_t>(my_len) << 6) | (63u - lane);
        int rank = 0;
        for (int i = 0; i < a.B; ++i)
            rank += static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(key), i)) > key;
        b = __builtin_ctzll(__ballot(lane < a.B && rank == static_cast<int>(blockIdx.z)));
        L = __builtin_amdgcn_readlane(my_len, b);
    } else if (ORDER == 2 && a.B > 1 && a.B <= 256) {
        uint32_t key[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int idx = 64 * r + lane;
            key[r] = idx < a.B ? (static_cast<uint32_t>(a.seq[idx] + 1) << 8) | (255u - idx) : 0u;
        }
        uint32_t want = 0;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = want | (1u << bit);
            int reach = 0;
#pragma unroll
            for (int r = 0; r < 4; ++r) reach += __popcll(__ballot(key[r] >= cand));
            if (reach > static_cast<int>(blockIdx.z)) want = cand;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint64_t hit = __ballot(key[r] == want);
            if (hit) b = 64 * r + __builtin_ctzll(hit);
        }
        L = static_cast<int>(want >> 8) - 1;
    } else {
        L = a.seq[b];
    }
    // q: this lane's 32 channels of head j % NH (16 dwords, channel 2i in the low half of dword i)
    // and channels 2*lane, 2*lane+1 of every head (for the channel pass)
    uint32_t qw[16], qraw[NH];      // qraw: channels 2*lane, 2*lane+1 of every head, for the thresholds below
    {
        const int slot = min(j & (NH - 1), heads - 1);
        // head_dim 64: the head's 64 channels are the pair's channels 64 * (slot / r_half) .. + 63
        const bool q_real = !half || (kq >> 1) == slot / r_half;
        const uint32_t* qh = reinterpret_cast<const uint32_t*>(
            a.q + b * a.q_sb + (int64_t)(qh0 + slot) * a.q_sh + (half ? 32 * (kq & 1) : 32 * kq));
#pragma unroll
        for (int i = 0; i < 16; ++i) qw[i] = q_real ? qh[i] : 0u;
#pragma unroll
        for (int r = 0; r < NH; ++r) {
            const int sl = min(r, heads - 1);
            const uint32_t w = *reinterpret_cast<const uint32_t*>(
                a.q + b * a.q_sb + (int64_t)(qh0 + sl) * a.q_sh + (half ? (2 * lane) & 63 : 2 * lane));
            qraw[r] = (!half || (lane >> 5) == sl / r_half) ? w : 0u;
        }
    }
    // The A operands are q * 2^(10-2m) as f16, up to q * 2^8: a query element of 256 or more would not
    // fit.  When the wave's largest |q| reaches 2^7 the whole query is taken divided by a power of two
    // (exact) that brings it below, and the softmax scale carries the factor back; 0 for ordinary queries.
    int q_down = 0;
    {
        float qa = 0.0f;
#pragma unroll
        for (int r = 0; r < NH; ++r)
            qa = fmaxf(qa, fmaxf(fabsf(__uint_as_float(qraw[r] << 16)), fabsf(__uint_as_float(qraw[r] & 0xFFFF0000u))));
        if (__builtin_expect(__any(qa >= 128.0f) != 0, 0)) {
            float m4[4] = {qa, qa, qa, qa};
            wave_max4(m4);
            q_down = min(static_cast<int>((__float_as_uint(m4[0]) >> 23) & 0xFFu) - 127 - 6, 100);
        }
    }
    const float q_mul = __uint_as_float(static_cast<uint32_t>(127 - q_down) << 23);      // 2^-q_down
    // (uniform: kept in a scalar register, like the argument it stands for)
    const float sm_scale = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(
        a.sm_scale * __uint_as_float(static_cast<uint32_t>(127 + q_down) << 23))));
    if (__builtin_expect(q_down != 0, 0)) {
        // the per-channel copies too (thresholds and exact residuals below then need no factor of their own)
#pragma unroll
        for (int r = 0; r < NH; ++r) {
            const float lo = __uint_as_float(qraw[r] << 16) * q_mul, hi = __uint_as_float(qraw[r] & 0xFFFF0000u) * q_mul;
            qraw[r] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xFFFF0000u);
        }
    }
    // The 32-token groups are dealt out evenly: every split takes G/S groups and the first G%S
    // splits one more, so no two splits differ by more than one group and none is empty while
    // G >= S.  (One 32-bit division; the combine weighs the states by their lse, -inf for an
    // empty split, so it need not know this rule.)
    if (L < 0) { L = 0; report_table_range(a.err, true); }      // a negative length: nothing packed, reported
    const uint32_t G = static_cast<uint32_t>(L + 31) >> 5, S = static_cast<uint32_t>(a.S);
    const uint32_t g_each = G / S, g_more = G - g_each * S;
    const uint32_t g_first = static_cast<uint32_t>(sp) * g_each + min(static_cast<uint32_t>(sp), g_more);
    const uint32_t g_count = g_each + (static_cast<uint32_t>(sp) < g_more ? 1u : 0u);
    const int n_begin = static_cast<int>(g_first << 5);
    const int n_end = min(static_cast<int>((g_first + g_count) << 5), L);

    if (n_begin >= n_end) {       // an empty split: the state of nothing attended
        for (int r = 0; r < heads; ++r) {
            float* dst = a.al + b * a.al_b + (int64_t)(qh0 + r) * a.al_h + (int64_t)sp * a.al_s;
            dst[lane] = 0.0f;
            if (!half) dst[64 + lane] = 0.0f;
            if (lane == 0) dst[Dout] = -INFINITY;
        }
        return;
    }

    // ---- addressing ---------------------------------------------------------------------------
    const uint32_t row_bytes = (uint32_t)Hkv * 32u;          // of a code row (k_base, v_main): below 2^24
    const int last = n_end - 1;
    const int ps_sh = __ffs(a.ps) - 1, ps_mask = a.ps - 1;
    const int tsh = a.i64 ? 3 : 2;
    const int tok_off = a.gbase * 32 + a.off;
    const char* const rt_b = static_cast<const char*>(a.rt) + ((b * a.rt_s) << tsh);
    const char* const rg_b = static_cast<const char*>(a.rg) + ((b * a.rg_s + a.gbase) << tsh);
    const uint8_t* const kb_head = a.k_base + kvh * 32;
    const uint8_t* const vb_head = a.v_main + kvh * 32;
    const int8_t* const vs_head = a.v_scale + kvh * 4;
    const uint16_t* const vz_head = a.v_zp + kvh * 4;

    int pg1, ps1, gsl[2];
    auto fetch_tables = [&](int n) {
        const int p = min(n + lane, last) + tok_off;
        pg1 = *reinterpret_cast<const int*>(rt_b + ((uint32_t)(p >> ps_sh) << tsh));
        ps1 = p & ps_mask;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const int gi = min((n + 32 * g) >> 5, last >> 5);
            gsl[g] = *reinterpret_cast<const int*>(rg_b + ((uint32_t)gi << tsh));
        }
    };
    bool bad_id = false;            // a table entry outside the planes was seen (and clamped)
    bool over_step = false;         // a K or V step above 2^MAX_STEP_EXP was seen (and held there); wave-uniform
    // Every plane this kernel is launched on is smaller than 4 GiB (the launcher sends larger ones to the
    // kernel in ommx_decode.hip), so a row or a group is a scalar plane pointer plus a 32-bit byte offset:
    // no 64-bit address arithmetic in the loop.
    u32x4 kr[2], vr[2];
    u32x2 vzp;
    uint32_t vsc, vro;
    auto at = [](const void* base, uint32_t byte_off) { return static_cast<const char*>(base) + byte_off; };
    auto fetch_k = [&]() {          // K code row of this lane's token; remembers the row offset for fetch_v
        pg1 = clamp_id(pg1, a.n_pages, bad_id);
        vro = __umul24(static_cast<uint32_t>((pg1 << ps_sh) + ps1), row_bytes);
        kr[0] = *reinterpret_cast<const u32x4*>(at(kb_head, vro));
        kr[1] = *reinterpret_cast<const u32x4*>(at(kb_head, vro + 16));
    };
    auto fetch_v = [&]() {          // a row of v_scale is an eighth, a row of v_zp a quarter of a code row
        vr[0] = *reinterpret_cast<const u32x4*>(at(vb_head, vro));
        vr[1] = *reinterpret_cast<const u32x4*>(at(vb_head, vro + 16));
        vsc = *reinterpret_cast<const uint32_t*>(at(vs_head, vro >> 3));
        vzp = *reinterpret_cast<const u32x2*>(at(vz_head, vro >> 2));
    };
    // channel pair (2*lane, 2*lane+1) parameters of both groups
    uint32_t g_sc[2], g_zp[2], g_ms[2] = {0, 0}, g_mc[2] = {0, 0};
    u32x2 g_bm[2], g_ov[2];
    uint32_t g_bx[2] = {0, 0};
    const uint32_t kvh_s = __builtin_amdgcn_readfirstlane(kvh);
    auto fetch_params_g = [&](int g) {
        // (the lane number goes through an opaque copy: otherwise plane pointer + lane offset is kept
        // as a 64-bit register pair per plane across the loop, twelve registers the QK phase lacks;
        // this way the loads take a scalar base and a 32-bit lane offset)
        uint32_t lane_b = lane;
        asm volatile("" : "+v"(lane_b));
        const uint32_t gs = __builtin_amdgcn_readfirstlane(clamp_id(gsl[g], a.n_gslots, bad_id));
        const uint32_t gidx = (gs * static_cast<uint32_t>(Hkv) + kvh_s) * D;      // first channel of the group, in elements
        const uint32_t ch = gidx + 2 * lane_b;                                    // this lane's channel pair
        g_sc[g] = *reinterpret_cast<const uint16_t*>(at(a.k_scale, ch));
        g_zp[g] = *reinterpret_cast<const uint32_t*>(at(a.k_zp, 2 * ch));
        if (OWN_MAP) {
            g_ms[g] = *reinterpret_cast<const uint32_t*>(at(a.k_ms, 2 * ch));
            g_mc[g] = *reinterpret_cast<const uint32_t*>(at(a.k_mc, 2 * ch));
        }
        if constexpr (IDX == 0) {
            g_bm[g] = *reinterpret_cast<const u32x2*>(at(a.k_obmp, 4 * ch));
        } else {
            const uint32_t* ixp = reinterpret_cast<const uint32_t*>(at(a.k_obmp, 6 * ch));
            g_bm[g] = u32x2{ixp[0], ixp[1]};
            g_bx[g] = ixp[2];
        }
        if constexpr (!GEN) {
            // 3 nibble bytes per channel: the two dwords that hold the pair's six bytes
            const uint32_t* ovp = reinterpret_cast<const uint32_t*>(at(a.k_oval, 3 * gidx + 4 * ((3 * lane_b) / 2)));
            g_ov[g] = u32x2{ovp[0], ovp[1]};
        } else {
            // (kout + 1) / 2 bytes per channel, two channels per lane: the dword(s) that hold them
            const uint32_t kb = static_cast<uint32_t>(kout + 1) >> 1;
            const uint32_t* ovp = reinterpret_cast<const uint32_t*>(at(a.k_oval, gidx * kb + ((2 * kb * lane_b) & ~3u)));
            g_ov[g][0] = ovp[0];
            g_ov[g][1] = kb > 2 ? ovp[1] : 0u;       // 1 or 2 bytes per channel: one dword holds the pair
        }
    };
    // The page and group ids of the first step are asked for here; what follows (the A operands) needs
    // none of it and runs while they are on their way.
    fetch_tables(n_begin);
    asm volatile("" ::: "memory");

    // ---- A operand of QK: q * 2^(10-2m) of head j % 4 for this lane's 32-channel quarter, f16, in
    // pair order: k=(ks,kq,r) <-> channel 32kq + 16(ks/2) + 4(ks%2) + r/2 + 8(r%2).  The base codes,
    // the outlier tile and the bias columns all use this one operand (the tile and the zero points
    // are stored divided by the channel's 2^(10-2m)).
    u32x4 aq[4];
    {
        auto q_at = [&](int c) {
            return __uint_as_float((c & 1) ? (qw[c >> 1] & 0xFFFF0000u) : (qw[c >> 1] << 16));
        };
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int cl = 16 * (ks >> 1) + 4 * (ks & 1) + rr;
                const float qs = static_cast<float>(1 << (10 - 2 * k_pos(4 * (ks & 1) + rr))) * q_mul;
                aq[ks][rr] = pack_f16x2(qs * q_at(cl), qs * q_at(cl + 8));
            }
        }
    }
    // The first step's data is asked for as soon as the page and group ids are here; clearing LDS, the
    // accumulators and the lane constants need none of it and run while it is on its way (the A operands
    // above ran while the ids were; with the clearing of LDS up there as well the request goes out late
    // again: 31.0 against 29.8 us at batch 1, 64K).  The instantiation with the most registers in flight (position
    // streams with their own outlier map, 4 heads) asks after the constants instead: with the loaded rows
    // live across them it would spill.
    constexpr bool FETCH_FIRST = !(IDX == 1 && OWN_MAP && NH == 4);
    auto first_fetch = [&]() {
        // in the order the first step needs them: K rows, the group parameters, then V
        fetch_k();
        fetch_params_g(0);
        fetch_params_g(1);
        fetch_v();
        fetch_tables(n_begin + 64);
        asm volatile("" ::: "memory");
    };
    if constexpr (FETCH_FIRST) first_fetch();

    // ---- LDS that starts out constant: zero tile, zero corrections, the zero and one rows ----
    {
        u32x4* p = reinterpret_cast<u32x4*>(sm + OFF_TILE);
        for (int i = lane; i < 32 * TILE_ROW / 16; i += 64) p[i] = u32x4{0, 0, 0, 0};
        if (lane < 8 * NH) reinterpret_cast<u32x4*>(sm + OFF_LC)[lane] = u32x4{0, 0, 0, 0};
        if (lane < 16) reinterpret_cast<u32x4*>(sm + OFF_ZERO)[lane] =
            lane < 8 ? u32x4{0, 0, 0, 0} : u32x4{0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
    }

    // output accumulators: with 4 heads the 16 columns are 4 replicas of the heads and replica x takes
    // the channel blocks Y = x, x + 4 (two accumulators); with 8 heads they are 2 replicas and replica x
    // takes Y = x, x + 2, x + 4, x + 6 (four)
    f32x4 acc[NH / 2];
#pragma unroll
    for (int i = 0; i < NH / 2; ++i) acc[i] = f32x4{0, 0, 0, 0};
    f32x4 accz = {0, 0, 0, 0};
    float m_run[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) m_run[r] = -INFINITY;


    auto q_of = [&](int u, int r) { return __uint_as_float(u ? (qraw[r] & 0xFFFF0000u) : (qraw[r] << 16)); };
    // ---- lane constants of the loop ------------------------------------------------------------
    // channel pass: lane = channels c0 = 2*lane, c0 + 1
    const uint32_t c0 = 2u * lane;
    const uint32_t y0 = c0 & 15u;
    // halfword slot of channel c0 in the pair-ordered arrays; channel c0 + 1 sits two slots on
    const uint32_t hw0 = ((c0 >> 4) * 8u + (y0 & 7u)) * 2u + (y0 >> 3);
    // 2^-(10-2m) of the two channels: what their zero points and tile entries are scaled by
    const float cs0 = 1.0f / static_cast<float>(1 << (10 - 2 * k_pos(int(y0 & 7u))));
    const float cs1 = 1.0f / static_cast<float>(1 << (10 - 2 * k_pos(int((y0 + 1u) & 7u))));
    // per channel: the |tile entry| from which its f16 rounding matters (infinite for q = 0)
    float big_thr[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        float qm = 0.0f;
#pragma unroll
        for (int r = 0; r < NH; ++r)
            qm = fmaxf(qm, fabsf(__uint_as_float(u ? (qraw[r] & 0xFFFF0000u) : (qraw[r] << 16))));
        big_thr[u] = ((GEN ? (kout < 6 ? 0.5f : 0.75f) : 1.0f) * BIG_DELTA * 16.0f * BIG_DELTA_SM_SCALE) * (u ? cs1 : cs0) *
                     __builtin_amdgcn_rcpf(qm * sm_scale);
    }
    const uint32_t kt_lane = OFF_KT + (c0 >> 2);                   // code byte of the channel pair (4 channels a byte), row 0
    const uint32_t code_sh = 2u * (c0 & 3u);                      // bit of channel c0's code in that byte; c0 + 1 sits two on
    const uint32_t kbytes = static_cast<uint32_t>(kout + 1) >> 1;            // nibble bytes per channel
    const uint32_t nib_sh = 8u * ((2u * kbytes * lane) & 3u);
    const float c2 = sm_scale * 1.4426950408889634f;
    if constexpr (!FETCH_FIRST) first_fetch();

    for (int n0 = n_begin; n0 < n_end; n0 += 64) {
        const bool more = n0 + 64 < n_end;
        const bool g1_live = n0 + 32 < n_end;
        {   // waves sharing a SIMD should finish together: the one with more work left goes first
            const int left = (n_end - n0 + 63) >> 6;
            if (left >= 4) __builtin_amdgcn_s_setprio(3);
            else if (left == 3) __builtin_amdgcn_s_setprio(2);
            else if (left == 2) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(0);
        }

        // ------------------------------------------------------------------ stage K
        bool exact_step;                        // some step of these 64 tokens is 2^EXACT_STEP_EXP or more (wave-uniform)
        {
            typedef short s16x2e __attribute__((ext_vector_type(2)));
            const s16x2e top2 = __builtin_elementwise_max(
                __builtin_bit_cast(s16x2e, __builtin_amdgcn_perm(0u, g_sc[0], 0x010C000Cu)),
                __builtin_bit_cast(s16x2e, __builtin_amdgcn_perm(0u, g_sc[1], 0x010C000Cu)));
            const short e_top = top2[0] > top2[1] ? top2[0] : top2[1];
            // (a scaled-down query means operands near the top of f16: the same cancellation, the same remedy)
            exact_step = __any(e_top >= EXACT_STEP_EXP * 256) != 0 || q_down != 0;
            if (__builtin_expect(exact_step, 0)) over_step |= __any(e_top > MAX_STEP_EXP * 256) != 0;
        }
        {
            u32x2* krow = reinterpret_cast<u32x2*>(sm + OFF_KT + lane * KT_ROW);
            krow[0] = u32x2{kr[0][0], kr[0][1]};
            krow[1] = u32x2{kr[0][2], kr[0][3]};
            krow[2] = u32x2{kr[1][0], kr[1][1]};
            krow[3] = u32x2{kr[1][2], kr[1][3]};
            uint16_t* mg = reinterpret_cast<uint16_t*>(sm + OFF_MAG) + hw0;
            uint16_t* zp = reinterpret_cast<uint16_t*>(sm + OFF_ZPP) + hw0;
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                // f16 2^e of both channels: (e + 15) << 10 per half, e a signed byte held at -15 or
                // above (a step below 2^-14 is immaterial next to the f16 operands of the others)
                const uint32_t e2 = __builtin_amdgcn_perm(0u, g_sc[g], 0x010C000Cu);       // (e1 << 8, e0 << 8)
                typedef short s16x2 __attribute__((ext_vector_type(2)));
                typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
                const s16x2 ec = __builtin_elementwise_min(
                    __builtin_elementwise_max(__builtin_bit_cast(s16x2, e2), s16x2{-15 * 256, -15 * 256}),
                    s16x2{MAX_STEP_EXP * 256, MAX_STEP_EXP * 256});
                const uint32_t m2 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, ec) * u16x2{4, 4} + u16x2{0x3C00, 0x3C00});
                mg[g * 128] = static_cast<uint16_t>(m2);
                mg[g * 128 + 2] = static_cast<uint16_t>(m2 >> 16);
                // zero points over the channel's A scale (exact: a power of two), f16
                const uint32_t z2 = pack_f16x2(cs0 * __uint_as_float(g_zp[g] << 16),
                                               cs1 * __uint_as_float(g_zp[g] & 0xFFFF0000u));
                zp[g * 128] = static_cast<uint16_t>(z2);
                zp[g * 128 + 2] = static_cast<uint16_t>(z2 >> 16);
            }
        }
        lds_fence();
        if (more) fetch_k();

        // ------------------------------------------------------------------ QK
        // 4 heads: the lane keeps the logits of its own token n0 + lane (one 16-token block of one group);
        // 8 heads: rows 4kq..4kq+3 are heads 4(kq & 1)..+3, and the lane keeps those four heads of token
        // 16(kq >> 1) + j of either group
        f32x4 dsel[NH / 4];
#pragma unroll
        for (int i = 0; i < NH / 4; ++i) dsel[i] = f32x4{0, 0, 0, 0};
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            if (g == 1 && !g1_live) break;
            float* lc = reinterpret_cast<float*>(sm + OFF_LC);
            // The channel pass of a group in two halves, so that the code bytes of both channels are on their
            // way before either channel's entries need them: positions and code reads, then entries and scatter.
            // The base MFMA takes every position of the K rows as it is stored; the tile entry of an
            // outlier is what is missing on top of its stored 2-bit code, which the lane looks up
            // in the staged K rows (a byte read per outlier; the packer's code of an outlier is the
            // clamped 0 or 3 nearly always, so the entry is small).
            auto walk_read = [&](auto U, int (&pos)[KMAX], uint32_t (&cb)[KMAX]) {
                constexpr int u = decltype(U)::value;
                uint32_t bm = 0, ix_lo = 0, ix_hi = 0;
                if constexpr (IDX == 0) {
                    bm = g_bm[g][u];
                } else {
                    ix_lo = u ? __builtin_amdgcn_alignbit(g_bx[g], g_bm[g][1], 16) : g_bm[g][0];
                    ix_hi = u ? (g_bx[g] >> 16) : g_bm[g][1];
                }
                const uint8_t* kt = sm + kt_lane + g * 32 * KT_ROW;
#pragma unroll
                for (int sidx = 0; sidx < KMAX; ++sidx) {
                    if constexpr (IDX == 0) {
                        pos[sidx] = __builtin_ctz(bm) & 31;
                        if (sidx < KMAX - 1) bm &= bm - 1;
                    } else {
                        pos[sidx] = sidx < 4 ? ((ix_lo >> (7 * sidx)) & 31)
                                  : sidx == 4 ? (__builtin_amdgcn_alignbit(ix_hi, ix_lo, 28) & 31)
                                              : ((ix_hi >> 3) & 31);
                    }
                    cb[sidx] = kt[pos[sidx] * KT_ROW];
                }
            };
            auto walk_write = [&](auto U, const int (&pos)[KMAX], const uint32_t (&cb)[KMAX], float (&dls)[KMAX]) {
                constexpr int u = decltype(U)::value;
                const float zp = __uint_as_float(u ? (g_zp[g] & 0xFFFF0000u) : (g_zp[g] << 16));
                const int e = static_cast<int8_t>((g_sc[g] >> (8 * u)) & 0xFFu);
                const float s = __uint_as_float(static_cast<uint32_t>(e + 127) << 23);
                // everything below is in units of the channel's A scale: tile entry =
                // (outlier - zp - code * 2^e) / 2^(10-2m) = level * a1 + b1 (less 3 * sc for code 3)
                const float cs = u ? cs1 : cs0;
                const float sc = s * cs;
                float a1, b1;
                if (OWN_MAP) {
                    const float ms = __uint_as_float(u ? (g_ms[g] & 0xFFFF0000u) : (g_ms[g] << 16));
                    const float mc = __uint_as_float(u ? (g_mc[g] & 0xFFFF0000u) : (g_mc[g] << 16));
                    a1 = cs * __builtin_amdgcn_rcpf(ms);
                    b1 = cs * (mc - zp);
                } else {
                    a1 = sc;
                    b1 = 0.0f;
                }
                const uint64_t ov64 = (static_cast<uint64_t>(g_ov[g][1]) << 32) | g_ov[g][0];
                const uint32_t nib = GEN ? static_cast<uint32_t>(ov64 >> (nib_sh + 8 * kbytes * u))
                                         : static_cast<uint32_t>(ov64 >> (nib_sh + 24 * u)) & 0xFFFFFFu;
                const f32x2 l01 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 0);
                const f32x2 l23 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 1);
                const f32x2 l45 = KMAX > 4 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 2) : f32x2{0.0f, 0.0f};
                const f32x2 l67 = KMAX > 6 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 3) : f32x2{0.0f, 0.0f};
                const float lv[8] = {l01[0], l01[1], l23[0], l23[1], l45[0], l45[1], l67[0], l67[1]};
                uint16_t* dt = reinterpret_cast<uint16_t*>(sm + OFF_TILE) + hw0 + 2 * u;      // pair order, like MAG
                float dl_max = 0.0f;
#pragma unroll
                for (int sidx = 0; sidx < KMAX; ++sidx) {
                    const float dl0 = fmaf(lv[sidx], a1, b1);
                    const float code = static_cast<float>((cb[sidx] >> (code_sh + 2 * u)) & 3u);
                    float dl = fmaf(-code, sc, dl0);
                    // (the entry as a value of its own: rounded to f16 here exactly as the residual pass rounds it)
                    asm("" : "+v"(dl));
                    dls[sidx] = dl;
                    if (GEN && sidx >= kout) continue;          // an unused slot (uniform): nothing to write
                    dt[pos[sidx] * (TILE_ROW / 2)] = __builtin_bit_cast(uint16_t, static_cast<_Float16>(dl));
                    dl_max = fmaxf(dl_max, fabsf(dl));
                }
                return dl_max;
            };
            // Entries whose f16 rounding matters add what the rounding dropped to the logits, exactly
            // (rare, and kept out of the walks so that both channels' walks run as one stretch of code:
            // their positions and entries are still at hand)
            auto residuals = [&](auto U, const int (&pos)[KMAX], const float (&dls)[KMAX]) {
                constexpr int u = decltype(U)::value;
                const float un = __builtin_amdgcn_rcpf(u ? cs1 : cs0);
#pragma unroll
                for (int sidx = 0; sidx < KMAX; ++sidx) {
                    if (GEN && sidx >= kout) continue;
                    const float dl = dls[sidx];
                    if (fabsf(dl) >= big_thr[u]) {
                        const float lo = (dl - static_cast<float>(static_cast<_Float16>(dl))) * un;
#pragma unroll
                        for (int r = 0; r < NH; ++r)
                            __hip_atomic_fetch_add(lc + pos[sidx] * NH + r, lo * q_of(u, r), __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_WAVEFRONT);
                    }
                }
            };
            int pos0[KMAX], pos1[KMAX];
            uint32_t cb0[KMAX], cb1[KMAX];
            float dls0[KMAX], dls1[KMAX];
            // (the general form has fewer registers to spare: one channel after the other there)
            walk_read(std::integral_constant<int, 0>{}, pos0, cb0);
            if constexpr (!GEN) walk_read(std::integral_constant<int, 1>{}, pos1, cb1);
            const float dlm0 = walk_write(std::integral_constant<int, 0>{}, pos0, cb0, dls0);
            if constexpr (GEN) walk_read(std::integral_constant<int, 1>{}, pos1, cb1);
            const float dlm1 = walk_write(std::integral_constant<int, 1>{}, pos1, cb1, dls1);
            const bool res_any = __any(dlm0 >= big_thr[0] || dlm1 >= big_thr[1]) != 0;
            if (__builtin_expect(res_any, 0)) {
                residuals(std::integral_constant<int, 0>{}, pos0, dls0);
                residuals(std::integral_constant<int, 1>{}, pos1, dls1);
            }
            lds_fence();
            if (more) fetch_params_g(g);
            // both 16-token blocks of the group go through the eight k-steps together (two independent
            // accumulation chains): tile rows (read, clear), then the base codes
            f32x4 d[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
            u32x2 kw[2];
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2)
                kw[t2] = *reinterpret_cast<const u32x2*>(sm + OFF_KT + (16 * (2 * g + t2) + j) * KT_ROW + 8 * kq);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                for (int t2 = 0; t2 < 2; ++t2) {
                    u32x4* row = reinterpret_cast<u32x4*>(sm + OFF_TILE + (16 * t2 + j) * TILE_ROW + 64 * kq);
                    const u32x4 bt = row[ks];
                    row[ks] = u32x4{0, 0, 0, 0};
                    d[t2] = mfma_f16(aq[ks], bt, d[t2]);
                }
            }
            const u32x4* mg = reinterpret_cast<const u32x4*>(sm + OFF_MAG + g * 256 + kq * 64);
            auto base_mfmas = [&](auto EX) {
                // EX: the operand without its constant, code * 2^(2m-10+e) = pattern - 2^e
                auto op = [&](uint32_t pat, uint32_t mag) {
                    if constexpr (!decltype(EX)::value) return pat;
                    else return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, pat) - __builtin_bit_cast(f16x2, mag));
                };
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {          // code dword: channels 16*hf .. 16*hf+15 of the quarter
                    uint32_t w[2], wu[2], wd[2];
#pragma unroll
                    for (int t2 = 0; t2 < 2; ++t2) { w[t2] = kw[t2][hf]; wu[t2] = w[t2] << 2; wd[t2] = w[t2] >> 6; }
                    const u32x4 ma = mg[2 * hf], mb = mg[2 * hf + 1];
#pragma unroll
                    for (int t2 = 0; t2 < 2; ++t2)
                        d[t2] = mfma_f16(aq[2 * hf], u32x4{op(k_pair<0>(w[t2], wu[t2], wd[t2], ma[0]), ma[0]), op(k_pair<1>(w[t2], wu[t2], wd[t2], ma[1]), ma[1]),
                                                           op(k_pair<2>(w[t2], wu[t2], wd[t2], ma[2]), ma[2]), op(k_pair<3>(w[t2], wu[t2], wd[t2], ma[3]), ma[3])}, d[t2]);
#pragma unroll
                    for (int t2 = 0; t2 < 2; ++t2)
                        d[t2] = mfma_f16(aq[2 * hf + 1], u32x4{op(k_pair<4>(w[t2], wu[t2], wd[t2], mb[0]), mb[0]), op(k_pair<5>(w[t2], wu[t2], wd[t2], mb[1]), mb[1]),
                                                               op(k_pair<6>(w[t2], wu[t2], wd[t2], mb[2]), mb[2]), op(k_pair<7>(w[t2], wu[t2], wd[t2], mb[3]), mb[3])}, d[t2]);
                }
            };
            if (__builtin_expect(exact_step, 0)) {
                base_mfmas(std::true_type{});
                // the bias MFMA must not take the constant out a second time: its 2^e column of this group reads zeros
                lds_fence();
                reinterpret_cast<uint32_t*>(sm + OFF_MAG + g * 256)[lane] = 0u;
            } else {
                base_mfmas(std::false_type{});
            }
            if constexpr (NH == 4) {
                // rows 4kq..4kq+3 of every result hold the four heads: the lane keeps its own token block
#pragma unroll
                for (int t2 = 0; t2 < 2; ++t2)
                    if (kq == 2 * g + t2) dsel[0] = d[t2];
                if (res_any) {       // exact residuals of this group's large deltas, then zero again
                    const f32x4 corr = *reinterpret_cast<const f32x4*>(sm + OFF_LC + 16 * (lane & 31));
                    if ((kq >> 1) == g) dsel[0] += corr;
                    lds_fence();
                    *reinterpret_cast<u32x4*>(sm + OFF_LC + 16 * (lane & 31)) = u32x4{0, 0, 0, 0};
                }
            } else {
                dsel[g] = (kq >> 1) ? d[1] : d[0];
                if (res_any) {
                    // the lane's token of this group, its four heads
                    dsel[g] += *reinterpret_cast<const f32x4*>(sm + OFF_LC + 32 * (16 * (kq >> 1) + j) + 16 * (kq & 1));
                    lds_fence();
                    *reinterpret_cast<u32x4*>(sm + OFF_LC + 16 * lane) = u32x4{0, 0, 0, 0};
                }
            }
            lds_fence();
        }
        // bias columns: 0 zp(g0) 1 zp(g1) 2 2^e(g0) 3 2^e(g1); other columns repeat them
        f32x4 dbias = {0, 0, 0, 0};
        {
            const int src = ((j & 2) ? OFF_MAG : OFF_ZPP) + (j & 1) * 256 + kq * 64;
            const u32x4* bp = reinterpret_cast<const u32x4*>(sm + src);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) dbias = mfma_f16(aq[ks], bp[ks], dbias);
        }
        if (more) fetch_tables(n0 + 128);
        lds_fence();

        // ------------------------------------------------------------------ stage V (over the K staging)
        {
            uint32_t* vt = reinterpret_cast<uint32_t*>(sm + OFF_VT) + lane;
#pragma unroll
            for (int c = 0; c < 8; ++c) vt[c * VT_COL] = vr[c >> 2][c & 3];
            typedef short s16x2 __attribute__((ext_vector_type(2)));
            typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
            // a V step above 2^MAX_STEP_EXP (a signed exponent byte of 16 or more) is held there and reported
            if (__builtin_expect(__any((((vsc & 0x7F7F7F7Fu) + 0x70707070u) & ~vsc & 0x80808080u) != 0u) != 0, 0)) over_step = true;
            uint16_t* vs16 = reinterpret_cast<uint16_t*>(sm + OFF_VS) + lane;
            uint16_t* vz16 = reinterpret_cast<uint16_t*>(sm + OFF_VZ) + lane;
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
                // f16 2^e of two channel groups: (e + 15) << 10 per half; below 2^-15 the step is
                // immaterial and is held there
                const uint32_t e2 = __builtin_amdgcn_perm(0u, vsc, h2 ? 0x030C020Cu : 0x010C000Cu);   // (e << 8) pairs
                const s16x2 ec = __builtin_elementwise_min(
                    __builtin_elementwise_max(__builtin_bit_cast(s16x2, e2), s16x2{-15 * 256, -15 * 256}),
                    s16x2{MAX_STEP_EXP * 256, MAX_STEP_EXP * 256});
                const u16x2 st = __builtin_bit_cast(u16x2, ec) * u16x2{4, 4} + u16x2{0x3C00, 0x3C00};
                const uint32_t s2 = __builtin_bit_cast(uint32_t, st);
                vs16[(2 * h2) * PT_ROW] = static_cast<uint16_t>(s2);
                vs16[(2 * h2 + 1) * PT_ROW] = static_cast<uint16_t>(s2 >> 16);
                const uint32_t z2 = pack_f16x2(__uint_as_float(vzp[h2] << 16), __uint_as_float(vzp[h2] & 0xFFFF0000u));
                vz16[(2 * h2) * PT_ROW] = static_cast<uint16_t>(z2);
                vz16[(2 * h2 + 1) * PT_ROW] = static_cast<uint16_t>(z2 >> 16);
            }
        }
        if (more) fetch_v();

        // ------------------------------------------------------------------ softmax
        if constexpr (NH == 4) {
            // the lane owns token n0 + lane and the four heads; bias of (group, head) = sum q*zp - sum A*2^e
            float x[4];
            {
                const int gsel = lane >> 5;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    // lane 0 / 1 of every row: column 0 / 1 (zp) minus column 2 / 3 (2^e)
                    // (each row goes through a register of its own first: read straight out of the 4-register
                    // result, the four moves came out as one, all reading row 0)
                    float mine = dbias[r];
                    asm volatile("" : "+v"(mine));
                    const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                        0, __builtin_bit_cast(int, mine), 0x4E, 0xF, 0xF, true));     // quad_perm [2,3,0,1]
                    x[r] = dsel[0][r] + lane_value(mine - other, gsel);
                }
            }
            float pe[4];          // base-2 logit minus the running maximum
            if (a.cap > 0.0f) {
                asm volatile("" ::: "memory");
#pragma unroll
                for (int r = 0; r < 4; ++r) x[r] = apply_cap(x[r] * sm_scale, a.cap) * 1.4426950408889634f;
#pragma unroll
                for (int r = 0; r < 4; ++r) pe[r] = x[r] - m_run[r];
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    x[r] *= c2;
                    pe[r] = x[r] - m_run[r];
                }
            }
            const bool tok_ok = n0 + lane < n_end;
            if (n0 + 64 > n_end) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (!tok_ok) { x[r] = -INFINITY; pe[r] = -INFINITY; }
                }
            }
            if (__any(fmaxf(fmaxf(pe[0], pe[1]), fmaxf(pe[2], pe[3])) > MAX_SLACK)) {
                // refresh the running maxima (always on the first step) and rescale what is summed so far
                float mxs[4] = {x[0], x[1], x[2], x[3]};
                wave_max4(mxs);
                float alpha[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float m_new = fmaxf(m_run[r], mxs[r]);
                    alpha[r] = (m_run[r] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run[r] - m_new);
                    m_run[r] = m_new;
                    pe[r] = x[r] - m_new;
                }
                // accumulators hold column (x, head j % 4) in every register
                const float al = (j & 3) == 0 ? alpha[0] : ((j & 3) == 1 ? alpha[1] : ((j & 3) == 2 ? alpha[2] : alpha[3]));
#pragma unroll
                for (int i = 0; i < 4; ++i) { acc[0][i] *= al; acc[1][i] *= al; accz[i] *= al; }
            }
            {
                const uint32_t p01 = pack_f16x2(__builtin_amdgcn_exp2f(pe[0]), __builtin_amdgcn_exp2f(pe[1]));
                const uint32_t p23 = pack_f16x2(__builtin_amdgcn_exp2f(pe[2]), __builtin_amdgcn_exp2f(pe[3]));
                uint16_t* pt = reinterpret_cast<uint16_t*>(sm + OFF_PT) + lane;
                pt[0] = static_cast<uint16_t>(p01);
                pt[PT_ROW] = static_cast<uint16_t>(p01 >> 16);
                pt[2 * PT_ROW] = static_cast<uint16_t>(p23);
                pt[3 * PT_ROW] = static_cast<uint16_t>(p23 >> 16);
            }
        } else {
            // the lane owns tokens n0 + 32g + 16(kq >> 1) + j, g = 0, 1, and heads 4(kq & 1)..+3.  Every quad
            // of a row holds the bias columns (zp g0, zp g1, 2^e g0, 2^e g1) of the row's own heads.
            float x[2][4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float mine = dbias[r];
                asm volatile("" : "+v"(mine));
                const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                    0, __builtin_bit_cast(int, mine), 0x4E, 0xF, 0xF, true));     // quad_perm [2,3,0,1]
                float t = mine - other;                                           // lanes 0, 1 of a quad: bias of group 0, 1
                asm volatile("" : "+v"(t));
                x[0][r] = dsel[0][r] + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                    0, __builtin_bit_cast(int, t), 0x00, 0xF, 0xF, true));        // quad_perm [0,0,0,0]
                x[1][r] = dsel[1][r] + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                    0, __builtin_bit_cast(int, t), 0x55, 0xF, 0xF, true));        // quad_perm [1,1,1,1]
            }
            float pe[2][4];
            if (a.cap > 0.0f) {
                asm volatile("" ::: "memory");
#pragma unroll
                for (int g = 0; g < 2; ++g)
#pragma unroll
                    for (int r = 0; r < 4; ++r) x[g][r] = apply_cap(x[g][r] * sm_scale, a.cap) * 1.4426950408889634f;
            } else {
#pragma unroll
                for (int g = 0; g < 2; ++g)
#pragma unroll
                    for (int r = 0; r < 4; ++r) x[g][r] *= c2;
            }
            const int tk = 16 * (kq >> 1) + j;           // the lane's token inside either group
            if (n0 + 64 > n_end) {
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    const bool tok_ok = n0 + 32 * g + tk < n_end;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (!tok_ok) x[g][r] = -INFINITY;
                }
            }
            float over = -INFINITY;
#pragma unroll
            for (int g = 0; g < 2; ++g)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pe[g][r] = x[g][r] - m_run[r];
                    over = fmaxf(over, pe[g][r]);
                }
            if (__any(over > MAX_SLACK)) {
                // refresh the running maxima of the lane's four heads (rows kq and kq ^ 2 hold the same
                // heads) and rescale what is summed so far
                float mxs[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) mxs[r] = fmaxf(x[0][r], x[1][r]);
                rowpair_max4(mxs);
                float alpha[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float m_new = fmaxf(m_run[r], mxs[r]);
                    alpha[r] = (m_run[r] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run[r] - m_new);
                    m_run[r] = m_new;
                    pe[0][r] = x[0][r] - m_new;
                    pe[1][r] = x[1][r] - m_new;
                }
                // accumulators hold column (x, head j % 8) in every register: the factor of that head is
                // the lane's own when (j >> 2 & 1) == (kq & 1), else that of the neighbouring row
                float al_own = (j & 3) == 0 ? alpha[0] : ((j & 3) == 1 ? alpha[1] : ((j & 3) == 2 ? alpha[2] : alpha[3]));
                const float al_nb = lane_value(al_own, lane ^ 16);
                const float al = (((j >> 2) & 1) == (kq & 1)) ? al_own : al_nb;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[0][i] *= al; acc[1][i] *= al; acc[2][i] *= al; acc[3][i] *= al; accz[i] *= al;
                }
            }
            {
                uint16_t* pt = reinterpret_cast<uint16_t*>(sm + OFF_PT) + 4 * (kq & 1) * PT_ROW + tk;
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    const uint32_t p01 = pack_f16x2(__builtin_amdgcn_exp2f(pe[g][0]), __builtin_amdgcn_exp2f(pe[g][1]));
                    const uint32_t p23 = pack_f16x2(__builtin_amdgcn_exp2f(pe[g][2]), __builtin_amdgcn_exp2f(pe[g][3]));
                    pt[32 * g] = static_cast<uint16_t>(p01);
                    pt[32 * g + PT_ROW] = static_cast<uint16_t>(p01 >> 16);
                    pt[32 * g + 2 * PT_ROW] = static_cast<uint16_t>(p23);
                    pt[32 * g + 3 * PT_ROW] = static_cast<uint16_t>(p23 >> 16);
                }
            }
        }
        lds_fence();

        // ------------------------------------------------------------------ P.V (transposed)
        // Lane addresses of this phase, formed here from the lane number rather than carried through
        // the QK phase, where registers are shortest (the copy below keeps them from being hoisted).
        // Row i = j of the V operand is channel 16*(j & 7) + 8*(j >> 3) + Y; column j is (x = j >> 2, head j & 3),
        // or (x = j >> 3, head j & 7) with 8 heads.
        int lane_pv = lane;
        asm volatile("" : "+v"(lane_pv));
        const int jp = lane_pv & 15, kqp = lane_pv >> 4;
        const uint32_t vt_addr = OFF_VT + ((jp & 7) * VT_COL + 8 * kqp) * 4;
        const uint32_t vs_addr = OFF_VS + (((jp & 7) >> 1) * PT_ROW + 8 * kqp) * 2;
        const uint32_t pt_addr = OFF_PT + ((jp & (NH - 1)) * PT_ROW + 8 * kqp) * 2;
        // rows of the sums operand: 0-3 V zero points, 4-7 V steps, 8 ones, others zero
        const uint32_t az_addr = jp < 8 ? OFF_VZ + (jp * PT_ROW + 8 * kqp) * 2 : (jp == 8 ? OFF_ONES : OFF_ZERO) + 16 * kqp;
        const uint32_t vsel = (jp & 8) ? 0x07060302u : 0x05040100u;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (kb == 1 && !g1_live) break;
            // sums: rows vz[cg], 2^e[cg], ones against the weights of column (x, head)
            const u32x4 pw = *reinterpret_cast<const u32x4*>(sm + pt_addr + 64 * kb);
            const u32x4 az = *reinterpret_cast<const u32x4*>(sm + az_addr + 64 * kb);
            accz = mfma_f16(az, pw, accz);
            const u32x4 sw = *reinterpret_cast<const u32x4*>(sm + vs_addr + 64 * kb);
            const u32x4 va = *reinterpret_cast<const u32x4*>(sm + vt_addr + 128 * kb);
            const u32x4 vb = *reinterpret_cast<const u32x4*>(sm + vt_addr + 128 * kb + 16);
            const uint32_t mg0 = __builtin_amdgcn_perm(va[1], va[0], vsel);
            const uint32_t mg1 = __builtin_amdgcn_perm(va[3], va[2], vsel);
            const uint32_t mg2 = __builtin_amdgcn_perm(vb[1], vb[0], vsel);
            const uint32_t mg3 = __builtin_amdgcn_perm(vb[3], vb[2], vsel);
            if constexpr (NH == 4) {
                // column replica x takes the channel blocks Y with Y % 4 == x: for the others the weights are zeroed
#define OMMX_PVX(X)                                                                                       \
                {                                                                                         \
                    const bool mine = (jp >> 2) == X;                                                     \
                    const u32x4 bx = {mine ? pw[0] : 0u, mine ? pw[1] : 0u, mine ? pw[2] : 0u, mine ? pw[3] : 0u}; \
                    acc[0] = mfma_f16(u32x4{v_pair<X>(mg0, sw[0]), v_pair<X>(mg1, sw[1]),                 \
                                            v_pair<X>(mg2, sw[2]), v_pair<X>(mg3, sw[3])}, bx, acc[0]);   \
                    acc[1] = mfma_f16(u32x4{v_pair<4 + X>(mg0, sw[0]), v_pair<4 + X>(mg1, sw[1]),         \
                                            v_pair<4 + X>(mg2, sw[2]), v_pair<4 + X>(mg3, sw[3])}, bx, acc[1]); \
                }
                OMMX_PVX(0) OMMX_PVX(1) OMMX_PVX(2) OMMX_PVX(3)
#undef OMMX_PVX
            } else {
                // two column replicas: x takes the channel blocks Y with Y % 2 == x; blocks 2i and 2i + 1 share
                // accumulator i
                const bool first = (jp >> 3) == 0;
                const u32x4 bx0 = {first ? pw[0] : 0u, first ? pw[1] : 0u, first ? pw[2] : 0u, first ? pw[3] : 0u};
                const u32x4 bx1 = {first ? 0u : pw[0], first ? 0u : pw[1], first ? 0u : pw[2], first ? 0u : pw[3]};
#define OMMX_PVY(Y)                                                                                       \
                acc[(Y) >> 1] = mfma_f16(u32x4{v_pair<Y>(mg0, sw[0]), v_pair<Y>(mg1, sw[1]),              \
                                               v_pair<Y>(mg2, sw[2]), v_pair<Y>(mg3, sw[3])},             \
                                         ((Y) & 1) ? bx1 : bx0, acc[(Y) >> 1]);
                OMMX_PVY(0) OMMX_PVY(1) OMMX_PVY(2) OMMX_PVY(3) OMMX_PVY(4) OMMX_PVY(5) OMMX_PVY(6) OMMX_PVY(7)
#undef OMMX_PVY
            }
        }
        lds_fence();
    }

    report_table_range(a.err, bad_id);
    if (over_step && a.err && lane == 0) atomicOr(a.err, OMMX_ERR_VALUE_RANGE);

    // ---- epilogue: o = (f*(acc - sum p*2^e) + sum p*zp) / l, f = 16 or 4; lse = m + ln l ----------
    // sums live in the lanes of the same column j: rows 0-3 (kq 0) zero points, 4-7 (kq 1) steps, 8 (kq 2) ones
    // (lane-derived values are formed afresh here: carried over from the top of the kernel they
    // would sit in registers the loop needs, or in scratch memory)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int je = lane_e & 15, kqe = lane_e >> 4;
    const int h = je & (NH - 1), x = NH == 8 ? je >> 3 : je >> 2;
    const float l_tot = lane_value(accz[0], 32 + je);
    float z4[4], s4[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        z4[r] = lane_value(accz[r], je);
        s4[r] = lane_value(accz[r], 16 + je);
    }
    const float inv = l_tot > 0.0f ? __builtin_amdgcn_rcpf(l_tot) : 0.0f;
    if (h < heads) {
        float* dst = a.al + b * a.al_b + (int64_t)(qh0 + h) * a.al_h + (int64_t)sp * a.al_s;
#pragma unroll
        for (int a2 = 0; a2 < NH / 2; ++a2) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // row i = 4kq + r of block Y (4*a2 + x with 4 heads, 2*a2 + x with 8): channel
                // 16*(i & 7) + 8*(i >> 3) + Y, group (i & 7) / 2
                const float pz = (r >> 1) ? ((kqe & 1) ? z4[3] : z4[1]) : ((kqe & 1) ? z4[2] : z4[0]);
                const float psum = (r >> 1) ? ((kqe & 1) ? s4[3] : s4[1]) : ((kqe & 1) ? s4[2] : s4[0]);
                const int ch = 64 * (kqe & 1) + 16 * r + 8 * (kqe >> 1) + (NH == 8 ? 2 : 4) * a2 + x;
                const float f = (x & 1) ? 4.0f : 16.0f;
                const float val = (f * (acc[a2][r] - psum) + pz) * inv;
                if (!half) dst[ch] = val;
                else if ((kqe & 1) == h / r_half) dst[ch & 63] = val;     // the head's own 64 channels
            }
        }
        // the running maximum of head h: with 8 heads it lives in the rows with (kq & 1) == h >> 2
        if (x == 0 && kqe == (NH == 8 ? (h >> 2) : 0)) {
            const int hr = h & 3;
            const float mt = hr == 0 ? m_run[0] : (hr == 1 ? m_run[1] : (hr == 2 ? m_run[2] : m_run[3]));
            dst[Dout] = l_tot > 0.0f ? (mt + log2f(l_tot)) * 0.6931471805599453f : -INFINITY;
        }
    }
}

}  // namespace

// Returns 0 when launched, 1 when the shape belongs to another kernel.
int launch_decode_gqa4(const DecodeArgs& a_in, int Dh, int R, hipStream_t st) {
    DecodeArgs a = a_in;
    a.half = 0;
    if (a.scale_bf16 || a.v_bf16 || a.gt != 32 || a.gc != 32 || a.kout < 1 || a.kout > 8) return 1;
    if ((reinterpret_cast<uintptr_t>(a.q) & 3) || (a.q_sb & 1) || (a.q_sh & 1)) return 1;
    int nh;                                   // q heads of a wave's (pair of) kv head(s)
    if (Dh == 128 && (R == 1 || R == 2 || R == 4 || R == 8)) {
        nh = R;
    } else if (Dh == 64 && (R == 1 || R == 2 || R == 4) && a.Hkv % 2 == 0) {
        a.half = 1;                           // two 64-channel kv heads read as one 128-channel head
        a.Hkv /= 2;
        nh = 2 * R;
    } else {
        return 1;
    }
    {
        // the kernel addresses a plane by 32-bit byte offsets: it takes planes whose extents are given and
        // below 4 GiB (code rows: pages * page size * kv heads * 32 B; the widest group plane has 6 B per channel)
        const uint64_t lim = 0xFFFFFF00ull;
        if (a.n_pages <= 0 || a.n_gslots <= 0) return 1;
        if (static_cast<uint64_t>(a.n_pages) * static_cast<uint64_t>(a.ps) >= (1ull << 24)) return 1;
        if (static_cast<uint64_t>(a.n_pages) * a.ps * a.Hkv * 32ull > lim) return 1;
        if (static_cast<uint64_t>(a.n_gslots) * a.Hkv * D * 6ull > lim) return 1;
    }
    const bool general = a.half || a.kout != 6;
    if (general && a.idx_repr != 0) return 1;       // the general form reads bitmaps only
    const int waves = (a.Hkv % 4 == 0) ? 4 : ((a.Hkv % 2 == 0) ? 2 : 1);
    const dim3 grid(a.S, a.Hkv / waves, a.B), block(64 * waves);
    const size_t shm = (size_t)waves * (nh == 8 ? LdsMap<8>::LDS_WAVE : LdsMap<4>::LDS_WAVE);
    const bool own_map = a.k_ms != nullptr;
    const int order = a.B == 1 ? 0 : (a.B > 64 && a.B <= 256 ? 2 : 1);
#define OMMX_GO(IDX, MAP, PART, ORD, NH, GEN) \
    hipLaunchKernelGGL((decode_gqa4_kernel<IDX, MAP, PART, ORD, NH, GEN>), grid, block, shm, st, a)
#define OMMX_GO_GEN(MAP, PART, NH)                                                                          \
    do {                                                                                                    \
        if (a.kout <= 4) hipLaunchKernelGGL((decode_gqa4_kernel<0, MAP, PART, 2, NH, true, 4>), grid, block, shm, st, a); \
        else if (a.kout <= 6) hipLaunchKernelGGL((decode_gqa4_kernel<0, MAP, PART, 2, NH, true, 6>), grid, block, shm, st, a); \
        else hipLaunchKernelGGL((decode_gqa4_kernel<0, MAP, PART, 2, NH, true, 8>), grid, block, shm, st, a);             \
    } while (0)
#define OMMX_GO_ORD(IDX, MAP, PART, NH)                              \
    do {                                                             \
        if (order == 0) OMMX_GO(IDX, MAP, PART, 0, NH, false);       \
        else if (order == 2) OMMX_GO(IDX, MAP, PART, 2, NH, false);  \
        else OMMX_GO(IDX, MAP, PART, 1, NH, false);                  \
    } while (0)
    if (general) {
        // one instantiation per (outlier map, head layout): outlier count, head count and head_dim at run time
        if (nh == 8) { if (own_map) OMMX_GO_GEN(true, false, 8); else OMMX_GO_GEN(false, false, 8); }
        else { if (own_map) OMMX_GO_GEN(true, true, 4); else OMMX_GO_GEN(false, true, 4); }
        return 0;
    }
    switch ((nh == 8 ? 8 : 0) | (nh < 4 ? 4 : 0) | (a.idx_repr ? 2 : 0) | (own_map ? 1 : 0)) {
        case 0: OMMX_GO_ORD(0, false, false, 4); break;
        case 1: OMMX_GO_ORD(0, true, false, 4); break;
        case 2: OMMX_GO_ORD(1, false, false, 4); break;
        case 3: OMMX_GO_ORD(1, true, false, 4); break;
        case 4: OMMX_GO(0, false, true, 1, 4, false); break;
        case 5: OMMX_GO(0, true, true, 1, 4, false); break;
        case 6: OMMX_GO(1, false, true, 1, 4, false); break;
        case 7: OMMX_GO(1, true, true, 1, 4, false); break;
        case 8: OMMX_GO_ORD(0, false, false, 8); break;
        case 9: OMMX_GO_ORD(0, true, false, 8); break;
        case 10: OMMX_GO_ORD(1, false, false, 8); break;
        default: OMMX_GO_ORD(1, true, false, 8); break;
    }
#undef OMMX_GO
#undef OMMX_GO_GEN
#undef OMMX_GO_ORD
    return 0;
}

}  // namespace ommx

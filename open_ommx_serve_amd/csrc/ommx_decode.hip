// Tuned split-KV decode kernel for gfx950: head_dim 128, 1, 2, 4 or 8 q heads per kv head, 6 (or
// 0) outliers per K vector of 32 tokens; with the position-stream index plane also K vectors of
// 64 / 128 tokens (6 outliers, or 10 with 128 tokens) and V vectors of 64 / 128 channels.
// Same operator as ommx_gpu_serve/attention/paged_decode.py:1255-2284.
//
// Work decomposition.  A wavefront owns one kv head (and all 4 or 8 of its q heads) of one
// split and walks it 64 tokens (two 32-token K groups) at a time; waves never synchronise with
// each other.  A workgroup is 4 waves = 4 neighbouring kv heads, so together they consume whole
// 128-byte pieces of the token-major k_base / v_main rows.
//
// Arithmetic.  All dot products run on the matrix pipe (v_mfma_f32_16x16x32, fp32
// accumulate) with operands that are EXACT in their 16-bit type:
//   K base   B = (1 + code*2^(2k-7)) * 2^e   bf16, built with one and-or per channel pair (and
//            a shift shared by two pairs): the 2-bit code lands at mantissa bits [2k+1:2k]
//            (k = 1 or 2, fixed per pair) of a bf16 whose exponent field already holds the
//            group's power-of-two scale; A = q * 2^(7-2k) (bf16, exact).
//            sum A*B = sum q*code*s + sum A*s; the second term and sum q*zp come out of one
//            small "bias" MFMA per 64 tokens.
//   outliers a channel-major pass (one lane = two channels) overwrites the base code of every
//            outlier position in the staged K rows by 0 or 3 (ds_mskor_b32), so that the base
//            term of such an element is known, and scatters (outlier - zp - code*2^e)/4 as f16
//            into a per-group tile [32 tokens][128 channels] that is consumed as the B
//            operand of an f16 MFMA against A = 4*q (f16).  Deltas whose f16 rounding could
//            show on a logit (see BIG_DELTA) add their rounding residual times q straight
//            onto the logits through LDS float atomics.
//   P.V      B = (1 + code/4) or (1 + code/16) f16 for 8 tokens of one channel (V rows are
//            transposed through LDS at dword granularity), A = p * 2^e_v (f16, exact scaling);
//            sum_t p*vs and sum_t p*vz come from one extra MFMA per 32 tokens.
// The 16 MFMA rows hold the q heads several times over, and the copies are used as selectors.
//   4 heads: rows 4x..4x+3 carry the heads for token block x (QK) or with the scales of V
//            channel group x (P.V); a lane keeps the row group that matches its column.
//   8 heads: rows 8x..8x+7.  QK: a lane takes two token blocks (kq and kq^1) for the four heads
//            its result rows hold.  P.V: two row groups cannot tell four channel groups
//            apart, so the V columns are dealt in two sets (channel groups {0,1} and {2,3}),
//            each with its own A operand; the MFMA count per token is the same as with 4
//            heads, only softmax and the A operands double.
#include <type_traits>

#include "ommx_decode_util.h"

namespace ommx {

namespace {

constexpr int D = 128;
// per-wave LDS map (bytes)
// Row strides are padded so that the lanes of one access spread over all LDS banks.
constexpr int KT_ROW = 40;          // bytes per K code row (32 used)
constexpr int VT_COL = 68;          // dwords per V dword column (64 used)
constexpr int PT_ROW = 96;          // halfwords per row of the [4][64] f16 arrays (64 used)
constexpr int OFF_MAGIC = 0;        // [2 groups][64 pairs] bf16x2: 2^e of channels (p, p+8)
constexpr int OFF_ZPP = 512;        // same order, bf16 zero points
constexpr int OFF_KT = 1024;        // [64 tokens][KT_ROW] K code rows
constexpr int OFF_VT = OFF_KT + 64 * KT_ROW;        // [8 dword columns][VT_COL] V code dwords
constexpr int OFF_PT = OFF_VT + 8 * VT_COL * 4;     // [HR heads][PT_ROW] f16 softmax weights
constexpr int DT_ROW = 272;
template <int HR>                   // the rest depends on the q heads per wave
struct LdsMap {
    static constexpr int VS = OFF_PT + HR * PT_ROW * 2;    // [4 channel groups][PT_ROW] f16 2^e_v
    static constexpr int VZ = VS + 4 * PT_ROW * 2;         // [4 channel groups][PT_ROW] f16 v zero points
    static constexpr int DT = VZ + 4 * PT_ROW * 2;         // [32 tokens][DT_ROW B] f16 outlier deltas of one group
    static constexpr int LC = DT + 32 * DT_ROW;            // [64 tokens][HR] f32 logit corrections
    static constexpr int END = LC + 64 * HR * 4;           // 17792 / 19584: two 4-wave workgroups fit a CU's 160 KB
    static_assert(DT % 16 == 0 && LC % 16 == 0, "b128 alignment");
};
static_assert(OFF_VT % 16 == 0 && OFF_PT % 16 == 0, "b128 alignment");
// One f16 carries 11 bits: rounding d (an outlier delta in units of 4) costs up to |d| * 2^-11,
// i.e. up to |d| * max|4q| * 2^-11 * sm_scale on a logit.  A delta with |d| * max|4q| >=
// BIG_DELTA * 16 (|d| >= 2 at |q| = 4; at most 1.4e-3 on a logit at sm_scale = 128^-0.5) gets its
// residual added exactly; smaller ones stay below that and average a quarter of it.
constexpr float BIG_DELTA = 2.0f;

using namespace decode_util;

// K pair p of a code dword: channels p (low half) and p+8 (high half) as bf16.  The 2-bit code
// may sit anywhere in the mantissa: at bits [2k+1:2k] the element reads (1 + c*2^(2k-7))*2^e, and
// the matching A operand carries q*2^(7-2k), so the product is still q*c*2^e plus a constant
// that the bias MFMA removes.  Using two positions (k = 1, 2) lets neighbouring pairs share a
// shift, or need none.
__host__ __device__ constexpr int k_class(int p) { return (p == 2 || p == 4 || p == 6) ? 2 : 1; }
template <int P>
__device__ __forceinline__ uint32_t k_pair(uint32_t w, uint32_t magic) {
    const uint32_t sh = P == 0 ? (w << 2) : P <= 2 ? w : P <= 4 ? (w >> 4) : P <= 6 ? (w >> 8) : (w >> 12);
    return (sh & (k_class(P) == 1 ? 0x000C000Cu : 0x00300030u)) | magic;
}
// V channel y of a merged dword (token a in the low 16 bits, token b in the high 16 bits) as
// f16 1 + c/16 (even y, code at mantissa bits [7:6]) or 1 + c/4 (odd y, bits [9:8]); channels
// y and y+1 share their shift.
template <int Y>
__device__ __forceinline__ uint32_t v_pair(uint32_t m, uint32_t one_f16x2) {
    const uint32_t sh = Y <= 1 ? (m << 6) : Y <= 3 ? (m << 2) : Y <= 5 ? (m >> 2) : (m >> 6);
    return (sh & ((Y & 1) ? 0x03000300u : 0x00C000C0u)) | one_f16x2;
}

// HR: q heads per kv head (4 or 8), all on one wave.  IDX: 0 = outlier positions from 32-bit
// bitmaps, 1 = from 7-bit position streams (6 bytes per channel and group at 6 outliers).
// OWN_MAP: outliers decode through their own (map_scale, centre) pair; false = through the
// base scale and zero point (level * 2^e + zp), and there are no map planes.
// PARTIAL (HR = 4 only): the kv head serves 1 or 2 q heads; the spare head slots repeat the
// last head and are not written out.
// GTS: K groups of 32 << GTS tokens (position streams only).  The kernel keeps working in
// 32-token pieces: piece v of a longer group reads the group's parameters again and takes the
// outliers whose position falls into it.  The V vectors may then be 32, 64 or 128 channels wide.
// KO: outliers per K vector, 6, or 10 (position streams, 128-token groups: the 2.75-bit recipe).
// ORDER: which request orders the code holds: 0 none (one request), 1 up to 64 requests, 2 up to
// 256 as well (a radix select at the start).  Separate instantiations, because the mere presence
// of that code costs the others at batch 1 (register allocation and scheduling of the start-up
// shift): 1.7 us for the radix select, 0.4 us for the 64-request loop.
template <bool OUTLIERS, int HR, int IDX, bool OWN_MAP, bool PARTIAL = false, int GTS = 0, int KO = 6,
          int ORDER = 1>
__global__ void __launch_bounds__(256, 2) decode_splitkv_mfma_kernel(DecodeArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem_all[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int OFF_VS = LdsMap<HR>::VS, OFF_VZ = LdsMap<HR>::VZ, OFF_DT = LdsMap<HR>::DT,
                  OFF_LC = LdsMap<HR>::LC;
    uint8_t* const sm = smem_all + wave * (OUTLIERS ? LdsMap<HR>::END : OFF_DT);   // no tile without outliers
    // the same place as an LDS byte address (for LDS instructions issued by hand)
    const uint32_t sm_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) uint8_t*)sm));
    const int j = lane & 15, kq = lane >> 4;
    // With 8 heads the MFMA rows are (row group x = row / 8, head = row % 8); a lane holds rows
    // 4kq..4kq+3 of a result, i.e. heads 4*hg + r of row group kq / 2.
    const int hg = HR == 8 ? (kq & 1) : 0;
    const int Hkv = a.Hkv;
    const int waves = blockDim.x >> 6;
    const int kvh = blockIdx.y * waves + wave;
    const int heads = PARTIAL ? a.Hq / Hkv : HR;      // q heads this kv head really serves
    const int qh0 = kvh * heads;          // first of this wave's q heads
    const int sp = blockIdx.x;
    // Requests are served longest first: workgroups are dispatched in grid order, so the ones that
    // start last, when most compute units have run dry, belong to the shortest requests.
    // blockIdx.z is the rank of the request by (length descending, index ascending); every wave
    // finds its request from the lengths: up to 64 requests by counting, lane by lane, the keys
    // above its own; up to 256 (four keys per lane) by a radix select of the key of that rank,
    // one bit per round (the serving recipe's instantiations only); more keep the grid order.
    int b = blockIdx.z, L;
    if (ORDER >= 1 && a.B > 1 && a.B <= 64) {
        const int my_len = lane < a.B ? a.seq[lane] : 0;
        const uint32_t key = (static_cast<uint32_t>(my_len) << 6) | (63u - lane);   // distinct per lane
        int rank = 0;
        for (int i = 0; i < a.B; ++i)
            rank += static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(key), i)) > key;
        b = __builtin_ctzll(__ballot(lane < a.B && rank == static_cast<int>(blockIdx.z)));
        L = __builtin_amdgcn_readlane(my_len, b);
    } else if (ORDER == 2 && a.B > 1 && a.B <= 256) {
        // key = (length + 1, 255 - index): distinct, and above the zero of an unused slot
        uint32_t key[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int idx = 64 * r + lane;
            key[r] = idx < a.B ? (static_cast<uint32_t>(a.seq[idx] + 1) << 8) | (255u - idx) : 0u;
        }
        // the largest value that more than blockIdx.z keys reach is the key of rank blockIdx.z
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
    // q is requested first: it only needs the request index, and it is long here when the A
    // operands are built (after the first plane rows have been requested, while they travel).
    // qw: this lane's 32 channels of q of head j % HR, 16 dwords, channel 2i in the low half of
    // dword i; qraw: channels 2*lane, 2*lane+1 of every head (for the channel pass).
    uint32_t qw[16], qraw[HR];
    {
        const uint32_t* qh = reinterpret_cast<const uint32_t*>(
            a.q + b * a.q_sb + (int64_t)(qh0 + min(j & (HR - 1), heads - 1)) * a.q_sh + 32 * kq);
#pragma unroll
        for (int i = 0; i < 16; ++i) qw[i] = qh[i];
        if (OUTLIERS) {
#pragma unroll
            for (int r = 0; r < HR; ++r)
                qraw[r] = *reinterpret_cast<const uint32_t*>(
                    a.q + b * a.q_sb + (int64_t)(qh0 + min(r, heads - 1)) * a.q_sh + 2 * lane);
        }
    }
    constexpr int GT = 32 << GTS;
    static_assert(GTS == 0 || IDX == 1, "longer groups are read through position streams");
    static_assert(KO == 6 || (KO == 10 && IDX == 1), "10 outliers: position streams only");
    if (L < 0) { L = 0; report_table_range(a.err, true); }      // a negative length: nothing packed, reported
    const int per = ((((L + a.S - 1) / a.S) + GT - 1) / GT) * GT;
    const int n_begin = per * sp;
    const int n_end = min(n_begin + per, L);
    const float c_log2e = 1.4426950408889634f;

    if (OUTLIERS) {   // the outlier tile starts out all zero; readers clear what they consume
        u32x4* dt = reinterpret_cast<u32x4*>(sm + OFF_DT);
        for (int i = lane; i < 32 * DT_ROW / 16; i += 64) dt[i] = u32x4{0, 0, 0, 0};
    }

    uint32_t one2;                        // f16 (1.0, 1.0), pinned to a VGPR
    asm volatile("v_mov_b32 %0, 0x3c003c00" : "=v"(one2));

    f32x4 acc[8];
    f32x4 accz = {0, 0, 0, 0};
#pragma unroll
    for (int y = 0; y < 8; ++y) acc[y] = f32x4{0, 0, 0, 0};
    float m_run[4], l_run[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) { m_run[r] = -INFINITY; l_run[r] = 0.0f; }

    // ---- addressing: 32-bit indices, 64-bit only in the final multiply-add ----------------
    const uint32_t row_bytes = (uint32_t)Hkv * 32u;       // k_base / v_main bytes per token row
    const int last = n_end - 1;
    const int ps_sh = __ffs(a.ps) - 1, ps_mask = a.ps - 1;     // page_size is a power of two
    const int tsh = a.i64 ? 3 : 2;                             // low dword of an int64 entry
    const int tok_off = a.gbase * GT + a.off;
    const char* const rt_b = static_cast<const char*>(a.rt) + ((b * a.rt_s) << tsh);
    const char* const rg_b = static_cast<const char*>(a.rg) + ((b * a.rg_s + a.gbase) << tsh);
    const uint8_t* const kb_head = a.k_base + kvh * 32;      // a lane loads its own token's 32-byte rows
    const uint8_t* const vb_head = a.v_main + kvh * 32;
    // V vectors per token: 4 of 32 channels, or fewer of 64 / 128 (longer-group recipes only)
    const int ngv = GTS == 0 ? 4 : D / a.gc;
    const int8_t* const vs_head = a.v_scale + kvh * ngv;
    const uint16_t* const vz_head = a.v_zp + kvh * ngv;

    // The loop is software-pipelined by hand: table entries are fetched two iterations
    // ahead, plane data one iteration ahead, each into the registers its previous use
    // has just released.
    // Page entry and slot in the page of token n + lane, group slots: of the NEXT data loads.  The
    // entries stay as loaded until fetch_kv turns them into a row: arithmetic on them here would
    // put a wait for the table loads (and for every older load) right behind their issue.
    int pg1, ps1, gsl[2];
    auto fetch_tables = [&](int n) {
        {
            const int p = min(n + lane, last) + tok_off;
            pg1 = *reinterpret_cast<const int*>(rt_b + ((uint32_t)(p >> ps_sh) << tsh));
            ps1 = p & ps_mask;
        }
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const int gi = min((n + 32 * g) / GT, last / GT);
            gsl[g] = *reinterpret_cast<const int*>(rg_b + ((uint32_t)gi << tsh));
        }
    };
    u32x4 kr[2], vr[2];
    u32x2 vzp;
    uint32_t vsc;
    bool bad_id = false;            // a table entry outside the planes was seen (and clamped)
    auto fetch_kv = [&]() {
        pg1 = clamp_id(pg1, a.n_pages, bad_id);
        const int row1 = (pg1 << ps_sh) + ps1;              // physical row of this lane's token
        const uint64_t ro = (uint64_t)(uint32_t)row1 * row_bytes;
        kr[0] = *reinterpret_cast<const u32x4*>(kb_head + ro);
        kr[1] = *reinterpret_cast<const u32x4*>(kb_head + ro + 16);
        vr[0] = *reinterpret_cast<const u32x4*>(vb_head + ro);
        vr[1] = *reinterpret_cast<const u32x4*>(vb_head + ro + 16);
        const uint32_t my_row = row1;
        if (GTS == 0 || ngv == 4) {
            vsc = *reinterpret_cast<const uint32_t*>(vs_head + (uint64_t)my_row * (uint32_t)(Hkv * 4));
            vzp = *reinterpret_cast<const u32x2*>(vz_head + (uint64_t)my_row * (uint32_t)(Hkv * 4));
        } else if (ngv == 2) {      // two 64-channel vectors: each serves two 32-channel quarters
            const uint32_t e2 = *reinterpret_cast<const uint16_t*>(vs_head + (uint64_t)my_row * (uint32_t)(Hkv * 2));
            const uint32_t z2 = *reinterpret_cast<const uint32_t*>(vz_head + (uint64_t)my_row * (uint32_t)(Hkv * 2));
            vsc = __builtin_amdgcn_perm(0u, e2, 0x01010000u);
            vzp = u32x2{(z2 & 0xFFFFu) * 0x10001u, (z2 >> 16) * 0x10001u};
        } else {                    // one 128-channel vector
            const uint32_t e1 = *reinterpret_cast<const uint8_t*>(vs_head + (uint64_t)my_row * (uint32_t)Hkv);
            const uint32_t z1 = *(vz_head + (uint64_t)my_row * (uint32_t)Hkv);
            vsc = e1 * 0x01010101u;
            vzp = u32x2{z1 * 0x10001u, z1 * 0x10001u};
        }
    };
    // channel pair (2*lane, 2*lane+1) parameters of both groups
    uint32_t g_sc[2], g_zp[2], g_ms[2] = {0, 0}, g_mc[2] = {0, 0};
    constexpr bool own_map = OWN_MAP;
    u32x2 g_bm[2], g_ov[2];
    uint32_t g_bx[2];                     // third index dword (position streams only)
    // 10 outliers: 18 index bytes and 10 nibble bytes per lane start at a multiple of 2; the
    // aligned dwords that cover them are loaded and shifted into place when they are used
    uint32_t g_ix10[2][5], g_ov10[2][3];
    // (the group index is wave-uniform: base addresses are formed on the scalar unit, the lane
    // adds a 32-bit byte offset)
    const uint32_t kvh_s = __builtin_amdgcn_readfirstlane(kvh);
    const uint32_t lane_b = lane;
    auto at = [](const void* base, uint32_t byte_off) {
        return static_cast<const char*>(base) + byte_off;
    };
    auto fetch_params_g = [&](int g) {
        {
            const uint32_t gs = __builtin_amdgcn_readfirstlane(clamp_id(gsl[g], a.n_gslots, bad_id));   // same for every lane
            const uint64_t gidx = ((uint64_t)gs * (uint32_t)Hkv + kvh_s) * D;
            g_sc[g] = *reinterpret_cast<const uint16_t*>(at(a.k_scale + gidx, 2 * lane_b));
            g_zp[g] = *reinterpret_cast<const uint32_t*>(at(a.k_zp + gidx, 4 * lane_b));
            if (OUTLIERS) {
                if (own_map) {
                    g_ms[g] = *reinterpret_cast<const uint32_t*>(at(a.k_ms + gidx, 4 * lane_b));
                    g_mc[g] = *reinterpret_cast<const uint32_t*>(at(a.k_mc + gidx, 4 * lane_b));
                }
                if constexpr (KO == 10) {
                    const uint32_t* ixp = reinterpret_cast<const uint32_t*>(at(a.k_obmp + gidx * 9, (18 * lane_b) & ~3u));
#pragma unroll
                    for (int i = 0; i < 5; ++i) g_ix10[g][i] = ixp[i];
                    const uint32_t* ovp = reinterpret_cast<const uint32_t*>(at(a.k_oval + gidx * 5, (10 * lane_b) & ~3u));
#pragma unroll
                    for (int i = 0; i < 3; ++i) g_ov10[g][i] = ovp[i];
                } else if constexpr (IDX == 0) {
                    g_bm[g] = *reinterpret_cast<const u32x2*>(at(a.k_obmp + gidx * 4, 8 * lane_b));
                } else {          // 12 bytes: the streams of both channels
                    const uint32_t* ixp = reinterpret_cast<const uint32_t*>(at(a.k_obmp + gidx * 6, 12 * lane_b));
                    g_bm[g] = u32x2{ixp[0], ixp[1]};
                    g_bx[g] = ixp[2];
                }
                if constexpr (KO == 6) {
                    const uint32_t* ovp = reinterpret_cast<const uint32_t*>(at(a.k_oval + gidx * 3, 4 * ((3 * lane_b) / 2)));
                    g_ov[g] = u32x2{ovp[0], ovp[1]};
                }
            }
        }
    };
    auto fetch_params = [&]() { fetch_params_g(0); fetch_params_g(1); };
    if (n_begin >= n_end) {
        // An empty split leaves the state of nothing attended (o = 0, lse = -inf) and is done.
        // (Leaving here, rather than running the rest with an empty loop, also keeps the loads
        // below on every path that reaches the A operands: the waits placed there then let the
        // plane rows travel while the operands are built.)
        for (int r = 0; r < heads; ++r) {
            float* dst = a.al + b * a.al_b + (int64_t)(qh0 + r) * a.al_h + (int64_t)sp * a.al_s;
            dst[lane] = 0.0f;
            dst[64 + lane] = 0.0f;
            if (lane == 0) dst[D] = -INFINITY;
        }
        return;
    }
    fetch_tables(n_begin);
    fetch_kv();
    fetch_params();
    fetch_tables(n_begin + 64);

    // ---- A operands: scaled q of head j % HR for this lane's 32-channel quarter ---------
    // (pair order: q * 2^(7-2k) with k the code position of the pair, see k_pair; natural
    // order: 4*q)
    // pair order (QK base, bias):   k=(ks,kq,r) <-> channel 32kq + 16(ks/2) + 4(ks%2) + r/2 + 8(r%2)
    // natural order (outlier tile): k=(ks,kq,r) <-> channel 32kq + 8ks + r
    u32x4 aq_pair[4], aq_nat[4];
    {
        auto q_at = [&](int c) {          // channel c of the quarter as fp32 (exact)
            return __uint_as_float((c & 1) ? (qw[c >> 1] & 0xFFFF0000u) : (qw[c >> 1] << 16));
        };
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int cl = 16 * (ks >> 1) + 4 * (ks & 1) + rr;
                const float qs = k_class(4 * (ks & 1) + rr) == 1 ? 32.0f : 8.0f;    // 2^(7-2k)
                const float lo = qs * q_at(cl), hi = qs * q_at(cl + 8);
                // bf16 pair (lo, hi): the upper halves of the two fp32 words (exact products)
                aq_pair[ks][rr] = __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
                aq_nat[ks][rr] = pack_f16x2(4.0f * q_at(8 * ks + 2 * rr), 4.0f * q_at(8 * ks + 2 * rr + 1));
            }
        }
    }
    // q of every head for the channel pass, channels 2*lane and 2*lane+1: as fp32 with 4
    // heads, left as the bf16 pair with 8 (registers are short there, and the residual walk
    // that reads them is rare)
    float qf[2][4];
    auto q4_at = [&](int u, int r) {      // 4*q
        if constexpr (HR == 4) return qf[u][r];
        else return 4.0f * __uint_as_float(u ? (qraw[r] & 0xFFFF0000u) : (qraw[r] << 16));
    };
    // per channel: the |delta/4| from which the residual matters (infinite for q = 0)
    float big_thr[2] = {0.0f, 0.0f};
    if (OUTLIERS) {
        if constexpr (HR == 4) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                qf[0][r] = 4.0f * __uint_as_float(qraw[r] << 16);
                qf[1][r] = 4.0f * __uint_as_float(qraw[r] & 0xFFFF0000u);
            }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            float qm = 0.0f;
#pragma unroll
            for (int r = 0; r < HR; ++r) qm = fmaxf(qm, fabsf(q4_at(u, r)));
            big_thr[u] = (BIG_DELTA * 16.0f) * __builtin_amdgcn_rcpf(qm);
        }
    }


    for (int n0 = n_begin; n0 < n_end; n0 += 64) {
        const bool tok_ok = n0 + lane < n_end;
        const bool more = n0 + 64 < n_end;
        // Waves that share a SIMD should finish together (a wave running alone leaves issue
        // slots empty), but the arbiter favours the older wave: give the wave with more work
        // left the higher priority.
        {
            const int left = (n_end - n0 + 63) >> 6;
            if (left >= 4) __builtin_amdgcn_s_setprio(3);
            else if (left == 3) __builtin_amdgcn_s_setprio(2);
            else if (left == 2) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(0);
        }

        // ---------------------------------------------------------------- stage to LDS
        // K code rows (for the outlier pass), transposed V dwords
        {   // row of token lane: 32 code bytes of K (rows are 8-byte aligned), 8 dwords of V
            u32x2* krow = reinterpret_cast<u32x2*>(sm + OFF_KT + lane * KT_ROW);
            krow[0] = u32x2{kr[0][0], kr[0][1]};
            krow[1] = u32x2{kr[0][2], kr[0][3]};
            krow[2] = u32x2{kr[1][0], kr[1][1]};
            krow[3] = u32x2{kr[1][2], kr[1][3]};
            uint32_t* vt = reinterpret_cast<uint32_t*>(sm + OFF_VT) + lane;
#pragma unroll
            for (int c = 0; c < 8; ++c) vt[c * VT_COL] = vr[c >> 2][c & 3];
        }
        // V scales / zero points of this lane's token as f16, [group][token]
        {
            uint16_t* vs16 = reinterpret_cast<uint16_t*>(sm + OFF_VS);
            uint16_t* vz16 = reinterpret_cast<uint16_t*>(sm + OFF_VZ);
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int e = static_cast<int8_t>((vsc >> (8 * g4)) & 0xFFu);
                float s = __uint_as_float(static_cast<uint32_t>(e + 127) << 23);
                const uint32_t zb = (g4 & 1) ? (vzp[g4 >> 1] & 0xFFFF0000u) : (vzp[g4 >> 1] << 16);
                float z = __uint_as_float(zb);
                if (!tok_ok) { s = 0.0f; z = 0.0f; }
                vs16[g4 * PT_ROW + lane] = __builtin_bit_cast(uint16_t, static_cast<_Float16>(s));
                vz16[g4 * PT_ROW + lane] = __builtin_bit_cast(uint16_t, static_cast<_Float16>(z));
            }
        }
        // per-channel 2^e and zp in pair order
        {
            uint16_t* mg = reinterpret_cast<uint16_t*>(sm + OFF_MAGIC);
            uint16_t* zp = reinterpret_cast<uint16_t*>(sm + OFF_ZPP);
#pragma unroll
            for (int g = 0; g < 2; ++g) {
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int c = 2 * lane + u;
                    const int y = c & 15;
                    const int hw = (((c >> 4) * 8) + (y & 7)) * 2 + (y >> 3);
                    const int e = static_cast<int8_t>((g_sc[g] >> (8 * u)) & 0xFFu);
                    mg[g * 128 + hw] = static_cast<uint16_t>((e + 127) << 7);
                    // zero point divided by the channel's A scale 2^(7-2k), so that the bias
                    // MFMA returns sum q*zp (exact: a shift of the exponent field)
                    const uint32_t zb = u ? (g_zp[g] >> 16) : (g_zp[g] & 0xFFFFu);
                    const uint32_t zsh = k_class(y & 7) == 1 ? 5u : 3u;
                    zp[g * 128 + hw] = static_cast<uint16_t>(
                        ((zb >> 7) & 0xFFu) > zsh ? zb - (zsh << 7) : (zb & 0x8000u));
                }
            }
        }
        if (OUTLIERS) {
#pragma unroll
            for (int i = 0; i < HR / 4; ++i)
                *reinterpret_cast<u32x4*>(sm + OFF_LC + 4 * HR * lane + 16 * i) = u32x4{0, 0, 0, 0};
        }
        lds_fence();
        if (more) fetch_kv();             // K/V registers are staged: start the next rows

        // ---------------------------------------------------------------- QK
        // per group: channel pass (clear outlier codes, scatter deltas), then the token
        // blocks of the group take tile and base terms in one accumulation chain
        f32x4 dq[4];
        const bool g1_live = n0 + 32 < n_end;     // a last step of one group skips the second
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            if (g == 1 && !g1_live) {
                dq[2] = f32x4{0, 0, 0, 0};
                dq[3] = f32x4{0, 0, 0, 0};
                break;
            }
            if (OUTLIERS) {
                // RES = false: the walk every group takes.  RES = true: a second walk that only
                // adds f16 rounding residuals of large deltas onto the logits.
                float dl_max[2] = {0.0f, 0.0f};
                const int piece = ((n0 >> 5) + g) & ((1 << GTS) - 1);     // 32-token piece of the group
                auto walk = [&](auto RES, auto U) {
                    constexpr int u = decltype(U)::value;
                    {
                        const int c = 2 * lane + u;
                        const float zp = __uint_as_float(u ? (g_zp[g] & 0xFFFF0000u) : (g_zp[g] << 16));
                        const float ms = __uint_as_float(u ? (g_ms[g] & 0xFFFF0000u) : (g_ms[g] << 16));
                        const float mc = __uint_as_float(u ? (g_mc[g] & 0xFFFF0000u) : (g_mc[g] << 16));
                        // tile value (outlier - zp)/4 = level * a1 + b1
                        const int e = static_cast<int8_t>((g_sc[g] >> (8 * u)) & 0xFFu);
                        const float s = __uint_as_float(static_cast<uint32_t>(e + 127) << 23);
                        const float a1 = own_map ? 0.25f * __builtin_amdgcn_rcpf(ms) : 0.25f * s;
                        const float b1 = own_map ? 0.25f * (mc - zp) : 0.0f;
                        uint32_t bm = 0;
                        if constexpr (IDX == 0) bm = g_bm[g][u];
                        // position stream of this channel: 42 bits from bit 0 (u = 0) or bit 48
                        uint32_t ix_lo = 0, ix_hi = 0;
                        if constexpr (IDX == 1 && KO == 6) {
                            ix_lo = u ? __builtin_amdgcn_alignbit(g_bx[g], g_bm[g][1], 16) : g_bm[g][0];
                            ix_hi = u ? (g_bx[g] >> 16) : g_bm[g][1];
                        }
                        float lv[KO];
                        uint32_t ixw[5] = {0, 0, 0, 0, 0};       // 10 outliers: index window, channel 0 at bit 0
                        if constexpr (KO == 6) {
                            // 6 nibbles of this channel: bytes 3c..3c+2 of the block
                            const uint64_t ov64 = (static_cast<uint64_t>(g_ov[g][1]) << 32) | g_ov[g][0];
                            const uint32_t nib = static_cast<uint32_t>(ov64 >> (8 * ((6 * lane) & 3) + 24 * u)) & 0xFFFFFFu;
                            const f32x2 l01 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 0);
                            const f32x2 l23 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 1);
                            const f32x2 l45 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 2);
                            lv[0] = l01[0]; lv[1] = l01[1]; lv[2] = l23[0]; lv[3] = l23[1]; lv[4] = l45[0]; lv[5] = l45[1];
                        } else {
                            // the lane's bytes start 0 or 2 bytes into the loaded dwords (odd lanes)
                            const uint32_t sh = (lane & 1) ? 16u : 0u;
                            const uint32_t o0 = __builtin_amdgcn_alignbit(g_ov10[g][1], g_ov10[g][0], sh);
                            const uint32_t o1 = __builtin_amdgcn_alignbit(g_ov10[g][2], g_ov10[g][1], sh);
                            const uint32_t o2 = g_ov10[g][2] >> sh;
                            // channel u: nibbles 10u .. 10u+9 = bytes 5u .. 5u+4 of (o0, o1, o2)
#pragma unroll
                            for (int i = 0; i < 5; ++i) {
                                const int byte = 5 * u + i;
                                const uint32_t w = byte < 4 ? o0 : (byte < 8 ? o1 : o2);
                                f32x2 l2;
                                switch (byte & 3) {
                                    case 0: l2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0); break;
                                    case 1: l2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1); break;
                                    case 2: l2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2); break;
                                    default: l2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3); break;
                                }
                                lv[2 * i] = l2[0];
                                lv[2 * i + 1] = l2[1];
                            }
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                ixw[i] = __builtin_amdgcn_alignbit(g_ix10[g][i + 1], g_ix10[g][i], sh);
                            ixw[4] = g_ix10[g][4] >> sh;
                        }
                        // The 2-bit base code of an outlier position is overwritten (in the staged
                        // K row) by 0 or 3, whichever base value is nearer to the outlier, so the
                        // delta left for the tile is small; the bias terms account for the rest.
                        const float thr = 0.375f * s, s34 = 0.75f * s;
                        const uint32_t field = 3u << (2 * (c & 15));
                        const uint32_t kt = sm_lds + OFF_KT + g * 32 * KT_ROW + 4 * (c >> 4);
                        uint16_t* dt = reinterpret_cast<uint16_t*>(sm + OFF_DT) + c;
                        float* lc = reinterpret_cast<float*>(sm + OFF_LC) + g * 32 * HR;
#pragma unroll
                        for (int sidx = 0; sidx < KO; ++sidx) {
                            int pos;
                            if constexpr (KO == 10) {          // 7-bit field at bit 72u + 7s of the window
                                constexpr int PM = GT - 1;
                                const int bit = 72 * u + 7 * sidx;
                                const int wi = bit >> 5, bo = bit & 31;
                                pos = (bo <= 25 ? (ixw[wi] >> bo)
                                                : __builtin_amdgcn_alignbit(ixw[wi < 4 ? wi + 1 : 4], ixw[wi], bo)) & PM;
                            } else if constexpr (IDX == 0) {
                                pos = __builtin_ctz(bm) & 31;           // v_ffbl_b32
                                bm &= bm - 1;
                            } else {                                    // bits [7s, 7s+7) of the stream
                                constexpr int PM = GT - 1;              // (5 bits suffice for 32-token groups)
                                pos = sidx < 4 ? ((ix_lo >> (7 * sidx)) & PM)
                                    : sidx == 4 ? (__builtin_amdgcn_alignbit(ix_hi, ix_lo, 28) & PM)
                                                : ((ix_hi >> 3) & PM);
                            }
                            // a longer group: only the outliers of this 32-token piece
                            bool here = true;
                            if constexpr (GTS > 0) {
                                here = (pos >> 5) == piece;
                                pos &= 31;
                            }
                            const float dl0 = fmaf(lv[sidx], a1, b1);
                            const bool top = dl0 > thr;
                            const float dl = top ? dl0 - s34 : dl0;
                            const _Float16 hi = static_cast<_Float16>(dl);
                            if constexpr (!decltype(RES)::value) {
                                if (here) {
                                    dt[pos * (DT_ROW / 2)] = __builtin_bit_cast(uint16_t, hi);
                                    // K row dword = (dword & ~field) | (top ? field : 0)
                                    asm volatile("ds_mskor_b32 %0, %1, %2"
                                                 :: "v"(kt + pos * KT_ROW), "v"(field), "v"(top ? field : 0u)
                                                 : "memory");
                                    dl_max[u] = fmaxf(dl_max[u], fabsf(dl));
                                }
                            } else {
                                if (here && fabsf(dl) >= big_thr[u]) {
                                    const float lo = dl - static_cast<float>(hi);
#pragma unroll
                                    for (int r = 0; r < HR; ++r)
                                        __hip_atomic_fetch_add(lc + pos * HR + r, lo * q4_at(u, r), __ATOMIC_RELAXED,
                                                               __HIP_MEMORY_SCOPE_WAVEFRONT);
                                }
                            }
                        }
                    }
                };
                walk(std::false_type{}, std::integral_constant<int, 0>{});
                walk(std::false_type{}, std::integral_constant<int, 1>{});
                // (see BIG_DELTA)
                // Channel halves holding a larger delta take the residual walk.
                if (__any(dl_max[0] >= big_thr[0])) walk(std::true_type{}, std::integral_constant<int, 0>{});
                if (__any(dl_max[1] >= big_thr[1])) walk(std::true_type{}, std::integral_constant<int, 1>{});
                lds_fence();
            }
            // this group's parameter registers are free: start the next iteration's loads
            if (more) fetch_params_g(g);
            const u32x4* mg = reinterpret_cast<const u32x4*>(sm + OFF_MAGIC + g * 256 + kq * 64);
            const u32x4 m0 = mg[0], m1 = mg[1], m2 = mg[2], m3 = mg[3];
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const int tb = 2 * g + t2;
                f32x4 d = {0, 0, 0, 0};
                if (OUTLIERS) {   // tile rows of this token block: read, clear, accumulate
                    u32x4* row = reinterpret_cast<u32x4*>(sm + OFF_DT + (16 * t2 + j) * DT_ROW + 64 * kq);
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) {
                        const u32x4 bt = row[ks];
                        row[ks] = u32x4{0, 0, 0, 0};
                        d = mfma_f16(aq_nat[ks], bt, d);
                    }
                }
                const u32x2 kw2 = *reinterpret_cast<const u32x2*>(sm + OFF_KT + (16 * tb + j) * KT_ROW + 8 * kq);
                const uint32_t w0 = kw2[0], w1 = kw2[1];
                d = mfma_bf16(aq_pair[0], u32x4{k_pair<0>(w0, m0[0]), k_pair<1>(w0, m0[1]), k_pair<2>(w0, m0[2]), k_pair<3>(w0, m0[3])}, d);
                d = mfma_bf16(aq_pair[1], u32x4{k_pair<4>(w0, m1[0]), k_pair<5>(w0, m1[1]), k_pair<6>(w0, m1[2]), k_pair<7>(w0, m1[3])}, d);
                d = mfma_bf16(aq_pair[2], u32x4{k_pair<0>(w1, m2[0]), k_pair<1>(w1, m2[1]), k_pair<2>(w1, m2[2]), k_pair<3>(w1, m2[3])}, d);
                d = mfma_bf16(aq_pair[3], u32x4{k_pair<4>(w1, m3[0]), k_pair<5>(w1, m3[1]), k_pair<6>(w1, m3[2]), k_pair<7>(w1, m3[3])}, d);
                dq[tb] = d;
            }
            if (OUTLIERS) lds_fence();        // the tile is zero again before the next scatter
        }
        // bias columns: 0 zp(g0) 1 zp(g1) 2 2^e(g0) 3 2^e(g1); other columns repeat them
        f32x4 dbias = {0, 0, 0, 0};
        {
            const int src = ((j & 2) ? OFF_MAGIC : OFF_ZPP) + (j & 1) * 256 + kq * 64;
            const u32x4* bp = reinterpret_cast<const u32x4*>(sm + src);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) dbias = mfma_bf16(aq_pair[ks], bp[ks], dbias);
        }

        if (more) fetch_tables(n0 + 128);  // after the parameter loads, which used the group slots

        // ---------------------------------------------------------------- softmax
        // bias of (group, head): sum q*zp - sum A*2^e, columns 0..3 of the bias result
        // 4 heads: a lane owns token n0 + lane (block kq) and heads 0..3.
        // 8 heads: a lane owns tokens n0 + lane and n0 + (lane ^ 16) (blocks kq and kq ^ 1, same
        //          K group) and heads 4*hg..4*hg+3.
        constexpr int NT = HR / 4;                  // tokens per lane
        const bool tok_ok2[2] = {tok_ok, n0 + (lane ^ 16) < n_end};
        float logit[NT][4];
        {
            f32x4 dsel[NT];
            dsel[0] = kq == 0 ? dq[0] : (kq == 1 ? dq[1] : (kq == 2 ? dq[2] : dq[3]));
            if constexpr (HR == 8) dsel[1] = kq == 0 ? dq[1] : (kq == 1 ? dq[0] : (kq == 2 ? dq[3] : dq[2]));
            const int gsel = lane >> 5;
            f32x4 corr[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                corr[t] = f32x4{0, 0, 0, 0};
                if (OUTLIERS)
                    corr[t] = *reinterpret_cast<const f32x4*>(
                        sm + OFF_LC + 4 * HR * (t ? (lane ^ 16) : lane) + 16 * hg);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // column gsel (zp) and 2 + gsel (2^e) of the rows that hold this lane's heads
                const float zpv = __shfl(dbias[r], 16 * hg + gsel);
                const float s1v = __shfl(dbias[r], 16 * hg + 2 + gsel);
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    logit[t][r] = (dsel[t][r] + corr[t][r] + (zpv - s1v)) * a.sm_scale;
            }
            if (a.cap > 0.0f) {           // one uniform branch around all the tanh work
                asm volatile("" ::: "memory");      // (keeps it a branch: never computed speculatively)
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) logit[t][r] = apply_cap(logit[t][r], a.cap);
            }
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) logit[t][r] = tok_ok2[t] ? logit[t][r] * c_log2e : -INFINITY;
        }
        float alpha[4], p[NT][4], mxs[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) mxs[r] = HR == 8 ? fmaxf(logit[0][r], logit[NT - 1][r]) : logit[0][r];
        if constexpr (HR == 8) rowpair_max4(mxs); else wave_max4(mxs);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float m_new = fmaxf(m_run[r], mxs[r]);
            alpha[r] = (m_run[r] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run[r] - m_new);
#pragma unroll
            for (int t = 0; t < NT; ++t)
                p[t][r] = tok_ok2[t] ? __builtin_amdgcn_exp2f(logit[t][r] - m_new) : 0.0f;
            m_run[r] = m_new;
        }
        {
            uint16_t* pt = reinterpret_cast<uint16_t*>(sm + OFF_PT);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // accumulate the weight that P.V really uses (the f16-rounded one)
                l_run[r] *= alpha[r];
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const _Float16 ph = static_cast<_Float16>(p[t][r]);
                    l_run[r] += static_cast<float>(ph);
                    pt[(4 * hg + r) * PT_ROW + (t ? (lane ^ 16) : lane)] = __builtin_bit_cast(uint16_t, ph);
                }
            }
        }
        // the running maxima seldom move after the first steps: rescale only when one did
        if (__any(alpha[0] != 1.0f || alpha[1] != 1.0f || alpha[2] != 1.0f || alpha[3] != 1.0f)) {
#pragma unroll
            for (int y = 0; y < 8; ++y)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[y][r] *= alpha[r];
#pragma unroll
            for (int r = 0; r < 4; ++r) accz[r] *= alpha[r];
        }
        lds_fence();

        // ---------------------------------------------------------------- P.V
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (kb == 1 && !g1_live) break;       // their weights are zero
            const int t0 = 32 * kb + 8 * kq;
            const u32x4 pw = *reinterpret_cast<const u32x4*>(sm + OFF_PT + ((j & (HR - 1)) * PT_ROW + t0) * 2);
            // columns 0..3: vz of channel group j, columns 4..7: vs; others repeat
            const u32x4 bz = *reinterpret_cast<const u32x4*>(
                sm + ((j & 4) ? OFF_VS : OFF_VZ) + ((j & 3) * PT_ROW + t0) * 2);
            accz = mfma_f16(pw, bz, accz);
            if constexpr (HR == 4) {
                // row group x = j / 4 carries the scales of channel group x
                const u32x4 sw = *reinterpret_cast<const u32x4*>(sm + OFF_VS + ((j >> 2) * PT_ROW + t0) * 2);
                const u32x4 apv = {pk_mul_f16(pw[0], sw[0]), pk_mul_f16(pw[1], sw[1]),
                                   pk_mul_f16(pw[2], sw[2]), pk_mul_f16(pw[3], sw[3])};
                // V codes: dword column j%8, half j/8, tokens t0..t0+7
                const uint32_t* vt = reinterpret_cast<const uint32_t*>(sm + OFF_VT) + (j & 7) * VT_COL + t0;
                const u32x4 va = *reinterpret_cast<const u32x4*>(vt);
                const u32x4 vb = *reinterpret_cast<const u32x4*>(vt + 4);
                const uint32_t sel = (j & 8) ? 0x07060302u : 0x05040100u;
                const uint32_t mg0 = __builtin_amdgcn_perm(va[1], va[0], sel);
                const uint32_t mg1 = __builtin_amdgcn_perm(va[3], va[2], sel);
                const uint32_t mg2 = __builtin_amdgcn_perm(vb[1], vb[0], sel);
                const uint32_t mg3 = __builtin_amdgcn_perm(vb[3], vb[2], sel);
#define OMMX_PV(Y) acc[Y] = mfma_f16(apv, u32x4{v_pair<Y>(mg0, one2), v_pair<Y>(mg1, one2), v_pair<Y>(mg2, one2), v_pair<Y>(mg3, one2)}, acc[Y]);
                OMMX_PV(0) OMMX_PV(1) OMMX_PV(2) OMMX_PV(3) OMMX_PV(4) OMMX_PV(5) OMMX_PV(6) OMMX_PV(7)
#undef OMMX_PV
            } else {
                // Two row groups only, so the channel groups go in two sets s = 0, 1: row group
                // x = j / 8 carries the scales of channel group 2s + x, and column j reads V
                // dword column 4s + j%4 (whose channel group is 2s + (j%4)/2), byte 2*((j/4)%2) +
                // j/8 of it: four channels per token, taken one per result (acc[4s + y]).
                const uint32_t bsel = 2 * ((j >> 2) & 1) + (j >> 3);
                const uint32_t sel = bsel | 0x0C000C00u | ((4u + bsel) << 16);
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const u32x4 sw = *reinterpret_cast<const u32x4*>(
                        sm + OFF_VS + ((2 * s + (j >> 3)) * PT_ROW + t0) * 2);
                    const u32x4 apv = {pk_mul_f16(pw[0], sw[0]), pk_mul_f16(pw[1], sw[1]),
                                       pk_mul_f16(pw[2], sw[2]), pk_mul_f16(pw[3], sw[3])};
                    const uint32_t* vt = reinterpret_cast<const uint32_t*>(sm + OFF_VT) + (4 * s + (j & 3)) * VT_COL + t0;
                    const u32x4 va = *reinterpret_cast<const u32x4*>(vt);
                    const u32x4 vb = *reinterpret_cast<const u32x4*>(vt + 4);
                    const uint32_t mg0 = __builtin_amdgcn_perm(va[1], va[0], sel);
                    const uint32_t mg1 = __builtin_amdgcn_perm(va[3], va[2], sel);
                    const uint32_t mg2 = __builtin_amdgcn_perm(vb[1], vb[0], sel);
                    const uint32_t mg3 = __builtin_amdgcn_perm(vb[3], vb[2], sel);
#define OMMX_PV(Y) acc[4 * s + Y] = mfma_f16(apv, u32x4{v_pair<Y>(mg0, one2), v_pair<Y>(mg1, one2), v_pair<Y>(mg2, one2), v_pair<Y>(mg3, one2)}, acc[4 * s + Y]);
                    OMMX_PV(0) OMMX_PV(1) OMMX_PV(2) OMMX_PV(3)
#undef OMMX_PV
                }
            }
        }
        lds_fence();
    }

    report_table_range(a.err, bad_id);

    // ---- epilogue: o = (f*(acc - PVS) + PVZ) / l with f = 4 or 16, lse = m + ln l ----------
    float l_tot[4] = {l_run[0], l_run[1], l_run[2], l_run[3]};
    if constexpr (HR == 8) rowpair_sum4(l_tot); else wave_sum4(l_tot);
    if constexpr (HR == 4) {
        const int jg = (j & 7) >> 1;
        float pvz[4], pvs[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            pvz[r] = __shfl(accz[r], jg);          // column jg, rows 0..3 (kq 0)
            pvs[r] = __shfl(accz[r], 4 + jg);
        }
        if (kq == jg) {
            const int ch0 = 16 * (j & 7) + 8 * (j >> 3);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (r >= heads) break;
                float* dst = a.al + b * a.al_b + (int64_t)(qh0 + r) * a.al_h + (int64_t)sp * a.al_s;
                const float inv = l_tot[r] > 0.0f ? __builtin_amdgcn_rcpf(l_tot[r]) : 0.0f;    // 1 ulp
#pragma unroll
                for (int y = 0; y < 8; ++y)
                    dst[ch0 + y] = (((y & 1) ? 4.0f : 16.0f) * (acc[y][r] - pvs[r]) + pvz[r]) * inv;
            }
        }
    } else {
        const int xg = (j & 3) >> 1;               // the row group that is valid in column j
        float pvz[2][4], pvs[2][4];
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int r = 0; r < 4; ++r) {          // columns 2s+xg / 4+2s+xg, rows of this head group
                pvz[s][r] = __shfl(accz[r], 16 * hg + 2 * s + xg);
                pvs[s][r] = __shfl(accz[r], 16 * hg + 4 + 2 * s + xg);
            }
        if ((kq >> 1) == xg) {
            const int bsel = 2 * ((j >> 2) & 1) + (j >> 3);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float* dst = a.al + b * a.al_b + (int64_t)(qh0 + 4 * hg + r) * a.al_h + (int64_t)sp * a.al_s;
                const float inv = l_tot[r] > 0.0f ? __builtin_amdgcn_rcpf(l_tot[r]) : 0.0f;    // 1 ulp
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int ch0 = 16 * (4 * s + (j & 3)) + 4 * bsel;
#pragma unroll
                    for (int y = 0; y < 4; ++y)
                        dst[ch0 + y] = (((y & 1) ? 4.0f : 16.0f) * (acc[4 * s + y][r] - pvs[s][r]) + pvz[s][r]) * inv;
                }
            }
        }
    }
    if (j < 4 && kq < HR / 4 && 4 * kq + j < heads) {     // lane 16*hg + r holds head 4*hg + r
        float* dst = a.al + b * a.al_b + (int64_t)(qh0 + 4 * kq + j) * a.al_h + (int64_t)sp * a.al_s;
        const float lt = j == 0 ? l_tot[0] : (j == 1 ? l_tot[1] : (j == 2 ? l_tot[2] : l_tot[3]));
        const float mt = j == 0 ? m_run[0] : (j == 1 ? m_run[1] : (j == 2 ? m_run[2] : m_run[3]));
        dst[D] = lt > 0.0f ? (mt + log2f(lt)) * 0.6931471805599453f : -INFINITY;
    }
}

}  // namespace

// Returns 0 when launched, 1 when the shape is not covered by the tuned kernel.
int launch_decode_fast(const DecodeArgs& a, int Dh, int R, hipStream_t st) {
    if (Dh != 128 || !(R == 1 || R == 2 || R == 4 || R == 8)) return 1;
    const bool paper = a.kout == 10 && a.gt == 128 && a.idx_repr == 1 && (R == 4 || R == 8);   // 128-token groups, 10 outliers
    if (!(a.kout == 6 || a.kout == 0 || paper)) return 1;
    if (a.scale_bf16) return 1;      // operands are exact only for power-of-two steps
    if (a.v_bf16) return 1;
    // longer K groups (and wider V vectors with them): position streams, 6 outliers, 4 or 8 heads
    const bool longer = a.gt == 64 || a.gt == 128;
    if (longer && !(a.idx_repr == 1 && (a.kout == 6 || paper) && (R == 4 || R == 8) &&
                    (a.gc == 32 || a.gc == 64 || a.gc == 128))) return 1;
    if (!longer && (a.gt != 32 || a.gc != 32)) return 1;
    // the kernel reads q two channels at a time
    if ((reinterpret_cast<uintptr_t>(a.q) & 3) || (a.q_sb & 1) || (a.q_sh & 1)) return 1;
    const int waves = (a.Hkv % 4 == 0) ? 4 : ((a.Hkv % 2 == 0) ? 2 : 1);    // one wave per kv head
    const dim3 grid(a.S, a.Hkv / waves, a.B), block(64 * waves);
    const size_t shm = (size_t)waves * (R <= 4 ? (a.kout > 0 ? LdsMap<4>::END : LdsMap<4>::DT)
                                               : (a.kout > 0 ? LdsMap<8>::END : LdsMap<8>::DT));
    const bool own_map = a.k_ms != nullptr;
#define OMMX_LAUNCH(HR, IDX, MAP)                                                                          \
    do {                                                                                                   \
        if (a.B == 1)                                                                                      \
            hipLaunchKernelGGL((decode_splitkv_mfma_kernel<true, HR, IDX, MAP, false, 0, 6, 0>), grid,     \
                               block, shm, st, a);                                                         \
        else if (a.B > 64 && a.B <= 256)                                                                   \
            hipLaunchKernelGGL((decode_splitkv_mfma_kernel<true, HR, IDX, MAP, false, 0, 6, 2>), grid,     \
                               block, shm, st, a);                                                         \
        else                                                                                               \
            hipLaunchKernelGGL((decode_splitkv_mfma_kernel<true, HR, IDX, MAP>), grid, block, shm, st, a); \
    } while (0)
#define OMMX_LAUNCH_PARTIAL(IDX, MAP) \
    hipLaunchKernelGGL((decode_splitkv_mfma_kernel<true, 4, IDX, MAP, true>), grid, block, shm, st, a)
#define OMMX_LAUNCH_LONG(HR, MAP, GTS) \
    hipLaunchKernelGGL((decode_splitkv_mfma_kernel<true, HR, 1, MAP, false, GTS>), grid, block, shm, st, a)
#define OMMX_LAUNCH_PAPER(HR, MAP) \
    hipLaunchKernelGGL((decode_splitkv_mfma_kernel<true, HR, 1, MAP, false, 2, 10>), grid, block, shm, st, a)
    if (paper) {
        switch ((R == 8 ? 2 : 0) | (own_map ? 1 : 0)) {
            case 0: OMMX_LAUNCH_PAPER(4, false); break;
            case 1: OMMX_LAUNCH_PAPER(4, true); break;
            case 2: OMMX_LAUNCH_PAPER(8, false); break;
            default: OMMX_LAUNCH_PAPER(8, true); break;
        }
    } else if (longer) {
        switch ((R == 8 ? 4 : 0) | (a.gt == 128 ? 2 : 0) | (own_map ? 1 : 0)) {
            case 0: OMMX_LAUNCH_LONG(4, false, 1); break;
            case 1: OMMX_LAUNCH_LONG(4, true, 1); break;
            case 2: OMMX_LAUNCH_LONG(4, false, 2); break;
            case 3: OMMX_LAUNCH_LONG(4, true, 2); break;
            case 4: OMMX_LAUNCH_LONG(8, false, 1); break;
            case 5: OMMX_LAUNCH_LONG(8, true, 1); break;
            case 6: OMMX_LAUNCH_LONG(8, false, 2); break;
            default: OMMX_LAUNCH_LONG(8, true, 2); break;
        }
    } else if (a.kout == 6 && R < 4) {
        switch ((a.idx_repr ? 2 : 0) | (own_map ? 1 : 0)) {
            case 0: OMMX_LAUNCH_PARTIAL(0, false); break;
            case 1: OMMX_LAUNCH_PARTIAL(0, true); break;
            case 2: OMMX_LAUNCH_PARTIAL(1, false); break;
            default: OMMX_LAUNCH_PARTIAL(1, true); break;
        }
    } else if (a.kout == 6) {
        const int variant = (R == 8 ? 4 : 0) | (a.idx_repr ? 2 : 0) | (own_map ? 1 : 0);
        switch (variant) {
            case 0: OMMX_LAUNCH(4, 0, false); break;
            case 1: OMMX_LAUNCH(4, 0, true); break;
            case 2: OMMX_LAUNCH(4, 1, false); break;
            case 3: OMMX_LAUNCH(4, 1, true); break;
            case 4: OMMX_LAUNCH(8, 0, false); break;
            case 5: OMMX_LAUNCH(8, 0, true); break;
            case 6: OMMX_LAUNCH(8, 1, false); break;
            default: OMMX_LAUNCH(8, 1, true); break;
        }
    } else if (R < 4) {
        hipLaunchKernelGGL((decode_splitkv_mfma_kernel<false, 4, 0, true, true>), grid, block, shm, st, a);
    } else if (R == 4) {
        hipLaunchKernelGGL((decode_splitkv_mfma_kernel<false, 4, 0, true>), grid, block, shm, st, a);
    } else {
        hipLaunchKernelGGL((decode_splitkv_mfma_kernel<false, 8, 0, true>), grid, block, shm, st, a);
    }
#undef OMMX_LAUNCH
#undef OMMX_LAUNCH_PARTIAL
#undef OMMX_LAUNCH_LONG
#undef OMMX_LAUNCH_PAPER
    return 0;
}

}  // namespace ommx

// Quantize-on-store for every recipe the tuned 32x32 kernel does not cover: K vectors of
// 16 / 32 / 64 / 128 tokens, V vectors of 16 / 32 / 64 / 128 channels, up to 16 outliers per
// K vector, either index plane, either outlier map, every step mode.  Same arithmetic and the
// same planes as ommx_gpu_serve/attention/pack.py:419-623, written for generality: one
// workgroup of D threads packs one (K group, kv head).
//   K: thread d owns "channel d over the GT tokens of the group".
//   V: the group's GT * D / GC vectors "token t, channels GC*j .. GC*j+GC-1" are dealt to the
//      threads round-robin.
// K codes cross from channel-major to token-major through an LDS tile.
#include "ommx_store_common.h"

namespace ommx {
namespace {

constexpr int MAX_OUT = 16;             // outliers per vector this kernel can index

template <bool F32>
__device__ __forceinline__ float load_any(const void* base, int64_t idx) {
    if (F32) return static_cast<const float*>(base)[idx];
    return bf16_to_f32(static_cast<const uint16_t*>(base)[idx]);
}

template <bool F32, int GT, int GC>
__global__ void __launch_bounds__(256) store_generic_kernel(StoreArgs a) {
    constexpr int MW = (GT + 31) / 32;              // 32-bit words of a lane mask
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int D = a.D, H = a.H;
    uint8_t* s_codes = smem;                        // [GT][D] one code per byte
    uint8_t* s_oval = smem + GT * D;                // [D][nval]
    uint8_t* s_oidx = s_oval + 8 * D;               // [D][nidx]
    const int g = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int kout = a.kout;
    const int nval = (kout + 1) >> 1;
    const int nidx = kout == 0 ? 0 : (a.idx_repr == 0 ? (GT + 7) / 8 : (7 * kout + 7) / 8);
    const int64_t gs = a.dst_groups ? a.dst_groups[g] : g;
    const float* __restrict__ tab = a.table;
    int err = 0;

    // ------------------------------------------------------------------ K vector
    {
        const int d = tid;
        float w[GT];
        bool fin = true;
#pragma unroll
        for (int i = 0; i < GT; ++i) {
            const int64_t row = a.src_rows ? a.src_rows[g * GT + i] : (int64_t)g * GT + i;
            w[i] = load_any<F32>(a.K, row * a.k_ts + (int64_t)h * a.k_hs + d);
            fin = fin && is_finite_f32(w[i]);
        }
        if (!fin) err |= OMMX_ERR_NONFINITE_K;

        // outlier mask (pack.py:436-448); ties go to the lower position
        uint32_t om[MW];
#pragma unroll
        for (int m = 0; m < MW; ++m) om[m] = 0;
        auto taken = [&](const uint32_t (&msk)[MW], int i) { return (msk[i >> 5] >> (i & 31)) & 1u; };
        if (a.select_abs) {
            for (int r = 0; r < kout; ++r) {
                float best = 0.0f; int bi = -1;
#pragma unroll
                for (int i = 0; i < GT; ++i)
                    if (!taken(om, i) && (bi < 0 || fabsf(w[i]) > best)) { best = fabsf(w[i]); bi = i; }
                if (bi >= 0) om[bi >> 5] |= 1u << (bi & 31);
            }
        } else {
            const int kt = (kout + 1) >> 1, kb = kout - kt;
            uint32_t top[MW], bot[MW];
#pragma unroll
            for (int m = 0; m < MW; ++m) top[m] = bot[m] = 0;
            for (int r = 0; r < kt; ++r) {
                float best = 0.0f; int bi = -1;
#pragma unroll
                for (int i = 0; i < GT; ++i)
                    if (!taken(top, i) && (bi < 0 || w[i] > best)) { best = w[i]; bi = i; }
                if (bi >= 0) top[bi >> 5] |= 1u << (bi & 31);
            }
            for (int r = 0; r < kb; ++r) {     // smallest of the rest, chosen lanes read +1e9
                float best = 0.0f; int bi = -1;
#pragma unroll
                for (int i = 0; i < GT; ++i) {
                    const float v = taken(top, i) ? 1e9f : w[i];
                    if (!taken(bot, i) && (bi < 0 || v < best)) { best = v; bi = i; }
                }
                if (bi >= 0) bot[bi >> 5] |= 1u << (bi & 31);
            }
#pragma unroll
            for (int m = 0; m < MW; ++m) om[m] = top[m] | bot[m];
        }
        int npicked = 0;
#pragma unroll
        for (int m = 0; m < MW; ++m) npicked += __popc(om[m]);
        if (npicked != kout) err |= OMMX_ERR_UNDERFILLED;

        // affine base over the other lanes (pack.py:455-465)
        float mn = 1e9f, mx = -1e9f, omn = 1e9f, omx = -1e9f;
#pragma unroll
        for (int i = 0; i < GT; ++i) {
            const bool o = taken(om, i);
            mn = fminf(mn, o ? 1e9f : w[i]);
            mx = fmaxf(mx, o ? -1e9f : w[i]);
            omn = fminf(omn, o ? w[i] : 1e9f);
            omx = fmaxf(omx, o ? w[i] : -1e9f);
        }
        if (mn > 1e8f) mn = 0.0f;
        if (mx < -1e8f) mx = 0.0f;
        if (omn > 1e8f) omn = 0.0f;
        if (omx < -1e8f) omx = 0.0f;
        const Step st = make_step(__fdiv_rn(fmaxf(mx - mn, 1e-8f), 3.0f), a.scale_mode, tab);
        if (!st.in_range) err |= OMMX_ERR_EXP_RANGE;
        if (st.e > 15) err |= OMMX_NOTE_WIDE_STEP;      // beyond the f16 operands of the matrix-core decode
        const uint16_t zp_b = f32_to_bf16_rne(mn);
        const float zp = bf16_to_f32(zp_b);

        // outlier code space: own map (pack.py:486-498) or the base step (pack.py:502-506)
        const bool own_map = a.k_ms != nullptr;
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
        uint64_t nib = 0;                   // nibble s = FP4 code of the s-th outlier position
        uint64_t stream[2] = {0, 0};        // relidx7: position s at bits [7s, 7s+7)
        int slot = 0;
        bool mfin = true;
#pragma unroll
        for (int i = 0; i < GT; ++i) {
            s_codes[i * D + d] = static_cast<uint8_t>(int2_code(w[i] - zp, st.scale, st.inv, st.inv_ok));
            if (kout > 0) {
                const float mapped = own_map ? (w[i] - mc) * ms
                                             : (st.inv_ok ? (w[i] - zp) * st.inv : __fdiv_rn(w[i] - zp, st.scale));
                mfin = mfin && is_finite_f32(mapped);
                if (taken(om, i)) {
                    nib |= static_cast<uint64_t>(fp4_encode(mapped, tab + 256)) << (4 * slot);
                    const int bit = 7 * slot;
                    stream[bit >> 6] |= static_cast<uint64_t>(i) << (bit & 63);
                    if ((bit & 63) > 57) stream[1] |= static_cast<uint64_t>(i) >> (64 - (bit & 63));
                    ++slot;
                }
            }
        }
        if (!mfin) err |= OMMX_ERR_NONFINITE_K;

        const int64_t gidx = (gs * H + h) * D + d;
        if (a.scale_mode == 0) a.k_scale[gidx] = static_cast<int8_t>(st.e);
        else reinterpret_cast<uint16_t*>(a.k_scale)[gidx] = st.bits;
        a.k_zp[gidx] = zp_b;
        if (kout > 0) {
            if (own_map) { a.k_ms[gidx] = ms_b; a.k_mc[gidx] = mc_b; }
            for (int b = 0; b < nval; ++b) s_oval[d * nval + b] = static_cast<uint8_t>(nib >> (8 * b));
            if (a.idx_repr == 0) {          // position p -> byte p >> 3, bit p & 7
                for (int b = 0; b < nidx; ++b)
                    s_oidx[d * nidx + b] = static_cast<uint8_t>(om[b >> 2] >> (8 * (b & 3)));
            } else {
                for (int b = 0; b < nidx; ++b)
                    s_oidx[d * nidx + b] = static_cast<uint8_t>(stream[b >> 3] >> (8 * (b & 7)));
            }
        }
    }
    __syncthreads();

    if (kout > 0) {     // D frames of nval / nidx bytes each, contiguous in memory: whole dwords
        const int64_t obase = (gs * H + h) * (int64_t)D * nval;
        for (int wd = tid; wd < D * nval / 4; wd += D)
            reinterpret_cast<uint32_t*>(a.k_oval + obase)[wd] = reinterpret_cast<const uint32_t*>(s_oval)[wd];
        const int64_t ibase = (gs * H + h) * (int64_t)D * nidx;
        for (int wd = tid; wd < D * nidx / 4; wd += D)
            reinterpret_cast<uint32_t*>(a.k_obmp + ibase)[wd] = reinterpret_cast<const uint32_t*>(s_oidx)[wd];
    }

    auto phys_row = [&](int tok) {
        const int lp = tok / a.ps;
        const int64_t page = a.dst_pages ? a.dst_pages[lp] : lp;
        return page * a.ps + (tok % a.ps);
    };

    // ------------------------------------------------- k_base rows: 8 bytes = 32 channels a piece
    const int pieces = D / 32;
    for (int it = tid; it < GT * pieces; it += D) {
        const int t = it / pieces, j = it % pieces;
        const int64_t prow = phys_row(g * GT + t);
        uint64_t kb8 = 0;
        const uint8_t* cr = s_codes + t * D + 32 * j;
#pragma unroll
        for (int c = 0; c < 32; ++c) kb8 |= static_cast<uint64_t>(cr[c] & 3u) << (2 * c);
        reinterpret_cast<uint64_t*>(a.k_base)[(prow * H + h) * pieces + j] = kb8;
    }

    // ------------------------------------------------- V vectors (pack.py:604-623)
    const int ngv = D / GC;
    for (int it = tid; it < GT * ngv; it += D) {
        const int t = it / ngv, j = it % ngv;
        const int tok = g * GT + t;
        const int64_t prow = phys_row(tok);
        const int64_t row = a.src_rows ? a.src_rows[tok] : tok;
        const int64_t vbase = row * a.v_ts + (int64_t)h * a.v_hs + GC * j;
        if (a.v_bf16) {     // the row itself, rounded to bf16; the step planes are placeholders
            uint16_t* dst16 = reinterpret_cast<uint16_t*>(a.v_main) + (prow * H + h) * (int64_t)D + GC * j;
#pragma unroll
            for (int c = 0; c < GC; ++c) {
                if (F32) dst16[c] = f32_to_bf16_any(static_cast<const float*>(a.V)[vbase + c]);
                else dst16[c] = static_cast<const uint16_t*>(a.V)[vbase + c];
            }
            const int64_t vidx = (prow * H + h) * ngv + j;
            if (a.scale_mode == 0) a.v_scale[vidx] = 1;
            else reinterpret_cast<uint16_t*>(a.v_scale)[vidx] = 0x3F80;     // bf16 1.0
            a.v_zp[vidx] = 0;
            continue;
        }
        float v[GC];
        bool fin = true;
        float mn = 0.0f, mx = 0.0f;
#pragma unroll
        for (int c = 0; c < GC; ++c) {
            v[c] = load_any<F32>(a.V, vbase + c);
            fin = fin && is_finite_f32(v[c]);
            mn = c == 0 ? v[c] : fminf(mn, v[c]);
            mx = c == 0 ? v[c] : fmaxf(mx, v[c]);
        }
        if (!fin) err |= OMMX_ERR_NONFINITE_V;
        const Step st = make_step(__fdiv_rn(fmaxf(mx - mn, 1e-8f), 3.0f), a.scale_mode, tab);
        if (!st.in_range) err |= OMMX_ERR_EXP_RANGE;
        if (st.e > 15) err |= OMMX_NOTE_WIDE_STEP;
        const uint16_t zp_b = f32_to_bf16_rne(mn);
        const float zp = bf16_to_f32(zp_b);
        uint32_t* dst = reinterpret_cast<uint32_t*>(a.v_main + (prow * H + h) * (D / 4) + j * (GC / 4));
#pragma unroll
        for (int wd = 0; wd < GC / 16; ++wd) {
            uint32_t bits = 0;
#pragma unroll
            for (int c = 0; c < 16; ++c)
                bits |= int2_code(v[16 * wd + c] - zp, st.scale, st.inv, st.inv_ok) << (2 * c);
            dst[wd] = bits;
        }
        const int64_t vidx = (prow * H + h) * ngv + j;
        if (a.scale_mode == 0) a.v_scale[vidx] = static_cast<int8_t>(st.e);
        else reinterpret_cast<uint16_t*>(a.v_scale)[vidx] = st.bits;
        a.v_zp[vidx] = zp_b;
    }
    if (err && a.err) atomicOr(a.err, err);
}

template <bool F32, int GT>
int launch_gt(const StoreArgs& a, int T, hipStream_t st) {
    const dim3 grid(T / GT, a.H), block(a.D);
    const size_t shm = (size_t)GT * a.D + 8 * (size_t)a.D + 16 * (size_t)a.D;
    switch (a.gc) {
        case 16: hipLaunchKernelGGL((store_generic_kernel<F32, GT, 16>), grid, block, shm, st, a); return 0;
        case 32: hipLaunchKernelGGL((store_generic_kernel<F32, GT, 32>), grid, block, shm, st, a); return 0;
        case 64: hipLaunchKernelGGL((store_generic_kernel<F32, GT, 64>), grid, block, shm, st, a); return 0;
        case 128: hipLaunchKernelGGL((store_generic_kernel<F32, GT, 128>), grid, block, shm, st, a); return 0;
    }
    return -1;
}

template <bool F32>
int launch_f(const StoreArgs& a, int T, hipStream_t st) {
    switch (a.gt) {
        case 16: return launch_gt<F32, 16>(a, T, st);
        case 32: return launch_gt<F32, 32>(a, T, st);
        case 64: return launch_gt<F32, 64>(a, T, st);
        case 128: return launch_gt<F32, 128>(a, T, st);
    }
    return -1;
}

}  // namespace

int launch_store_generic(const StoreArgs& a, int T, int in_dtype, hipStream_t st) {
    if (a.kout > MAX_OUT || a.kout > a.gt) return -1;
    return in_dtype == 1 ? launch_f<true>(a, T, st) : launch_f<false>(a, T, st);
}

}  // namespace ommx

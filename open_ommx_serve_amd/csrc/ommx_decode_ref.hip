// Split-KV decode, plain fp32 variant: dequantise one 32-token K group into LDS, splice
// the FP4 outliers, attend, accumulate P.V from the INT2 V rows.  One workgroup per
// (request, kv head, split); 256 threads.  This is the straightforward formulation of
// ommx_gpu_serve/attention/paged_decode.py:1657-2284 (production branch), used as the
// on-device cross-check of the tuned kernel and for head shapes the tuned kernel does
// not cover.
#include "ommx_decode_args.h"

namespace ommx {

template <int D, int R>
__global__ void __launch_bounds__(256) decode_splitkv_ref_kernel(DecodeArgs a) {
    constexpr int KS = D + 4;             // padded K row
    constexpr int TPD = 8 / R;            // threads per (q head, token) dot product
    constexpr int SEG = D / TPD;
    constexpr int BC = D / 4;             // V byte columns
    constexpr int TS = 256 / BC;          // token slices in the P.V phase
    constexpr int TPS = 32 / TS;          // tokens per slice
    extern __shared__ float sm[];
    float* s_K = sm;                      // [32][KS]   (reused for the final reduction)
    float* s_q = s_K + (32 * KS > TS * R * D ? 32 * KS : TS * R * D);   // [R][D]
    float* s_sc = s_q + R * D;            // [2][D]  (two K groups per tile when groups are 16 tokens)
    float* s_zp = s_sc + 2 * D;           // [2][D]
    float* s_p = s_zp + 2 * D;            // [R][32]
    float* s_al = s_p + R * 32;           // [R]
    int64_t* s_row = reinterpret_cast<int64_t*>(s_al + 8);   // [32]

    const int b = blockIdx.x, kvh = blockIdx.y, sp = blockIdx.z, tid = threadIdx.x;
    const int L = max(a.seq[b], 0);      // a negative length: nothing packed, reported
    if (a.seq[b] < 0 && a.err && tid == 0) atomicOr(a.err, OMMX_ERR_TABLE_RANGE);
    const int per = ((((L + a.S - 1) / a.S) + a.gt - 1) / a.gt) * a.gt;      // paged_decode.py:1429-1430
    const int n_begin = per * sp;
    const int n_end = min(n_begin + per, L);

    for (int i = tid; i < R * D; i += 256) {
        const int r = i / D, d = i % D;
        s_q[i] = bf16_to_f32(a.q[b * a.q_sb + (int64_t)(kvh * R + r) * a.q_sh + d]);
    }

    float acc[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;       // live in threads tid < 32*R

    const int gt = a.gt;                          // tokens per K group: 16, 32, 64 or 128
    const int ngv = D / a.gc;                     // V vectors per token
    for (int n0 = n_begin; n0 < n_end; n0 += 32) {
        // A tile is 32 tokens.  With 16-token groups it spans two K groups (sub-group u = t / 16),
        // otherwise it lies inside one (n0 is a multiple of 32 and so is the group size).
        const int nsub = gt == 16 ? 2 : 1;
        const int g_first = n0 / gt;
        int64_t gidx_u[2] = {0, 0};
        for (int u = 0; u < nsub; ++u) {
            const int gi = min(g_first + u, (n_end - 1) / gt);
            int64_t gslot = table_at(a.rg, b * a.rg_s + a.gbase + gi, a.i64);
            if (a.n_gslots > 0 && (gslot < 0 || gslot >= a.n_gslots)) {      // held inside the plane, reported
                gslot = gslot < 0 ? 0 : a.n_gslots - 1;
                if (a.err && tid == 0) atomicOr(a.err, OMMX_ERR_TABLE_RANGE);
            }
            gidx_u[u] = (gslot * a.Hkv + kvh) * D;
        }
        for (int i = tid; i < nsub * D; i += 256) {
            const int u = i / D, d = i % D;
            s_sc[i] = a.scale_bf16
                ? bf16_to_f32(reinterpret_cast<const uint16_t*>(a.k_scale)[gidx_u[u] + d])
                : __uint_as_float(static_cast<uint32_t>(a.k_scale[gidx_u[u] + d] + 127) << 23);
            s_zp[i] = bf16_to_f32(a.k_zp[gidx_u[u] + d]);
        }
        if (tid < 32) {
            const int n = n0 + tid;
            int64_t prow = 0;
            if (n < n_end) {
                const int64_t p = (int64_t)n + (int64_t)a.gbase * gt + a.off;
                int64_t page = table_at(a.rt, b * a.rt_s + p / a.ps, a.i64);
                if (a.n_pages > 0 && (page < 0 || page >= a.n_pages)) {
                    page = page < 0 ? 0 : a.n_pages - 1;
                    if (a.err) atomicOr(a.err, OMMX_ERR_TABLE_RANGE);
                }
                prow = page * a.ps + p % a.ps;
            }
            s_row[tid] = prow;
        }
        __syncthreads();

        {   // base dequant: thread (token t, slice c of D/8 channels)
            const int t = tid >> 3, c = tid & 7;
            const int u = gt == 16 ? (t >> 4) : 0;
            constexpr int NB = D / 32;            // bytes per thread
            const uint8_t* src = a.k_base + (s_row[t] * a.Hkv + kvh) * (D / 4) + c * NB;
            uint32_t bits = 0;
#pragma unroll
            for (int j = 0; j < NB; ++j) bits |= static_cast<uint32_t>(src[j]) << (8 * j);
#pragma unroll
            for (int j = 0; j < 4 * NB; ++j) {
                const int d = c * 4 * NB + j;
                const float code = static_cast<float>((bits >> (2 * j)) & 3u);
                s_K[t * KS + d] = code * s_sc[u * D + d] + s_zp[u * D + d];
            }
        }
        __syncthreads();

        if (a.kout > 0 && tid < D) {   // outlier splice: thread = channel
            const int nval = (a.kout + 1) >> 1;
            const int nidx = a.idx_repr == 0 ? (gt + 7) / 8 : relidx7_bytes(a.kout);
            const bool own_map = a.k_ms != nullptr;
            for (int u = 0; u < nsub; ++u) {
                if ((g_first + u) * gt >= n_end) break;
                const int64_t fr = gidx_u[u] + tid;
                // tile-local index of group position 0 (negative when the group began before the tile)
                const int base = (g_first + u) * gt - n0;
                const uint8_t* ip = a.k_obmp + fr * nidx;
                const uint8_t* ov = a.k_oval + fr * nval;
                // dedicated map: level / map_scale + centre; else the base scale and zero point
                const float ms = own_map ? bf16_to_f32(a.k_ms[fr]) : 0.0f;
                const float mc = own_map ? bf16_to_f32(a.k_mc[fr]) : 0.0f;
                int byte_i = 0, bit0 = 0;           // bitmap walk state: next byte, bit offset of the current one
                uint32_t cur = 0;
                for (int sl = 0; sl < a.kout; ++sl) {
                    int pos;
                    if (a.idx_repr == 0) {          // next set bit, ascending
                        while (cur == 0 && byte_i < nidx) { cur = ip[byte_i]; bit0 = 8 * byte_i; ++byte_i; }
                        if (cur == 0) break;
                        pos = bit0 + __ffs(cur) - 1;
                        cur &= cur - 1;
                    } else {                        // 7-bit field sl of the stream
                        const int bit = 7 * sl;
                        const uint32_t two = static_cast<uint32_t>(ip[bit >> 3]) |
                            ((bit >> 3) + 1 < nidx ? static_cast<uint32_t>(ip[(bit >> 3) + 1]) << 8 : 0u);
                        pos = (two >> (bit & 7)) & 127;
                    }
                    const uint32_t code = (ov[sl >> 1] >> (4 * (sl & 1))) & 0xFu;
                    const int tl = base + pos;
                    if (tl < 0 || tl >= 32) continue;
                    float lvl = fp4_level(code & 7u);
                    if (code & 8u) lvl = -lvl;
                    s_K[tl * KS + tid] = own_map ? __fdiv_rn(lvl, ms) + mc
                                                 : lvl * s_sc[u * D + tid] + s_zp[u * D + tid];
                }
            }
        }
        __syncthreads();

        {   // logits: thread (dot = (r, t), part)
            const int dot = tid / TPD, part = tid % TPD;
            const int r = dot >> 5, t = dot & 31;
            const float* kr = s_K + t * KS + part * SEG;
            const float* qr = s_q + r * D + part * SEG;
            float s = 0.0f;
#pragma unroll 8
            for (int i = 0; i < SEG; ++i) s = fmaf(qr[i], kr[i], s);
#pragma unroll
            for (int o = 1; o < TPD; o <<= 1) s += __shfl_xor(s, o);
            if (part == 0) {
                s = apply_cap(s * a.sm_scale, a.cap);
                s_p[r * 32 + t] = (n0 + t < n_end) ? s : -INFINITY;
            }
        }
        __syncthreads();

        if (tid < 32 * R) {   // online softmax: thread (r, t); 32-lane groups
            const int r = tid >> 5;
            const float s = s_p[tid];
            float mx = s;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            const float m_new = fmaxf(m_run, mx);
            const float p = (s == -INFINITY) ? 0.0f : __expf(s - m_new);
            float ps = p;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) ps += __shfl_xor(ps, o);
            const float alpha = (m_run == -INFINITY) ? 0.0f : __expf(m_run - m_new);
            l_run = l_run * alpha + ps;
            m_run = m_new;
            s_p[tid] = p;
            if ((tid & 31) == 0) s_al[r] = alpha;
        }
        __syncthreads();

        {   // P.V: thread (byte column bc = 4 channels, token slice ts)
            const int bc = tid % BC, ts = tid / BC;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float al = s_al[r];
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[r][c] *= al;
            }
#pragma unroll
            for (int i = 0; i < TPS; ++i) {
                const int t = ts * TPS + i;
                if (n0 + t < n_end) {
                    const int64_t rowh = s_row[t] * a.Hkv + kvh;
                    if (a.v_bf16) {                 // the rows as they are
                        const uint16_t* vr = reinterpret_cast<const uint16_t*>(a.v_main) + rowh * D + bc * 4;
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            const float p = s_p[r * 32 + t];
#pragma unroll
                            for (int c = 0; c < 4; ++c) acc[r][c] = fmaf(p, bf16_to_f32(vr[c]), acc[r][c]);
                        }
                        continue;
                    }
                    const uint32_t byte = a.v_main[rowh * (D / 4) + bc];
                    const int64_t vg = rowh * ngv + (bc * 4) / a.gc;
                    const float vs = a.scale_bf16
                        ? bf16_to_f32(reinterpret_cast<const uint16_t*>(a.v_scale)[vg])
                        : __uint_as_float(static_cast<uint32_t>(a.v_scale[vg] + 127) << 23);
                    const float vz = bf16_to_f32(a.v_zp[vg]);
                    float v[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        v[c] = static_cast<float>((byte >> (2 * c)) & 3u) * vs + vz;
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const float p = s_p[r * 32 + t];
#pragma unroll
                        for (int c = 0; c < 4; ++c) acc[r][c] = fmaf(p, v[c], acc[r][c]);
                    }
                }
            }
        }
        __syncthreads();
    }

    // reduce the token slices, normalise, write the partial state
    {
        const int bc = tid % BC, ts = tid / BC;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) s_K[(ts * R + r) * D + bc * 4 + c] = acc[r][c];
        if (tid < 32 * R && (tid & 31) == 0) { s_p[tid >> 5] = m_run; s_p[8 + (tid >> 5)] = l_run; }
    }
    __syncthreads();
    for (int i = tid; i < R * D; i += 256) {
        const int r = i / D, d = i % D;
        float s = 0.0f;
#pragma unroll
        for (int ts = 0; ts < TS; ++ts) s += s_K[(ts * R + r) * D + d];
        const float l = s_p[8 + r];
        float* dst = a.al + b * a.al_b + (int64_t)(kvh * R + r) * a.al_h + (int64_t)sp * a.al_s;
        dst[d] = l > 0.0f ? s / l : 0.0f;
        if (d == 0) dst[D] = l > 0.0f ? s_p[r] + __logf(l) : -INFINITY;
    }
}

template <int D, int R>
static void launch_ref(const DecodeArgs& a, hipStream_t st) {
    constexpr int KS = D + 4;
    constexpr int TS = 256 / (D / 4);
    constexpr int big = 32 * KS > TS * R * D ? 32 * KS : TS * R * D;
    const size_t shm = sizeof(float) * (big + R * D + 4 * D + R * 32 + 8) + sizeof(int64_t) * 32;
    hipLaunchKernelGGL((decode_splitkv_ref_kernel<D, R>), dim3(a.B, a.Hkv, a.S), dim3(256), shm, st, a);
}

int launch_decode_ref(const DecodeArgs& a, int D, int R, hipStream_t st) {
#define OMMX_CASE(d, r) if (D == d && R == r) { launch_ref<d, r>(a, st); return 0; }
    OMMX_CASE(128, 1) OMMX_CASE(128, 2) OMMX_CASE(128, 4) OMMX_CASE(128, 8)
    OMMX_CASE(64, 1) OMMX_CASE(64, 2) OMMX_CASE(64, 4) OMMX_CASE(64, 8)
#undef OMMX_CASE
    return -1;
}

}  // namespace ommx

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
    float* s_sc = s_q + R * D;            // [D]
    float* s_zp = s_sc + D;               // [D]
    float* s_p = s_zp + D;                // [R][32]
    float* s_al = s_p + R * 32;           // [R]
    int64_t* s_row = reinterpret_cast<int64_t*>(s_al + 8);   // [32]

    const int b = blockIdx.x, kvh = blockIdx.y, sp = blockIdx.z, tid = threadIdx.x;
    const int L = a.seq[b];
    const int per = ((((L + a.S - 1) / a.S) + 31) / 32) * 32;
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

    for (int n0 = n_begin; n0 < n_end; n0 += 32) {
        const int64_t gslot = table_at(a.rg, b * a.rg_s + a.gbase + n0 / 32, a.i64);
        const int64_t gidx0 = (gslot * a.Hkv + kvh) * D;
        if (tid < D) {
            s_sc[tid] = a.scale_bf16
                ? bf16_to_f32(reinterpret_cast<const uint16_t*>(a.k_scale)[gidx0 + tid])
                : __uint_as_float(static_cast<uint32_t>(a.k_scale[gidx0 + tid] + 127) << 23);
            s_zp[tid] = bf16_to_f32(a.k_zp[gidx0 + tid]);
        }
        if (tid < 32) {
            const int n = n0 + tid;
            int64_t prow = 0;
            if (n < n_end) {
                const int64_t p = (int64_t)n + (int64_t)a.gbase * 32 + a.off;
                prow = table_at(a.rt, b * a.rt_s + p / a.ps, a.i64) * a.ps + p % a.ps;
            }
            s_row[tid] = prow;
        }
        __syncthreads();

        {   // base dequant: thread (token t, slice c of D/8 channels)
            const int t = tid >> 3, c = tid & 7;
            constexpr int NB = D / 32;            // bytes per thread
            const uint8_t* src = a.k_base + (s_row[t] * a.Hkv + kvh) * (D / 4) + c * NB;
            uint32_t bits = 0;
#pragma unroll
            for (int j = 0; j < NB; ++j) bits |= static_cast<uint32_t>(src[j]) << (8 * j);
#pragma unroll
            for (int j = 0; j < 4 * NB; ++j) {
                const int d = c * 4 * NB + j;
                const float code = static_cast<float>((bits >> (2 * j)) & 3u);
                s_K[t * KS + d] = code * s_sc[d] + s_zp[d];
            }
        }
        __syncthreads();

        if (a.kout > 0 && tid < D) {   // outlier splice: thread = channel
            const int nval = (a.kout + 1) >> 1;
            uint32_t bm = 0;
            if (a.idx_repr == 0) {
                bm = reinterpret_cast<const uint32_t*>(a.k_obmp)[gidx0 + tid];
            } else {               // 7-bit position stream -> the same occupancy mask
                const int nidx = relidx7_bytes(a.kout);
                const uint8_t* ip = a.k_obmp + (gidx0 + tid) * nidx;
                uint64_t stream = 0;
                for (int j = 0; j < nidx; ++j) stream |= static_cast<uint64_t>(ip[j]) << (8 * j);
                for (int s = 0; s < a.kout; ++s) bm |= 1u << ((stream >> (7 * s)) & 31u);
            }
            const uint8_t* ov = a.k_oval + (gidx0 + tid) * nval;
            uint32_t nib = 0;
            for (int j = 0; j < nval; ++j) nib |= static_cast<uint32_t>(ov[j]) << (8 * j);
            // dedicated map: level / map_scale + centre; else the base scale and zero point
            const bool own_map = a.k_ms != nullptr;
            const float ms = own_map ? bf16_to_f32(a.k_ms[gidx0 + tid]) : 0.0f;
            const float mc = own_map ? bf16_to_f32(a.k_mc[gidx0 + tid]) : 0.0f;
            while (bm) {
                const int pos = __ffs(bm) - 1;
                bm &= bm - 1;
                float lvl = fp4_level(nib & 7u);
                if (nib & 8u) lvl = -lvl;
                nib >>= 4;
                s_K[pos * KS + tid] = own_map ? __fdiv_rn(lvl, ms) + mc : lvl * s_sc[tid] + s_zp[tid];
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
                    const uint32_t byte = a.v_main[rowh * (D / 4) + bc];
                    const int64_t vg = rowh * (D / 32) + (bc >> 3);
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
    const size_t shm = sizeof(float) * (big + R * D + 2 * D + R * 32 + 8) + sizeof(int64_t) * 32;
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

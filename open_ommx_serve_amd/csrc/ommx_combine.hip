// Split combine with the bf16 sink/recent tail folded in: one workgroup of 2*D threads per
// (request, q head).  Follows ommx_gpu_serve/attention/paged_decode.py:2366-2500: valid
// splits are recomputed from the packed length with the stage-1 rounding; the tail is one
// more softmax part computed here from k_tail/v_tail; o = sum w_i o_i / sum w_i,
// lse = max + ln sum w_i; nothing attended gives o = 0, lse = -inf.
//
// The two halves of the workgroup work side by side: threads [0,D) reduce the split
// partials for channel d, threads [D,2D) compute the tail (one row's q.k per thread with
// 16-byte loads, then one channel's p.v per thread) and hand it over through LDS.
#include "ommx_decode_args.h"

namespace ommx {

template <int D>
__global__ void __launch_bounds__(2 * D) combine_kernel(CombineArgs a) {
    constexpr int MAXS = 256;            // split slots kept in LDS (host checks S <= MAXS)
    __shared__ float s_q[D];
    __shared__ float s_lse[MAXS];
    __shared__ float s_logit[D];         // tail logits / weights of the current chunk
    __shared__ float s_tail[D + 2];      // tail part: o[D], l, m
    const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int kvh = h / (a.Hq / a.Hkv);
    const int L = a.seq[b];
    const int tail = a.tail ? a.tail[b] : 0;
    const int per = ((((L + a.S - 1) / a.S) + 31) / 32) * 32;
    const float* base = a.al + b * a.al_b + (int64_t)h * a.al_h;
    const bool lower = tid < D;

    if (lower) {
        if (tail > 0) s_q[tid] = bf16_to_f32(a.q[b * a.q_sb + (int64_t)h * a.q_sh + tid]);
        for (int s = tid; s < a.S; s += D) {
            const bool valid = min(per * s + per, L) > per * s;
            s_lse[s] = valid ? base[(int64_t)s * a.al_s + D] : -INFINITY;
        }
    }
    __syncthreads();

    float t_m = -INFINITY, t_l = 0.0f, t_acc = 0.0f;
    float acc = 0.0f, wsum = 0.0f, g_max = -INFINITY;
    if (lower) {
        // ---- packed splits, channel d = tid -------------------------------------------
        for (int s = 0; s < a.S; ++s) g_max = fmaxf(g_max, s_lse[s]);
        const float g_safe = (g_max == -INFINITY) ? 0.0f : g_max;
#pragma unroll 8
        for (int s = 0; s < a.S; ++s) {
            const float ls = s_lse[s];
            if (ls != -INFINITY) {
                const float w = __expf(ls - g_safe);
                wsum += w;
                acc = fmaf(w, base[(int64_t)s * a.al_s + tid], acc);
            }
        }
    }
    // ---- tail, chunks of D rows (uniform trip count for the whole workgroup) -----------
    for (int r0 = 0; r0 < tail; r0 += D) {
        const int nr = min(D, tail - r0);
        if (!lower) {
            const int r = tid - D;
            float s = -INFINITY;
            if (r < nr) {
                const uint4* kr = reinterpret_cast<const uint4*>(
                    a.kt + b * a.kt_b + (int64_t)(r0 + r) * a.kt_t + (int64_t)kvh * a.kt_h);
                float dot = 0.0f;
#pragma unroll
                for (int i = 0; i < D / 8; ++i) {
                    const uint4 u = kr[i];
                    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        dot = fmaf(s_q[8 * i + 2 * j], __uint_as_float(w[j] << 16), dot);
                        dot = fmaf(s_q[8 * i + 2 * j + 1], __uint_as_float(w[j] & 0xFFFF0000u), dot);
                    }
                }
                s = apply_cap(dot * a.sm_scale, a.cap);
            }
            s_logit[r] = s;
        }
        __syncthreads();
        if (!lower) {
            const int d = tid - D;
            float mx = -INFINITY;
            for (int i = 0; i < nr; ++i) mx = fmaxf(mx, s_logit[i]);
            const float m_new = fmaxf(t_m, mx);
            const float alpha = (t_m == -INFINITY) ? 0.0f : __expf(t_m - m_new);
            t_l *= alpha;
            t_acc *= alpha;
            const uint16_t* vr = a.vt + b * a.vt_b + (int64_t)r0 * a.vt_t + (int64_t)kvh * a.vt_h + d;
#pragma unroll 8
            for (int i = 0; i < nr; ++i) {
                const float p = __expf(s_logit[i] - m_new);
                t_l += p;
                t_acc = fmaf(p, bf16_to_f32(vr[(int64_t)i * a.vt_t]), t_acc);
            }
            t_m = m_new;
        }
        __syncthreads();
    }
    if (!lower) {
        const int d = tid - D;
        s_tail[d] = t_l > 0.0f ? t_acc / t_l : 0.0f;
        if (d == 0) { s_tail[D] = t_l; s_tail[D + 1] = t_m; }
    }
    __syncthreads();
    if (lower) {
        const float tl = s_tail[D], tm = s_tail[D + 1];
        const float tail_lse = tl > 0.0f ? tm + __logf(tl) : -INFINITY;
        const float n_max = fmaxf(g_max, tail_lse);
        const float n_safe = (n_max == -INFINITY) ? 0.0f : n_max;
        // re-base the split sums on the joint maximum, then add the tail part
        const float rs = (g_max == -INFINITY) ? 0.0f : __expf(g_max - n_safe);
        wsum *= rs;
        acc *= rs;
        if (tl > 0.0f) {
            const float w = __expf(tail_lse - n_safe);
            wsum += w;
            acc = fmaf(w, s_tail[tid], acc);
        }
        a.o[b * a.o_b + (int64_t)h * a.o_h + tid] = wsum > 0.0f ? acc / wsum : 0.0f;
        if (tid == 0) a.lse[b * a.lse_b + h] = wsum > 0.0f ? n_max + __logf(wsum) : -INFINITY;
    }
}

int launch_combine(const CombineArgs& a, int D, hipStream_t st) {
    if (a.S > 256) return -1;
    const dim3 grid(a.B, a.Hq);
    if (D == 128) hipLaunchKernelGGL(combine_kernel<128>, grid, dim3(256), 0, st, a);
    else if (D == 64) hipLaunchKernelGGL(combine_kernel<64>, grid, dim3(128), 0, st, a);
    else return -1;
    return 0;
}

}  // namespace ommx

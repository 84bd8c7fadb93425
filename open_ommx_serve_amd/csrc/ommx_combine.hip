// Split combine with the bf16 sink/recent tail folded in: one workgroup of D threads per
// (request, q head).  Follows ommx_gpu_serve/attention/paged_decode.py:2366-2500: valid
// splits are recomputed from the packed length with the stage-1 rounding; the tail is one
// more softmax part computed here from k_tail/v_tail; o = sum w_i o_i / sum w_i,
// lse = max + ln sum w_i; nothing attended gives o = 0, lse = -inf.
#include "ommx_decode_args.h"

namespace ommx {

template <int D>
__global__ void __launch_bounds__(D) combine_kernel(CombineArgs a) {
    constexpr int NW = D / 64;
    __shared__ float s_q[D];
    __shared__ float s_p[D];           // tail weights of the current chunk of D rows
    __shared__ float s_red[8];
    const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
    const int kvh = h / (a.Hq / a.Hkv);
    const int L = a.seq[b];
    const int tail = a.tail ? a.tail[b] : 0;
    const int per = ((((L + a.S - 1) / a.S) + 31) / 32) * 32;

    // ---- tail part: online softmax over chunks of D rows ------------------------------
    float t_m = -INFINITY, t_l = 0.0f, t_acc = 0.0f;
    if (tail > 0) {
        s_q[d] = bf16_to_f32(a.q[b * a.q_sb + (int64_t)h * a.q_sh + d]);
        __syncthreads();
        for (int r0 = 0; r0 < tail; r0 += D) {
            const int r = r0 + d;
            float s = -INFINITY;
            if (r < tail) {
                const uint16_t* kr = a.kt + b * a.kt_b + (int64_t)r * a.kt_t + (int64_t)kvh * a.kt_h;
                float dot = 0.0f;
#pragma unroll 8
                for (int i = 0; i < D; ++i) dot = fmaf(s_q[i], bf16_to_f32(kr[i]), dot);
                s = apply_cap(dot * a.sm_scale, a.cap);
            }
            float mx = s;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            if ((d & 63) == 0) s_red[d >> 6] = mx;
            __syncthreads();
            mx = s_red[0];
#pragma unroll
            for (int w = 1; w < NW; ++w) mx = fmaxf(mx, s_red[w]);
            const float m_new = fmaxf(t_m, mx);
            const float p = (r < tail) ? __expf(s - m_new) : 0.0f;
            s_p[d] = p;
            float ps = p;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) ps += __shfl_xor(ps, o);
            if ((d & 63) == 0) s_red[4 + (d >> 6)] = ps;
            __syncthreads();
            ps = s_red[4];
#pragma unroll
            for (int w = 1; w < NW; ++w) ps += s_red[4 + w];
            const float alpha = (t_m == -INFINITY) ? 0.0f : __expf(t_m - m_new);
            t_l = t_l * alpha + ps;
            t_acc *= alpha;
            const int nr = min(D, tail - r0);
            const uint16_t* vr = a.vt + b * a.vt_b + (int64_t)r0 * a.vt_t + (int64_t)kvh * a.vt_h + d;
            for (int i = 0; i < nr; ++i)
                t_acc = fmaf(s_p[i], bf16_to_f32(vr[(int64_t)i * a.vt_t]), t_acc);
            t_m = m_new;
            __syncthreads();
        }
    }
    const float tail_lse = t_l > 0.0f ? t_m + __logf(t_l) : -INFINITY;

    // ---- packed splits -----------------------------------------------------------------
    const float* base = a.al + b * a.al_b + (int64_t)h * a.al_h;
    float g_max = tail_lse;
    for (int s = 0; s < a.S; ++s) {
        const bool valid = min(per * s + per, L) > per * s;
        if (valid) g_max = fmaxf(g_max, base[(int64_t)s * a.al_s + D]);
    }
    const float g_safe = (g_max == -INFINITY) ? 0.0f : g_max;
    float wsum = 0.0f, acc = 0.0f;
    for (int s = 0; s < a.S; ++s) {
        const bool valid = min(per * s + per, L) > per * s;
        if (valid) {
            const float ls = base[(int64_t)s * a.al_s + D];
            const float w = (ls == -INFINITY) ? 0.0f : __expf(ls - g_safe);
            wsum += w;
            acc = fmaf(w, base[(int64_t)s * a.al_s + d], acc);
        }
    }
    if (t_l > 0.0f) {
        const float w = __expf(tail_lse - g_safe);
        wsum += w;
        acc = fmaf(w, t_acc / t_l, acc);
    }
    a.o[b * a.o_b + (int64_t)h * a.o_h + d] = wsum > 0.0f ? acc / wsum : 0.0f;
    if (d == 0) a.lse[b * a.lse_b + h] = wsum > 0.0f ? g_max + __logf(wsum) : -INFINITY;
}

int launch_combine(const CombineArgs& a, int D, hipStream_t st) {
    const dim3 grid(a.B, a.Hq);
    if (D == 128) hipLaunchKernelGGL(combine_kernel<128>, grid, dim3(128), 0, st, a);
    else if (D == 64) hipLaunchKernelGGL(combine_kernel<64>, grid, dim3(64), 0, st, a);
    else return -1;
    return 0;
}

}  // namespace ommx

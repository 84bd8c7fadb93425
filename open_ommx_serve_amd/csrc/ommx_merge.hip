// Merge of partial attention states: P parts (o_p [R,D], lse_p [R]) of the same query rows,
// computed over disjoint KV segments, into the state over their union:
//   m = max_p lse_p;  w_p = exp(lse_p - m);  o = sum w_p o_p / sum w_p;  lse = m + ln sum w_p.
// Same operator as merge_attention_states of
// ommx_gpu_serve/attention/paged_decode.py:3556-3624 (rows are independent; a part whose lse
// is -inf has weight zero; a row with no attended part gives o = 0, lse = -inf).
#include "ommx_common.h"

namespace ommx {

__global__ void __launch_bounds__(256) merge_states_kernel(
    const float* __restrict__ o_parts, const float* __restrict__ lse_parts,
    const int32_t* __restrict__ valid_lens, float* __restrict__ o, float* __restrict__ lse,
    int P, int R, int D, int64_t op_sp, int64_t op_sr, int64_t lp_sp, int64_t o_sr) {
    const int r = blockIdx.x;
    int np = P;
    if (valid_lens) { const int v = valid_lens[r]; if (v >= 0 && v < P) np = v; }
    // every thread scans the lse column (P is small: segments, ranks, chunks)
    float m = -INFINITY;
    for (int p = 0; p < np; ++p) m = fmaxf(m, lse_parts[p * lp_sp + r]);
    const float m_safe = (m == -INFINITY) ? 0.0f : m;
    float wsum = 0.0f;
    for (int p = 0; p < np; ++p) {
        const float l = lse_parts[p * lp_sp + r];
        wsum += (l == -INFINITY) ? 0.0f : __expf(l - m_safe);
    }
    const float inv = wsum > 0.0f ? 1.0f / wsum : 0.0f;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float acc = 0.0f;
        for (int p = 0; p < np; ++p) {
            const float l = lse_parts[p * lp_sp + r];
            if (l != -INFINITY) acc = fmaf(__expf(l - m_safe), o_parts[p * op_sp + r * op_sr + d], acc);
        }
        o[r * o_sr + d] = acc * inv;
    }
    if (threadIdx.x == 0) lse[r] = wsum > 0.0f ? m + __logf(wsum) : -INFINITY;
}

}  // namespace ommx

extern "C" int ommx_merge_states(const float* o_parts, const float* lse_parts,
                                 const int32_t* valid_lens, float* o, float* lse,
                                 int P, int R, int D, int64_t op_stride_p, int64_t op_stride_r,
                                 int64_t lp_stride_p, int64_t o_stride_r, void* stream) {
    using namespace ommx;
    if (P <= 0 || R < 0 || D <= 0) { set_error("ommx_merge_states: bad shape"); return -1; }
    if (!o_parts || !lse_parts || !o || !lse) { set_error("ommx_merge_states: null pointer"); return -1; }
    if (R == 0) return 0;
    const int threads = D >= 256 ? 256 : (D >= 128 ? 128 : 64);
    hipLaunchKernelGGL(merge_states_kernel, dim3(R), dim3(threads), 0, static_cast<hipStream_t>(stream),
                       o_parts, lse_parts, valid_lens, o, lse, P, R, D, op_stride_p, op_stride_r,
                       lp_stride_p, o_stride_r);
    if (hipGetLastError() != hipSuccess) { set_error("ommx_merge_states: launch failed"); return -2; }
    return 0;
}

// bf16 residual ring of the KV store: the rows that are not (yet) packed.
//
//   ring_write_kernel   one new K/V row per request into its ring slot; follows
//                       ommx_gpu_serve/attention/kv_store_ops.py:22-40 (_kv_write_token) and
//                       the batched scatter of attention/kv_pool.py:407-419.
//   tail_gather_kernel  sink + recent rows of every request into the fixed tail buffers,
//                       with the window arithmetic of attention/kv_pool.py:1048-1105
//                       (decode_inputs_device) done in the kernel from the device sequence
//                       lengths; or, given explicit positions, the plain gather of
//                       kv_store_ops.py:42-61 (_kv_gather_tail).
//
// Ring slot of absolute position p (kv_store.py:301-327): p below the sink count stays,
// everything else slides modulo the ring span: sink + (p - sink) % span.  span == 0 means
// the history is kept whole and the slot is the position.
//
// Both kernels are pure row copies (H*D bf16 per row), 16 bytes per thread when rows are
// 16-byte aligned, one workgroup per row.
#include "ommx_ring_args.h"

namespace ommx {

__device__ __forceinline__ int64_t ring_slot(int64_t pos, int sink, int span) {
    if (span <= 0 || pos < sink) return pos;
    return sink + (pos - sink) % span;
}

// Copies n_elem bf16 from src (rows of D contiguous elements, head stride hs) to a dense row.
__device__ __forceinline__ void copy_row_in(uint16_t* dst, const uint16_t* src, int64_t hs,
                                            int H, int D, bool vec) {
    if (vec) {
        const int per_head = D / 8;
        for (int i = threadIdx.x; i < H * per_head; i += blockDim.x) {
            const int h = i / per_head, c = (i % per_head) * 8;
            *reinterpret_cast<uint4*>(dst + h * D + c) =
                *reinterpret_cast<const uint4*>(src + h * hs + c);
        }
    } else {
        for (int i = threadIdx.x; i < H * D; i += blockDim.x) dst[i] = src[(i / D) * hs + i % D];
    }
}

__global__ void __launch_bounds__(256) ring_write_kernel(
    RingArgs a, const uint16_t* k, const uint16_t* v, int64_t k_bs, int64_t k_hs, int64_t v_bs,
    int64_t v_hs, const int64_t* pos, int64_t* pos_next, int vec) {
    const int b = blockIdx.x;
    const int64_t p = pos[b];
    const int64_t slot = a.slots ? a.slots[b] : b;
    const int64_t row = ring_slot(p, a.sink, a.span);
    __syncthreads();                       // every thread has read pos[b] before it moves
    if (pos_next && threadIdx.x == 0) pos_next[b] = p + 1;
    if (row < 0 || row >= a.cap) {         // kv_store_ops.py:33-34 asserts here
        if (a.err && threadIdx.x == 0) atomicOr(a.err, OMMX_ERR_RING_RANGE);
        return;
    }
    const int64_t off = slot * a.req_stride + row * (int64_t)(a.H * a.D);
    copy_row_in(a.k_hist + off, k + b * k_bs, k_hs, a.H, a.D, vec);
    copy_row_in(a.v_hist + off, v + b * v_bs, v_hs, a.H, a.D, vec);
}

__global__ void __launch_bounds__(256) tail_gather_kernel(
    RingArgs a, const int64_t* seq, const int64_t* tail_idx, uint16_t* k_tail, uint16_t* v_tail,
    int T, int recent, int gt, int lag, int32_t* b_tail_len, int32_t* b_seq_len, int vec) {
    const int t = blockIdx.x, b = blockIdx.y;
    int64_t abs_pos;
    if (tail_idx) {
        abs_pos = tail_idx[(int64_t)b * T + t];
    } else {
        // kv_pool.py:1080-1097: boundary, counts and the sink ++ recent position ramp.  The
        // packed boundary is the one of the length the planes were last packed for, `lag`
        // tokens ago: rows appended since then are read from the ring, the group they may
        // have completed included.
        const int64_t s = seq[b];
        const int64_t s_packed = s > lag ? s - lag : 0;
        const int64_t extra = s_packed - a.sink - recent;
        const int64_t n_sink = s < a.sink ? s : a.sink;
        const int64_t boundary = extra <= 0 ? n_sink : a.sink + (extra / gt) * gt;
        const int64_t n_rec = s > boundary ? s - boundary : 0;
        const int64_t n_total = n_sink + n_rec;
        abs_pos = t < n_sink ? t : boundary + (t - n_sink);
        if (t >= n_total) abs_pos = 0;     // padding rows repeat position 0; readers mask them
        if (t == 0 && threadIdx.x == 0) {
            if (b_tail_len) b_tail_len[b] = (int32_t)(n_total < T ? n_total : T);
            if (b_seq_len) b_seq_len[b] = (int32_t)(boundary > a.sink ? boundary - a.sink : 0);
        }
    }
    const int64_t slot = a.slots ? a.slots[b] : b;
    const int64_t row = ring_slot(abs_pos, a.sink, a.span);
    const int HD = a.H * a.D;
    uint16_t* kd = k_tail + ((int64_t)b * T + t) * HD;
    uint16_t* vd = v_tail + ((int64_t)b * T + t) * HD;
    if (row < 0 || row >= a.cap) {         // kv_store_ops.py:52-53 asserts here
        if (a.err && threadIdx.x == 0) atomicOr(a.err, OMMX_ERR_RING_RANGE);
        for (int i = threadIdx.x; i < HD; i += blockDim.x) { kd[i] = 0; vd[i] = 0; }
        return;
    }
    const uint16_t* ks = a.k_hist + slot * a.req_stride + row * (int64_t)HD;
    const uint16_t* vs = a.v_hist + slot * a.req_stride + row * (int64_t)HD;
    if (vec) {
        for (int i = threadIdx.x; i < HD / 8; i += blockDim.x) {
            reinterpret_cast<uint4*>(kd)[i] = reinterpret_cast<const uint4*>(ks)[i];
            reinterpret_cast<uint4*>(vd)[i] = reinterpret_cast<const uint4*>(vs)[i];
        }
    } else {
        for (int i = threadIdx.x; i < HD; i += blockDim.x) { kd[i] = ks[i]; vd[i] = vs[i]; }
    }
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int launch_ring_write(const RingArgs& a, const uint16_t* k, const uint16_t* v, int64_t k_bs,
                      int64_t k_hs, int64_t v_bs, int64_t v_hs, const int64_t* pos,
                      int64_t* pos_next, int B, hipStream_t st) {
    const int vec = a.D % 8 == 0 && aligned16(a.k_hist) && aligned16(a.v_hist) && aligned16(k) &&
                    aligned16(v) && a.req_stride % 8 == 0 && k_bs % 8 == 0 && k_hs % 8 == 0 &&
                    v_bs % 8 == 0 && v_hs % 8 == 0;
    const int threads = (a.H * a.D / (vec ? 8 : 1)) >= 256 ? 256 : 128;
    hipLaunchKernelGGL(ring_write_kernel, dim3(B), dim3(threads), 0, st, a, k, v, k_bs, k_hs, v_bs,
                       v_hs, pos, pos_next, vec);
    return 0;
}

int launch_tail_gather(const RingArgs& a, const int64_t* seq, const int64_t* tail_idx,
                       uint16_t* k_tail, uint16_t* v_tail, int B, int T, int recent, int gt,
                       int lag, int32_t* b_tail_len, int32_t* b_seq_len, hipStream_t st) {
    const int vec = (a.H * a.D) % 8 == 0 && aligned16(a.k_hist) && aligned16(a.v_hist) &&
                    aligned16(k_tail) && aligned16(v_tail) && a.req_stride % 8 == 0;
    const int threads = (a.H * a.D / (vec ? 8 : 1)) >= 256 ? 256 : 128;
    hipLaunchKernelGGL(tail_gather_kernel, dim3(T, B), dim3(threads), 0, st, a, seq, tail_idx,
                       k_tail, v_tail, T, recent, gt, lag, b_tail_len, b_seq_len, vec);
    return 0;
}

}  // namespace ommx

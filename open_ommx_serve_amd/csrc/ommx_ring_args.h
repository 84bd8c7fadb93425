// Argument block and launchers of the bf16 residual-ring kernels.
#pragma once
#include "ommx_common.h"

namespace ommx {

struct RingArgs {
    uint16_t* k_hist;
    uint16_t* v_hist;
    int64_t req_stride;        // elements between the histories of two pool slots
    int cap;                   // rows per history
    int sink, span;            // pinned rows, sliding span (0: the history is kept whole)
    int H, D;
    const int64_t* slots;      // NULL: request b uses pool slot b
    int32_t* err;
};

int launch_ring_write(const RingArgs& a, const uint16_t* k, const uint16_t* v, int64_t k_bs,
                      int64_t k_hs, int64_t v_bs, int64_t v_hs, const int64_t* pos,
                      int64_t* pos_next, int B, hipStream_t st);
int launch_tail_gather(const RingArgs& a, const int64_t* seq, const int64_t* tail_idx,
                       uint16_t* k_tail, uint16_t* v_tail, int B, int T, int recent, int gt,
                       int lag, int32_t* b_tail_len, int32_t* b_seq_len, hipStream_t st);

}  // namespace ommx

// Split combine with the bf16 sink/recent tail folded in.  Follows
// ommx_gpu_serve/attention/paged_decode.py:2366-2500: valid splits are recomputed from the
// packed length with the stage-1 rounding; the tail is one more softmax part computed here from
// k_tail/v_tail; o = sum w_i o_i / sum w_i, lse = max + ln sum w_i; nothing attended gives
// o = 0, lse = -inf.
//
// Two kernels.  combine_kernel: Q workgroups per (request, q head), one per piece of the head's
// channels.  It is latency bound (few small workgroups, a few KB each), so every global load is
// issued before the first wait: thread (d, sg) owns channel d of the splits sg, sg+NSG, ... and
// of the tail rows sg, sg+NSG, ...; for the tail logits the same threads regroup as (row, 16
// parts of the row).  combine_grouped_kernel (further down): one workgroup per (request, kv head)
// for large batches, where the tail rows are most of the bytes and are read once for all the
// q heads of the kv head.
#include "ommx_decode_args.h"

namespace ommx {

namespace {
// Lane exchanges inside the vector ALU (DPP): no trip through the LDS crossbar, no index arithmetic.
template <int CTRL>
__device__ __forceinline__ float dpp_of(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        __builtin_bit_cast(int, v), __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
// sum over each row of 16 lanes, left in every lane of the row
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_of<0xB1>(v);        // quad_perm [1,0,3,2]
    v += dpp_of<0x4E>(v);        // quad_perm [2,3,0,1]
    v += dpp_of<0x141>(v);       // row_half_mirror
    v += dpp_of<0x140>(v);       // row_mirror
    return v;
}
// maximum over the 64 lanes, uniform
__device__ __forceinline__ float wave64_max(float v) {
    v = fmaxf(v, dpp_of<0xB1>(v));
    v = fmaxf(v, dpp_of<0x4E>(v));
    v = fmaxf(v, dpp_of<0x141>(v));
    v = fmaxf(v, dpp_of<0x140>(v));
    v = fmaxf(v, dpp_of<0x142>(v));      // row_bcast15: lane 15 of a row into the next row
    v = fmaxf(v, dpp_of<0x143>(v));      // row_bcast31: lane 31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
}  // namespace

// NT threads per workgroup, at most MAXS splits: 1024 / 256 in general, 512 / 64 when many
// (request, head) pairs with few splits each fill the chip (fewer idle lanes per workgroup).
template <int D, int Q, int NT = 1024, int MAXS = 256>
__global__ void __launch_bounds__(NT) combine_kernel(CombineArgs a) {
    constexpr int CH = D / Q;            // channels of this workgroup (one of Q pieces of the head)
    constexpr int NSG = NT / CH;         // split groups: thread (d, sg) owns splits sg, sg + NSG, ...
    static_assert(MAXS <= NT && MAXS % 64 == 0, "one thread per split slot");
    constexpr int NSP = MAXS / NSG;      // split partials per thread, upper bound
    constexpr int ROWS = NT / 16;        // tail rows handled per chunk (64)
    constexpr int PER = ROWS / NSG;      // tail rows per thread in the P.V step
    static_assert(PER >= 1 && NSP % 4 == 0, "thread layout");
    __shared__ float s_q[D];
    __shared__ __attribute__((aligned(16))) float s_logit[ROWS];
    __shared__ float s_acc[NSG][CH];     // per-sg sums of the split part
    __shared__ float s_tacc[NSG][CH];    // per-sg sums of the tail part
    __shared__ float s_w[NSG], s_tl[NSG], s_wmax[MAXS / 64];
    __shared__ __attribute__((aligned(16))) float s_wT[NSG][NSP];   // weight of split sg + NSG*i at [sg][i]
    const int b = blockIdx.x, h = blockIdx.y, cq = blockIdx.z, tid = threadIdx.x;
    const int dl = tid % CH, sg = tid / CH;
    const int d = cq * CH + dl;          // this thread's channel of the head
    const int kvh = h / (a.Hq / a.Hkv);
    const float* base = a.al + b * a.al_b + (int64_t)h * a.al_h;
    // the two scalars that everything after the split loads waits for: requested first
    const int L = a.seq[b];
    // a length outside the tail buffer (when the caller has said how many rows it holds) is held
    // inside it, so that no row address leaves the buffer whatever b_tail_len contains
    int tail = a.tail ? a.tail[b] : 0;
    tail = max(tail, 0);
    if (a.T > 0) tail = min(tail, a.T);

    // ---- all loads of the split part --------------------------------------------------
    // They depend on the arguments only, so they go out before anything is read from
    // memory; one pointer per thread, advanced by NSG split slots per load.  (A uniform trip
    // count and a clamped last address keep the loads free of per-lane branches, so they
    // are all in flight together.)
    float pv[NSP];
    const int n_i = (a.S + NSG - 1) / NSG;
    {
        const float* p = base + (int64_t)sg * a.al_s + d;
        const int64_t step = NSG * a.al_s;
#pragma unroll
        for (int i = 0; i < NSP; ++i) {
            pv[i] = 0.0f;
            if (i < n_i) {
                const bool inside = sg + NSG * i < a.S;        // only the last trip can fall outside
                pv[i] = *(inside ? p : base + (int64_t)(a.S - 1) * a.al_s + d);
                p += step;
            }
        }
    }
    const uint32_t q_raw = (a.q && tid < D) ? a.q[b * a.q_sb + (int64_t)h * a.q_sh + tid] : 0u;
    // Every split wrote its state, an empty one with lse = -inf (paged_decode.py:2262-2284), so the
    // weights follow from the lse column alone, whatever rule dealt the tokens out to the splits
    // (the reference recomputes its rounding here, paged_decode.py:2407-2410).
    float my_lse = -INFINITY;
    if (tid < MAXS && tid < a.S) my_lse = base[(int64_t)tid * a.al_s + D];
    (void)L;

    if (tid < D) s_q[tid] = __uint_as_float(q_raw << 16);
    if (tid < MAXS) {
        const float wm = wave64_max(my_lse);
        if ((tid & 63) == 0) s_wmax[tid >> 6] = wm;
    }

    // ---- tail: chunks of ROWS rows (one chunk in practice: sink + recent <= 72 rows) ----
    // Every quarter computes all the logits (they need the whole q and K rows) and its own
    // channels of P.V.
    float t_m = -INFINITY, t_l = 0.0f, t_acc = 0.0f;
    const int row = tid >> 4, part = tid & 15;
    // loads of one chunk: 16 bytes of one K row, PER elements of V; rows from `last` on repeat it
    uint4 ku;
    uint32_t vv[PER];
    auto load_rows = [&](int r0, int last) {
        ku = *reinterpret_cast<const uint4*>(
            a.kt + b * a.kt_b + (int64_t)(r0 + min(row, last)) * a.kt_t + (int64_t)kvh * a.kt_h +
            (part * 8) % D);
#pragma unroll
        for (int i = 0; i < PER; ++i)
            vv[i] = a.vt[b * a.vt_b + (int64_t)(r0 + min(sg + NSG * i, last)) * a.vt_t +
                         (int64_t)kvh * a.vt_h + d];
    };
    // When the caller has said how many rows the tail buffers hold, the first chunk is asked for
    // here, with the split loads and before the tail length has arrived (its uses below wait for
    // it): rows past the tail are addressable, and neither their logits nor their V are used.
    const bool early = a.T > 0 && a.tail != nullptr;
    if (early) load_rows(0, min(ROWS, a.T) - 1);
    for (int r0 = 0; r0 < tail; r0 += ROWS) {
        const int nr = min(ROWS, tail - r0);
        if (!(early && r0 == 0)) load_rows(r0, nr - 1);
        __syncthreads();                              // s_q ready (and previous chunk consumed)
        float dot = 0.0f;
        if (part * 8 < D) {
            const uint32_t w[4] = {ku.x, ku.y, ku.z, ku.w};
            const float* qq = s_q + part * 8;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                dot = fmaf(qq[2 * i], __uint_as_float(w[i] << 16), dot);
                dot = fmaf(qq[2 * i + 1], __uint_as_float(w[i] & 0xFFFF0000u), dot);
            }
        }
        dot = row16_sum(dot);
        if (part == 0) s_logit[row] = row < nr ? apply_cap(dot * a.sm_scale, a.cap) : -INFINITY;
        __syncthreads();
        // maximum of the chunk's logits: one logit per lane, reduced over the wave (every thread
        // reading all ROWS of them cost 16 LDS reads of 16 bytes each); s_logit holds -inf past nr
        static_assert(ROWS <= 64, "one logit per lane");
        const float mx = wave64_max((tid & 63) < ROWS ? s_logit[tid & 63] : -INFINITY);
        const float m_new = fmaxf(t_m, mx);
        const float alpha = (t_m == -INFINITY) ? 0.0f : __expf(t_m - m_new);
        t_l *= alpha;
        t_acc *= alpha;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int r = sg + NSG * i;
            if (r < nr) {
                const float p = __expf(s_logit[r] - m_new);
                t_l += p;
                t_acc = fmaf(p, __uint_as_float(vv[i] << 16), t_acc);
            }
        }
        t_m = m_new;
    }
    __syncthreads();                                  // s_wmax ready

    // ---- split part: weights from the lse column -----------------------------------------
    // One thread per split turns its lse into a weight; the weights are laid out so that
    // thread (d, sg) reads the ones of its splits sg, sg+NSG, ... as float4.
    float g_max = s_wmax[0];
#pragma unroll
    for (int w = 1; w < MAXS / 64; ++w) g_max = fmaxf(g_max, s_wmax[w]);
    const float g_safe = (g_max == -INFINITY) ? 0.0f : g_max;
    if (tid < MAXS) s_wT[tid % NSG][tid / NSG] = my_lse == -INFINITY ? 0.0f : __expf(my_lse - g_safe);
    __syncthreads();
    float acc = 0.0f, wsum = 0.0f;
#pragma unroll
    for (int i4 = 0; i4 < NSP / 4; ++i4) {
        const float4 w4 = reinterpret_cast<const float4*>(s_wT[sg])[i4];
        const float w[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {          // absent splits have weight zero; their slot
            wsum += w[k];                      // may hold anything, so it is not multiplied
            acc = w[k] > 0.0f ? fmaf(w[k], pv[4 * i4 + k], acc) : acc;
        }
    }
    s_acc[sg][dl] = acc;
    s_tacc[sg][dl] = t_acc;
    if (dl == 0) { s_w[sg] = wsum; s_tl[sg] = t_l; }
    __syncthreads();
    if (sg == 0) {
        float A = 0.0f, W = 0.0f, TA = 0.0f, TL = 0.0f;
#pragma unroll
        for (int k = 0; k < NSG; ++k) { A += s_acc[k][dl]; W += s_w[k]; TA += s_tacc[k][dl]; TL += s_tl[k]; }
        const float tail_lse = TL > 0.0f ? t_m + __logf(TL) : -INFINITY;
        const float n_max = fmaxf(g_max, tail_lse);
        const float n_safe = (n_max == -INFINITY) ? 0.0f : n_max;
        const float rs = (g_max == -INFINITY) ? 0.0f : __expf(g_max - n_safe);
        W *= rs;
        A *= rs;
        if (TL > 0.0f) {
            const float w = __expf(tail_lse - n_safe);
            W += w;
            A = fmaf(w, TA / TL, A);
        }
        a.o[b * a.o_b + (int64_t)h * a.o_h + d] = W > 0.0f ? A / W : 0.0f;
        if (d == 0) a.lse[b * a.lse_b + h] = W > 0.0f ? n_max + __logf(W) : -INFINITY;
    }
}

__device__ __forceinline__ float wave_max_f32(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// The same merge for a whole kv head at a time: one workgroup of 512 threads per (request, kv
// head) serves the R = 4 or 8 q heads of that kv head, so the bf16 tail rows -- most of the bytes
// when there are few splits -- are read once instead of once per q head.  Used when (request, kv
// head) pairs alone fill the chip twice over (then nothing is gained by one workgroup per q
// head) and there are at most 64 splits.  Wave r < R owns the scalars of head r (split weights, running tail maximum
// and sum); the channel work is dealt out as (head, channel) for the splits and as (channel
// pair, row group) for the tail's P.V.
// EARLY: the tail rows of the first pass are asked for before the split part and held in registers
// (32 more: one workgroup per compute unit instead of two, which pays while the grid is no larger
// than the chip).
template <int D, int R, bool EARLY>
__global__ void __launch_bounds__(512) combine_grouped_kernel(CombineArgs a) {
    constexpr int NT = 512, MAXS = 64;
    constexpr int ROWS = 128;              // tail rows per pass (two per thread of the logit layout)
    constexpr int CHP = D / 8;             // channels per thread of a K row (8 threads per row)
    constexpr int NRG = NT / (D / 2);      // row groups of the P.V layout
    constexpr int HD = (R * D + NT - 1) / NT;   // (head, channel) items per thread
    __shared__ __attribute__((aligned(16))) float s_q[R][D];
    __shared__ float s_w[R][MAXS];
    __shared__ float s_gmax[R], s_W[R], s_alpha[R], s_tm[R], s_tl[R];
    __shared__ float s_logit[R][ROWS];
    __shared__ float s_p[R][ROWS];
    __shared__ float s_red[NRG][R][D];
    const int b = blockIdx.x, kvh = blockIdx.y, tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int h0 = kvh * R;
    const float* base = a.al + b * a.al_b + (int64_t)h0 * a.al_h;
    const int L = a.seq[b];
    // a length outside the tail buffer (when the caller has said how many rows it holds) is held
    // inside it, so that no row address leaves the buffer whatever b_tail_len contains
    int tail = a.tail ? a.tail[b] : 0;
    tail = max(tail, 0);
    if (a.T > 0) tail = min(tail, a.T);

    // ---- split weights: wave r, lane s ----------------------------------------------------
    if (a.q) {
        for (int i = tid; i < R * D / 2; i += NT) {
            const int r = i / (D / 2), c2 = i % (D / 2);
            const uint32_t w = *reinterpret_cast<const uint32_t*>(
                a.q + b * a.q_sb + (int64_t)(h0 + r) * a.q_sh + 2 * c2);
            s_q[r][2 * c2] = __uint_as_float(w << 16);
            s_q[r][2 * c2 + 1] = __uint_as_float(w & 0xFFFF0000u);
        }
    }
    (void)L;
    if (wave < R) {
        const bool valid = lane < a.S;          // an empty split's lse is -inf
        const float my_lse = valid ? base[(int64_t)wave * a.al_h + (int64_t)lane * a.al_s + D] : -INFINITY;
        const float g_max = wave_max_f32(my_lse);
        const float g_safe = (g_max == -INFINITY) ? 0.0f : g_max;
        const float w = my_lse == -INFINITY ? 0.0f : __expf(my_lse - g_safe);
        const float W = wave_sum_f32(w);
        s_w[wave][lane] = w;
        if (lane == 0) { s_gmax[wave] = g_max; s_W[wave] = W; }
    }
    __syncthreads();

    // ---- the tail rows of the first pass are asked for here, before the split part waits for its
    // own loads: thread (row, part) holds CHP channels of K rows row and row + 64, thread (channel
    // pair, row group) the V dwords of rows rg, rg + NRG, ...
    constexpr int VPT = ROWS / NRG;        // V rows per thread and pass
    const int dp = tid % (D / 2), rg = tid / (D / 2);
    uint4 kk[2][CHP / 8];
    uint32_t vv[VPT];
    auto ask_rows = [&](int r0, int nr) {
        const int part = tid & 7, row = tid >> 3;
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
            const int t = row + 64 * h2;
#pragma unroll
            for (int c8 = 0; c8 < CHP / 8; ++c8) kk[h2][c8] = uint4{0u, 0u, 0u, 0u};
            if (t < nr) {
                const uint16_t* kp = a.kt + b * a.kt_b + (int64_t)(r0 + t) * a.kt_t +
                                     (int64_t)kvh * a.kt_h + part * CHP;
#pragma unroll
                for (int c8 = 0; c8 < CHP / 8; ++c8) kk[h2][c8] = reinterpret_cast<const uint4*>(kp)[c8];
            }
        }
        if constexpr (EARLY) {
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                const int t = rg + NRG * i;
                vv[i] = 0u;
                if (t < nr)
                    vv[i] = *reinterpret_cast<const uint32_t*>(
                        a.vt + b * a.vt_b + (int64_t)(r0 + t) * a.vt_t + (int64_t)kvh * a.vt_h + 2 * dp);
            }
        }
    };
    if constexpr (EARLY) ask_rows(0, min(ROWS, tail));

    // ---- split part: item (head, channel) ---------------------------------------------------
    // Every split slot is read (it exists; an absent split's content is stale and is dropped by
    // the select), so that the loads carry no branch and go out eight at a time.
    float A[HD];
#pragma unroll
    for (int k = 0; k < HD; ++k) {
        A[k] = 0.0f;
        const int i = tid + k * NT;
        if (i < R * D) {
            const int r = i / D, d = i % D;
            const float* p = base + (int64_t)r * a.al_h + d;
            float acc = 0.0f;
            for (int s0 = 0; s0 < a.S; s0 += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = p[(int64_t)min(s0 + u, a.S - 1) * a.al_s];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const float w = s0 + u < a.S ? s_w[r][s0 + u] : 0.0f;
                    acc = w > 0.0f ? fmaf(w, v[u], acc) : acc;
                }
            }
            A[k] = acc;
        }
    }

    // ---- tail: passes of up to ROWS rows, online over passes ------------------------------
    float m_run = -INFINITY, l_run = 0.0f;          // of head `wave` (waves < R)
    float acc[R][2];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r][0] = acc[r][1] = 0.0f;
    for (int r0 = 0; r0 < tail; r0 += ROWS) {
        const int nr = min(ROWS, tail - r0);
        if (!EARLY || r0 > 0) ask_rows(r0, nr);
        {   // logits: thread (row, part) takes CHP channels of rows row and row + 64
            const int part = tid & 7, row = tid >> 3;
#pragma unroll
            for (int rr = 0; rr < ROWS; rr += 64) {
                const int t = row + rr;
                float dot[R];
#pragma unroll
                for (int r = 0; r < R; ++r) dot[r] = 0.0f;
                if (t < nr) {
#pragma unroll
                    for (int c8 = 0; c8 < CHP / 8; ++c8) {
                        const uint4 ku = kk[rr / 64][c8];
                        const uint32_t w[4] = {ku.x, ku.y, ku.z, ku.w};
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float k0 = __uint_as_float(w[i] << 16);
                            const float k1 = __uint_as_float(w[i] & 0xFFFF0000u);
                            const int c = part * CHP + 8 * c8 + 2 * i;
#pragma unroll
                            for (int r = 0; r < R; ++r)
                                dot[r] = fmaf(s_q[r][c + 1], k1, fmaf(s_q[r][c], k0, dot[r]));
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
#pragma unroll
                    for (int o = 1; o < 8; o <<= 1) dot[r] += __shfl_xor(dot[r], o);
                }
                if (part == 0) {
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        s_logit[r][t] = t < nr ? apply_cap(dot[r] * a.sm_scale, a.cap) : -INFINITY;
                }
            }
        }
        __syncthreads();
        if (wave < R) {   // softmax bookkeeping of head `wave`: rows lane and lane + 64
            const float x0 = s_logit[wave][lane], x1 = s_logit[wave][lane + 64];
            const float m_new = fmaxf(m_run, wave_max_f32(fmaxf(x0, x1)));
            const float alpha = (m_run == -INFINITY) ? 0.0f : __expf(m_run - m_new);
            const float p0 = x0 == -INFINITY ? 0.0f : __expf(x0 - m_new);
            const float p1 = x1 == -INFINITY ? 0.0f : __expf(x1 - m_new);
            l_run = l_run * alpha + wave_sum_f32(p0 + p1);
            m_run = m_new;
            s_p[wave][lane] = p0;
            s_p[wave][lane + 64] = p1;
            if (lane == 0) s_alpha[wave] = alpha;
        }
        __syncthreads();
        {   // P.V: thread (channel pair, row group)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float al = s_alpha[r];
                acc[r][0] *= al;
                acc[r][1] *= al;
            }
            if constexpr (EARLY) {
#pragma unroll
                for (int i = 0; i < VPT; ++i) {
                    const int t = rg + NRG * i;
                    if (t < nr) {
                        const float v0 = __uint_as_float(vv[i] << 16), v1 = __uint_as_float(vv[i] & 0xFFFF0000u);
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            const float p = s_p[r][t];
                            acc[r][0] = fmaf(p, v0, acc[r][0]);
                            acc[r][1] = fmaf(p, v1, acc[r][1]);
                        }
                    }
                }
            } else {
                for (int t = rg; t < nr; t += NRG) {
                    const uint32_t vw = *reinterpret_cast<const uint32_t*>(
                        a.vt + b * a.vt_b + (int64_t)(r0 + t) * a.vt_t + (int64_t)kvh * a.vt_h + 2 * dp);
                    const float v0 = __uint_as_float(vw << 16), v1 = __uint_as_float(vw & 0xFFFF0000u);
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const float p = s_p[r][t];
                        acc[r][0] = fmaf(p, v0, acc[r][0]);
                        acc[r][1] = fmaf(p, v1, acc[r][1]);
                    }
                }
            }
        }
        // (the next pass writes s_logit before its first barrier and s_p after it: both are
        // past every read of this pass)
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        s_red[rg][r][2 * dp] = acc[r][0];
        s_red[rg][r][2 * dp + 1] = acc[r][1];
    }
    if (wave < R && lane == 0) { s_tm[wave] = m_run; s_tl[wave] = l_run; }
    __syncthreads();

    // ---- both parts together, item (head, channel) ------------------------------------------
#pragma unroll
    for (int k = 0; k < HD; ++k) {
        const int i = tid + k * NT;
        if (i < R * D) {
            const int r = i / D, d = i % D;
            float TA = 0.0f;
#pragma unroll
            for (int g = 0; g < NRG; ++g) TA += s_red[g][r][d];
            const float TL = s_tl[r], t_m = s_tm[r], g_max = s_gmax[r];
            float W = s_W[r], Av = A[k];
            const float tail_lse = TL > 0.0f ? t_m + __logf(TL) : -INFINITY;
            const float n_max = fmaxf(g_max, tail_lse);
            const float n_safe = (n_max == -INFINITY) ? 0.0f : n_max;
            const float rs = (g_max == -INFINITY) ? 0.0f : __expf(g_max - n_safe);
            W *= rs;
            Av *= rs;
            if (TL > 0.0f) {
                const float w = __expf(tail_lse - n_safe);
                W += w;
                Av = fmaf(w, TA / TL, Av);
            }
            a.o[b * a.o_b + (int64_t)(h0 + r) * a.o_h + d] = W > 0.0f ? Av / W : 0.0f;
            if (d == 0) a.lse[b * a.lse_b + h0 + r] = W > 0.0f ? n_max + __logf(W) : -INFINITY;
        }
    }
}

int launch_combine(const CombineArgs& a, int D, hipStream_t st) {
    if (a.S > 512) return -1;
    // Pieces per head.  At batch 1 the kernel is latency bound and 2 pieces measured best (1.4 us
    // per step at 64K less than one, the same as four, 0.5 us less than eight); with many
    // (request, head) pairs the grid fills the chip by itself and one piece repeats no work.
    const bool split2 = a.B * a.Hq < 256;
    const dim3 grid(a.B, a.Hq, split2 ? 2 : 1);
    const bool small = !split2 && a.S <= 64;
    const int R = a.Hq / a.Hkv;
    // a whole kv head per workgroup once those alone are one per compute unit (32 requests of 8 kv
    // heads: 10 against 16 us; 128 requests: 25 against 47 us; with fewer, one workgroup per q head
    // spreads the work better: 16 requests 9.8 against 13 us)
    if (small && (R == 4 || R == 8) && a.Hq == R * a.Hkv && a.B * a.Hkv >= 256) {
        const dim3 g2(a.B, a.Hkv);
        const bool early = a.B * a.Hkv <= 320;       // about one workgroup per compute unit
#define OMMX_GROUPED(DD, RR)                                                                              \
        do {                                                                                              \
            if (early) hipLaunchKernelGGL((combine_grouped_kernel<DD, RR, true>), g2, dim3(512), 0, st, a);  \
            else hipLaunchKernelGGL((combine_grouped_kernel<DD, RR, false>), g2, dim3(512), 0, st, a);       \
        } while (0)
        if (D == 128 && R == 4) OMMX_GROUPED(128, 4);
        else if (D == 128) OMMX_GROUPED(128, 8);
        else if (D == 64 && R == 4) OMMX_GROUPED(64, 4);
        else if (D == 64) OMMX_GROUPED(64, 8);
        else return -1;
#undef OMMX_GROUPED
        return 0;
    }
    if (a.S > 256) {        // 257..512 splits: the same kernel with twice the split slots per thread
        const dim3 g1(a.B, a.Hq, split2 ? 2 : 1);
        if (D == 128 && split2) hipLaunchKernelGGL((combine_kernel<128, 2, 1024, 512>), g1, dim3(1024), 0, st, a);
        else if (D == 128) hipLaunchKernelGGL((combine_kernel<128, 1, 1024, 512>), g1, dim3(1024), 0, st, a);
        else if (D == 64 && split2) hipLaunchKernelGGL((combine_kernel<64, 2, 1024, 512>), g1, dim3(1024), 0, st, a);
        else if (D == 64) hipLaunchKernelGGL((combine_kernel<64, 1, 1024, 512>), g1, dim3(1024), 0, st, a);
        else return -1;
        return 0;
    }
    if (D == 128 && split2) hipLaunchKernelGGL((combine_kernel<128, 2>), grid, dim3(1024), 0, st, a);
    else if (D == 128 && small) hipLaunchKernelGGL((combine_kernel<128, 1, 512, 64>), grid, dim3(512), 0, st, a);
    else if (D == 128) hipLaunchKernelGGL((combine_kernel<128, 1>), grid, dim3(1024), 0, st, a);
    else if (D == 64 && split2) hipLaunchKernelGGL((combine_kernel<64, 2>), grid, dim3(1024), 0, st, a);
    else if (D == 64 && small) hipLaunchKernelGGL((combine_kernel<64, 1, 512, 64>), grid, dim3(512), 0, st, a);
    else if (D == 64) hipLaunchKernelGGL((combine_kernel<64, 1>), grid, dim3(1024), 0, st, a);
    else return -1;
    return 0;
}

}  // namespace ommx

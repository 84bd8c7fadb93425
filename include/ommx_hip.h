/*
 * C ABI of libommx_hip.so: the OMMX paged decode-attention path for AMD gfx950.
 *
 * Three device entry points replace the reference's Python/Triton functions
 * (paths relative to the reference checkout):
 *
 *   ommx_store_pack       <- ommx_gpu_serve/attention/pack.py:293-655
 *                            ommx_pack_kv_canonical_block (quantize-on-store), and the
 *                            slot placement of attention/kv_pool.py:711-734
 *   ommx_decode_splitkv   <- ommx_gpu_serve/attention/paged_decode.py:1255-2284
 *                            _canonical_splitkv_stage1 as launched at :3344-3436
 *   ommx_decode_combine   <- ommx_gpu_serve/attention/paged_decode.py:2366-2500
 *                            _canonical_lse_merge (bf16 tail folded in) at :3528-3549
 *
 * Conventions: every pointer is a device pointer unless its name starts with host_;
 * strides are in ELEMENTS of the pointed-to type; nothing is allocated, freed or
 * retained; nothing synchronises; `stream` is a hipStream_t passed as void*.
 * Return value 0 = launched, negative = argument error (text in ommx_last_error()).
 */
#ifndef OMMX_HIP_H
#define OMMX_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OMMX_ABI_VERSION 8   /* 2: ring, tail-gather, state-merge; 3: index_repr arguments; 4: index-plane conversion;
                                5: decode without a workspace argument; 6: plane extents + error flag on
                                the decode entry points, up to 512 splits; 7: packed_lag on the tail gather;
                                8: tail_rows on the combine and on the decode without a workspace */

/* step of the INT2 quantisers and the dtype of the k_scale / v_scale planes */
#define OMMX_SCALE_POW2_INT8  0
#define OMMX_SCALE_POW2_BF16  1
#define OMMX_SCALE_BF16       2

/* outlier index plane (pack.py:23-40, `outlier_repr`) */
#define OMMX_INDEX_BITMAP   0   /* k_index u8[G,H,D,4]: bit p of the frame = position p (codec.py:330-372) */
#define OMMX_INDEX_RELIDX7  1   /* k_index u8[G,H,D,ceil(7k/8)]: ascending positions, 7 bits each,
                                   least significant bit first (pack.py:128-164) */
#define OMMX_INDEX_COMBINADIC 2 /* k_index u8[G,H,D,ceil(log2 C(gt,k)/8)]: rank sum_i C(p_i, i) of the ascending
                                   positions, little endian (pack.py:179-206, codec.py:131-180); accepted by
                                   ommx_index_convert only: store and decode work on the other two planes */

/* number of floats in the store decision table: 256 pow2 thresholds + 8 FP4 slots */
#define OMMX_STORE_TABLE_FLOATS 264

/* error bits OR-ed into *err_flag by ommx_store_pack */
#define OMMX_ERR_NONFINITE_K   1   /* pack.py:515-538 / codec.py:55-57 */
#define OMMX_ERR_NONFINITE_V   2   /* pack.py:605-607 */
#define OMMX_ERR_UNDERFILLED   4   /* fewer than k distinct outlier lanes, pack.py:520-538 */
#define OMMX_ERR_EXP_RANGE     8   /* scale exponent does not fit the int8 plane */
/* error bit OR-ed into *err_flag by ommx_ring_write / ommx_tail_gather */
#define OMMX_ERR_RING_RANGE   16   /* row outside the history (kv_store_ops.py:33-34,52-53) */
/* error bits OR-ed into *err_flag by the decode entry points */
#define OMMX_ERR_TABLE_RANGE  64   /* a page id or group slot outside the planes (kv_pool.py:526-550 guards these on the host) */
#define OMMX_ERR_VALUE_RANGE 128   /* a K step above 2^15 (K values beyond some 1e5) does not fit the f16 operands of
                                      the matrix-core kernels; it is held at 2^15 and the result is off */
/* not an error: OR-ed into *err_flag by ommx_store_pack when it writes a K step above 2^15, so that the owner
   of the cache can send its decodes to ommx_decode_splitkv_ref before OMMX_ERR_VALUE_RANGE ever happens */
#define OMMX_NOTE_WIDE_STEP  256
/* error bit OR-ed into *err_flag by ommx_index_convert */
#define OMMX_ERR_INDEX_PLANE  32   /* a vector that does not name exactly k positions below group_tokens
                                      (codec.py:173-178 raises ValueError there) */

int ommx_abi_version(void);
const char* ommx_last_error(void);

/*
 * Decision tables of the quantiser, exact-arithmetic defaults (host memory out).
 *   host_table[kb], kb = biased fp32 exponent 0..255: smallest x in that binade with
 *       rint(log2(x)) == kb-127+1, i.e. the first float above sqrt(2)*2^(kb-127)
 *       (pack.py:462 `2^round(log2(scale))`);
 *   host_table[256+j], j = 1..7: smallest |x| that encodes to FP4 level index j
 *       (codec.py:45-65, geometric-mean boundaries, ties to the lower level).
 * A caller that must agree bit-for-bit with a particular libm replaces entries with
 * thresholds measured from that libm and uploads the table to the device.
 */
void ommx_store_default_table(float* host_table);

/*
 * Quantize-on-store: pack T = 32*n tokens of K and V into the ten planes.
 *   K, V          rows [*, H, D]; element type bf16 (in_dtype 0) or fp32 (in_dtype 1);
 *                 row r of head h starts at r*tok_stride + h*head_stride, D contiguous
 *   src_rows      NULL, or int32[T]: source row of packed token t (ring gather)
 *   dst_pages     NULL (identity), or int32[T/page_size]: physical page of logical page
 *   dst_groups    NULL (identity), or int32[T/group_tokens]: group slot of logical group
 *   table         float[OMMX_STORE_TABLE_FLOATS] on the device
 *   planes        as written by pack.py:576-623:
 *                 k_base,v_main u8[P,ps,H,D/4]; k_scale i8[G,H,D]; k_zp,k_ms,k_mc bf16[G,H,D];
 *                 k_index as index_repr says (k_obmp or k_oidx of the reference);
 *                 k_oval u8[G,H,D,ceil(k/2)]; v_scale i8[P,ps,H,D/32]; v_zp bf16[P,ps,H,D/32]
 *                 k_ms and k_mc both NULL: base-shared outliers, the FP4 code is taken of
 *                 (w - zp) / scale and no map planes exist (pack.py:502-506)
 *   scale_mode    how the quantisation step of a vector is formed and stored in k_scale /
 *                 v_scale (pack.py:459-463, 586-590, 612-623):
 *                 OMMX_SCALE_POW2_INT8  2^rint(log2(range/3)), int8 exponent planes
 *                                       (`use_pow2=True`, the serving recipe);
 *                 OMMX_SCALE_POW2_BF16  the same step stored as bf16 (`kv_int8_scale=False`);
 *                 OMMX_SCALE_BF16       bf16(range/3) as it comes (`use_pow2=False`), bf16 planes
 *   select_abs    0: outliers = the ceil(k/2) largest and floor(k/2) smallest values
 *                 (`outlier_select="signed"`, pack.py:436-445); 1: the k largest magnitudes
 *                 (`"abs"`, pack.py:446-448); ties go to the lower position either way
 *   err_flag      NULL or int32[1], OR-ed with OMMX_ERR_* (caller zeroes it)
 *   group_tokens, group_channels   tokens per K vector / channels per V vector, each 16, 32,
 *                 64 or 128 (pack.py:403-408); 32 and 32 is the serving recipe and runs the
 *                 tuned kernel, everything else a general one
 *   v_bf16        1: V is not quantised; v_main is bf16 [P,ps,H,D] (the rows rounded to bf16),
 *                 v_scale is filled with ones and v_zp with zeros (`v_format="bf16"`,
 *                 pack.py:596-602)
 * k_outliers in 0..min(16, group_tokens); D a multiple of 32 and of group_channels, at most 256;
 * T a multiple of group_tokens and page_size; G = T / group_tokens, the bitmap plane has
 * group_tokens / 8 bytes per frame.
 */
int ommx_store_pack(const void* K, const void* V, int in_dtype,
                    int64_t k_tok_stride, int64_t k_head_stride,
                    int64_t v_tok_stride, int64_t v_head_stride,
                    const int32_t* src_rows,
                    int T, int H, int D, int page_size, int k_outliers, int index_repr,
                    int select_abs, int scale_mode, int group_tokens, int group_channels,
                    int v_bf16, const int32_t* dst_pages, const int32_t* dst_groups,
                    const float* table,
                    uint8_t* k_base, void* k_scale, uint16_t* k_zp,
                    uint16_t* k_ms, uint16_t* k_mc, uint8_t* k_index, uint8_t* k_oval,
                    uint8_t* v_main, void* v_scale, uint16_t* v_zp,
                    int32_t* err_flag, void* stream);

/*
 * Split-KV decode over the packed planes (stage 1).
 *   q             bf16 [B,Hq,D], strides q_stride_b, q_stride_h, D contiguous
 *   planes        contiguous, layouts as above; k_outliers in 0..8 with either index
 *                 plane, int8 exponents, and the dedicated FP4 map (the serving recipe) or,
 *                 with k_ms = k_mc = NULL, outliers on the base scale and zero point
 *   req_to_token  int32 or int64 (table_i64) [B, >= ceil((L+off)/ps)], row stride rt_stride
 *   req_to_group  same type [B, >= seg_group_base + ceil(L/group_tokens)], row stride rg_stride
 *   b_seq_len     int32[B] packed tokens per request (device; bounds the loop)
 *   attn_logits   f32 [B,Hq,>=num_splits,D+1] with strides al_stride_b/h/s: partial
 *                 o (normalised) in [0,D) and lse at D; an empty split writes o=0,
 *                 lse=-inf (paged_decode.py:2262-2284)
 * How the tokens are dealt out to the splits is the kernel's own business (the reference rounds
 * ceil(L/S) up to whole groups, paged_decode.py:1429-1432; the serving-recipe kernel deals whole
 * groups out evenly): every split writes its state, an empty one o = 0 and
 * lse = -inf, and ommx_decode_combine weighs the states by their lse.
 * Hq = Hkv * r with r in {1,2,4,8}; D = 128 or 64; num_splits <= 512; planes 8-byte aligned.
 *   group_tokens / group_channels   tokens per K group and channels per V vector: 16, 32, 64, 128
 *   scale_bf16 = 1   k_scale / v_scale hold the steps themselves as bf16, not int8 exponents
 *   v_bf16 = 1       v_main is bf16 [P,ps,H,D]; v_scale / v_zp are ignored
 * The matrix-core kernels run INT2 V, int8 exponents, either outlier map, and, at head_dim 128,
 *   32-token groups with 32-channel V vectors and 6 (or 0) outliers, either index plane;
 *   the same with 1..8 outliers on the bitmap plane, also at head_dim 64 (r in {1,2,4}, Hkv even);
 *   64- or 128-token groups with 32/64/128-channel V vectors and 6 outliers, relidx7 plane;
 *   128-token groups with 10 outliers, relidx7 plane (4 or 8 q heads per kv head).
 * Every other supported shape or recipe (k_outliers up to 16) runs on the plain fp32 kernel.
 *   num_pages, num_group_slots   extents of the planes the tables index (k_base / v_main pages,
 *                 k_scale group slots); the reference guards table entries on the host
 *                 (kv_pool.py:526-550), here an entry outside its plane is clamped into it, so no
 *                 access leaves the planes, and OMMX_ERR_TABLE_RANGE is OR-ed into *err_flag
 *                 (NULL allowed; the caller zeroes it).  0 = extent not given, entries used as
 *                 they are.  A negative b_seq_len counts as 0 and is reported the same way.
 *                 The serving-recipe kernel addresses its planes by 32-bit byte offsets: it runs when
 *                 both extents are given and every plane is below 4 GiB (pages * page_size * Hkv * 32
 *                 bytes of code rows, group slots * Hkv * D * 6 bytes of index plane); other calls run
 *                 on the matrix-core kernel with 64-bit addressing (same results, more time).
 *                 OMMX_ERR_VALUE_RANGE: a K or V step above 2^15 met by the serving-recipe kernel, whose
 *                 f16 operands end there (the step is held at 2^15: finite output, but off); the store
 *                 announces such a cache with OMMX_NOTE_WIDE_STEP, and ommx_decode_splitkv_ref serves it.
 *                 Query elements of any size are served (a query with elements of 128 or more is taken
 *                 divided by a power of two, exactly, and the softmax scale carries the factor).
 */
int ommx_decode_splitkv(const uint16_t* q, int64_t q_stride_b, int64_t q_stride_h,
                        const uint8_t* k_base, const void* k_scale, const uint16_t* k_zp,
                        const uint16_t* k_ms, const uint16_t* k_mc,
                        const uint8_t* k_index, const uint8_t* k_oval,
                        const uint8_t* v_main, const void* v_scale, const uint16_t* v_zp,
                        const void* req_to_token, int64_t rt_stride,
                        const void* req_to_group, int64_t rg_stride, int table_i64,
                        const int32_t* b_seq_len,
                        float* attn_logits, int64_t al_stride_b, int64_t al_stride_h,
                        int64_t al_stride_s,
                        int B, int Hq, int Hkv, int D, int page_size, int k_outliers,
                        int index_repr, int scale_bf16, int group_tokens, int group_channels,
                        int v_bf16, int num_splits, float sm_scale, float logit_cap,
                        int packed_start_offset, int seg_group_base,
                        int num_pages, int num_group_slots, int32_t* err_flag, void* stream);

/*
 * The clamp the decode kernels apply to a page id / group slot read from a table, evaluated on the
 * host: returns the id held inside [0, extent) (unchanged when extent is 0 = not given) and sets
 * *out_of_range (may be NULL) to whether it had to be moved.  For tests of the arithmetic.
 */
int ommx_clamp_table_id(int id, int extent, int* out_of_range);

/*
 * The same operator through the plain fp32 kernel only; identical arguments.  It has no
 * counterpart in the reference: it exists so that tests can cross-check the two device
 * kernels against each other and against the CPU oracle.
 */
int ommx_decode_splitkv_ref(const uint16_t* q, int64_t q_stride_b, int64_t q_stride_h,
                            const uint8_t* k_base, const void* k_scale, const uint16_t* k_zp,
                            const uint16_t* k_ms, const uint16_t* k_mc,
                            const uint8_t* k_index, const uint8_t* k_oval,
                            const uint8_t* v_main, const void* v_scale, const uint16_t* v_zp,
                            const void* req_to_token, int64_t rt_stride,
                            const void* req_to_group, int64_t rg_stride, int table_i64,
                            const int32_t* b_seq_len,
                            float* attn_logits, int64_t al_stride_b, int64_t al_stride_h,
                            int64_t al_stride_s,
                            int B, int Hq, int Hkv, int D, int page_size, int k_outliers,
                            int index_repr, int scale_bf16, int group_tokens, int group_channels,
                            int v_bf16, int num_splits, float sm_scale, float logit_cap,
                            int packed_start_offset, int seg_group_base,
                            int num_pages, int num_group_slots, int32_t* err_flag, void* stream);

/*
 * Split combine with the bf16 sink/recent tail folded in (stage 2).
 *   k_tail,v_tail bf16 [B,Tmax,Hkv,D] with strides t_stride_b/t/h (K and V alike)
 *   b_tail_len    int32[B] valid tail rows (0 allowed)
 *   o             f32 [B,Hq,D] strides o_stride_b/h;  lse f32 [B,Hq] stride lse_stride_b
 * A split with lse = -inf weighs nothing (the reference recomputes which splits are empty from
 * b_seq_len, paged_decode.py:2407-2410; here stage 1 marks them); nothing attended gives o = 0,
 * lse = -inf.
 * b_tail_len == NULL (then k_tail, v_tail, q may be NULL too) combines the splits alone:
 * the un-merged state of a group-range segment (paged_decode.py:2892-2902).
 * k_tail rows must be 16-byte aligned (base pointer and strides multiples of 8 elements);
 * num_splits <= 512.  tail_rows = Tmax, the rows every request's tail buffer holds (0 when
 * unknown): the kernel asks for the first min(64, tail_rows) rows before b_tail_len has
 * arrived, which takes one memory round trip off its critical path; rows past a request's
 * b_tail_len are read but never used, so they only have to be addressable.  With tail_rows
 * given, a b_tail_len above it counts as tail_rows and a negative one as 0: no row address
 * leaves the buffers whatever the length tensor holds.
 */
int ommx_decode_combine(const float* attn_logits, int64_t al_stride_b, int64_t al_stride_h,
                        int64_t al_stride_s,
                        const uint16_t* q, int64_t q_stride_b, int64_t q_stride_h,
                        const uint16_t* k_tail, const uint16_t* v_tail,
                        int64_t kt_stride_b, int64_t kt_stride_t, int64_t kt_stride_h,
                        int64_t vt_stride_b, int64_t vt_stride_t, int64_t vt_stride_h,
                        const int32_t* b_tail_len, const int32_t* b_seq_len,
                        float* o, int64_t o_stride_b, int64_t o_stride_h,
                        float* lse, int64_t lse_stride_b,
                        int B, int Hq, int Hkv, int D, int num_splits, int group_tokens,
                        int tail_rows, float sm_scale, float logit_cap, void* stream);

/*
 * Whole decode step (split-KV stage, then the combine with the bf16 tail) for callers that
 * cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference.
 * Arguments are those of ommx_decode_splitkv and ommx_decode_combine without the workspace:
 * the partial states of the splits are kept in a device array built into the library
 * (2 Mi floats = 8 MiB, held by every GPU the library runs on until the process ends).
 * num_pages / num_group_slots / err_flag as for ommx_decode_splitkv.
 * Limit: B * Hq * (num_splits + 1) * (D + 1) <= 2097152 floats; larger calls return -1 with a
 * message naming the limit.  Calls that overlap in time on one GPU share the array and race;
 * calls on one stream (or otherwise ordered) are safe, and nothing needs clearing between
 * them.  The call makes no hipMalloc / hipFree and nothing that allocates; its first use on a
 * device looks the array's device address up (hipGetSymbolAddress), so make that first call
 * outside stream capture.  seg_group_base is 0 (a segment has no tail to fold in).
 */
int ommx_decode_attention_noalloc(
    const uint16_t* q, int64_t q_stride_b, int64_t q_stride_h,
    const uint8_t* k_base, const void* k_scale, const uint16_t* k_zp,
    const uint16_t* k_ms, const uint16_t* k_mc, const uint8_t* k_index, const uint8_t* k_oval,
    const uint8_t* v_main, const void* v_scale, const uint16_t* v_zp,
    const void* req_to_token, int64_t rt_stride, const void* req_to_group, int64_t rg_stride,
    int table_i64, const int32_t* b_seq_len,
    const uint16_t* k_tail, const uint16_t* v_tail,
    int64_t kt_stride_b, int64_t kt_stride_t, int64_t kt_stride_h,
    int64_t vt_stride_b, int64_t vt_stride_t, int64_t vt_stride_h,
    const int32_t* b_tail_len,
    float* o, int64_t o_stride_b, int64_t o_stride_h, float* lse, int64_t lse_stride_b,
    int B, int Hq, int Hkv, int D, int page_size, int k_outliers, int index_repr, int scale_bf16,
    int group_tokens, int group_channels, int v_bf16, int num_splits, int tail_rows,
    float sm_scale, float logit_cap, int packed_start_offset,
    int num_pages, int num_group_slots, int32_t* err_flag, void* stream);

/*
 * bf16 residual ring, write side: one new K/V row per request.
 * Replaces ommx_gpu_serve/attention/kv_store_ops.py:22-40,63-68 (_kv_write_token /
 * write_token) and the batched scatter of attention/kv_pool.py:407-419.
 *   k, v          bf16 [B,H,D] with strides k_stride_b/h (D contiguous)
 *   k_hist,v_hist bf16 [num_slots, hist_rows, H, D] dense rows; hist_stride_req elements
 *                 between two slots (single-sequence store: num_slots = 1)
 *   slots         NULL (request b lives in slot b) or int64[B]
 *   pos           int64[B] absolute token position of the new row (device)
 *   pos_next      NULL, or int64[B] that receives pos+1 (may alias pos: the device-side
 *                 sequence counter of kv_pool.py:1037-1046 advanced by the same launch)
 * Ring slot of position p (kv_store.py:301-327): p < sink_rows ? p
 * : sink_rows + (p - sink_rows) % ring_span; ring_span == 0 keeps the whole history
 * (slot = position).  A slot outside [0,hist_rows) sets OMMX_ERR_RING_RANGE and the row is
 * not written.
 */
int ommx_ring_write(const uint16_t* k, const uint16_t* v, int64_t k_stride_b, int64_t k_stride_h,
                    int64_t v_stride_b, int64_t v_stride_h,
                    uint16_t* k_hist, uint16_t* v_hist, int64_t hist_stride_req, int hist_rows,
                    const int64_t* slots, const int64_t* pos, int64_t* pos_next,
                    int B, int H, int D, int sink_rows, int ring_span,
                    int32_t* err_flag, void* stream);

/*
 * bf16 residual ring, read side: the sink + recent rows of every request into the fixed
 * tail buffers k_tail, v_tail bf16 [B,T,H,D] (dense).
 * Two modes:
 *   seq != NULL       int64[B] absolute sequence lengths on the device.  The kernel does
 *                     the window arithmetic of attention/kv_pool.py:1048-1105
 *                     (decode_inputs_device): boundary = seq-sink-recent <= 0 ?
 *                     min(sink,seq) : sink + ((seq-sink-recent)/gt)*gt; rows = positions
 *                     [0,min(sink,seq)) ++ [boundary,seq); and writes
 *                     b_tail_len[b] = min(rows, T), b_seq_len[b] = max(boundary-sink, 0)
 *                     (either may be NULL).  Rows past the count repeat position 0; the
 *                     decode kernels mask them by b_tail_len.  packed_lag (0..group_tokens)
 *                     is the number of tokens appended since the planes were last packed:
 *                     the boundary is then the one of seq - packed_lag, so a step that
 *                     appends and decodes before the host packs (one graph replay) reads
 *                     the group its token may have completed from the ring, not from a
 *                     group slot nobody has written yet.  T must hold sink + recent +
 *                     group_tokens - 1 + packed_lag rows, and so must the ring.
 *   tail_idx != NULL  int64[B,T] explicit absolute positions (kv_store_ops.py:42-61,71-76
 *                     _kv_gather_tail / gather_tail); the length outputs are not written.
 * Positions map to history rows as in ommx_ring_write; a row outside the history sets
 * OMMX_ERR_RING_RANGE and yields zeros.
 */
int ommx_tail_gather(const uint16_t* k_hist, const uint16_t* v_hist, int64_t hist_stride_req,
                     int hist_rows, const int64_t* slots, const int64_t* seq,
                     const int64_t* tail_idx,
                     uint16_t* k_tail, uint16_t* v_tail, int32_t* b_tail_len, int32_t* b_seq_len,
                     int B, int T, int H, int D, int sink_rows, int recent_rows, int group_tokens,
                     int ring_span, int packed_lag, int32_t* err_flag, void* stream);

/*
 * Merge of partial attention states over disjoint KV segments (cascade / context-parallel /
 * chunked composition).  Replaces merge_attention_states,
 * ommx_gpu_serve/attention/paged_decode.py:3556-3624 (kernel :2650-2690).
 *   o_parts    f32 [P,R,D] with strides op_stride_p / op_stride_r (D contiguous)
 *   lse_parts  f32 [P,R] with stride lp_stride_p (R contiguous)
 *   valid_lens NULL, or int32[R]: row r uses its first valid_lens[r] parts (negative = all)
 *   o          f32 [R,D] row stride o_stride_r;  lse f32 [R]
 * m = max lse_p, w_p = exp(lse_p - m), o = sum w_p o_p / sum w_p, lse = m + ln sum w_p;
 * a part with lse = -inf weighs nothing; no attended part gives o = 0, lse = -inf.
 */
int ommx_merge_states(const float* o_parts, const float* lse_parts, const int32_t* valid_lens,
                      float* o, float* lse, int P, int R, int D,
                      int64_t op_stride_p, int64_t op_stride_r, int64_t lp_stride_p,
                      int64_t o_stride_r, void* stream);

/*
 * Bytes per K vector of an outlier index plane, 0 if the combination is not supported
 * (1..16 outliers, group_tokens <= 128, combinadic ranks of at most 64 bits).  Replaces
 * combinadic_index_bytes, ommx_gpu_serve/attention/codec.py:131-143, and the plane widths of
 * pack.py:128-164 (position streams) and codec.py:330-372 (bitmask).
 */
int ommx_index_plane_bytes(int index_repr, int group_tokens, int k);

/*
 * Convert the outlier index plane of K groups between the three encodings (bitmask, position
 * streams, combinadic rank).  Replaces _pack_combinadic_frames / _unpack_combinadic_frames
 * (pack.py:179-223), combinadic_to_bitmap (codec.py:239-255) and the plane rewrite of
 * derive_relidx7_from_combinadic (pack.py:662-699), which run on the host one vector at a time.
 *   src / dst  u8 [slots, vectors_per_group, bytes(repr)] contiguous, bytes as ommx_index_plane_bytes
 *   groups     NULL (slots 0..n_groups-1) or int32[n_groups] slots to convert
 * A vector that does not decode to exactly k distinct positions below group_tokens is written
 * as zeros and sets OMMX_ERR_INDEX_PLANE in *err_flag (may be NULL).
 */
int ommx_index_convert(const uint8_t* src, uint8_t* dst, const int32_t* groups, int n_groups,
                       int vectors_per_group, int group_tokens, int k, int src_repr, int dst_repr,
                       int32_t* err_flag, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OMMX_HIP_H */

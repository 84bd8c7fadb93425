// extern "C" entry points of libommx_hip.so for the decode side, argument checks and
// kernel selection.  The store entry point lives beside its kernel in ommx_store.hip.
#include <string>

#include "ommx_decode_args.h"
#include "ommx_ring_args.h"

namespace ommx {

static thread_local std::string g_error;

void set_error(const char* msg) { g_error = msg; }

int launch_decode_fast(const DecodeArgs& a, int D, int R, hipStream_t st);
int launch_decode_gqa4(const DecodeArgs& a, int D, int R, hipStream_t st);

}  // namespace ommx

extern "C" int ommx_abi_version(void) { return OMMX_ABI_VERSION; }

extern "C" const char* ommx_last_error(void) { return ommx::g_error.c_str(); }

// The clamp the decode kernels apply to every page id / group slot they read from a table, on the
// host (for tests of the arithmetic: no kernel has to be given a bad table to check it).
extern "C" int ommx_clamp_table_id(int id, int extent, int* out_of_range) {
    bool bad = false;
    const int r = ommx::clamp_id(id, extent, bad);
    if (out_of_range) *out_of_range = bad ? 1 : 0;
    return r;
}

// The two split-KV entry points take the same arguments and refuse the same ones.
#define OMMX_DECODE_PARAMS                                                                          \
    const uint16_t* q, int64_t q_stride_b, int64_t q_stride_h,                                      \
    const uint8_t* k_base, const void* k_scale, const uint16_t* k_zp,                               \
    const uint16_t* k_ms, const uint16_t* k_mc, const uint8_t* k_index, const uint8_t* k_oval,      \
    const uint8_t* v_main, const void* v_scale, const uint16_t* v_zp,                               \
    const void* req_to_token, int64_t rt_stride, const void* req_to_group, int64_t rg_stride,       \
    int table_i64, const int32_t* b_seq_len,                                                        \
    float* attn_logits, int64_t al_stride_b, int64_t al_stride_h, int64_t al_stride_s,              \
    int B, int Hq, int Hkv, int D, int page_size, int k_outliers, int index_repr, int scale_bf16,   \
    int group_tokens, int group_channels, int v_bf16, int num_splits,                               \
    float sm_scale, float logit_cap, int packed_start_offset, int seg_group_base,                   \
    int num_pages, int num_group_slots, int32_t* err_flag, void* stream
#define OMMX_DECODE_ARGS                                                                            \
    q, q_stride_b, q_stride_h, k_base, k_scale, k_zp, k_ms, k_mc, k_index, k_oval, v_main, v_scale, \
    v_zp, req_to_token, rt_stride, req_to_group, rg_stride, table_i64, b_seq_len, attn_logits,      \
    al_stride_b, al_stride_h, al_stride_s, B, Hq, Hkv, D, page_size, k_outliers, index_repr,        \
    scale_bf16, group_tokens, group_channels, v_bf16, num_splits, sm_scale, logit_cap,              \
    packed_start_offset, seg_group_base, num_pages, num_group_slots, err_flag, stream

namespace ommx {

static bool is_group_size(int g) { return g == 16 || g == 32 || g == 64 || g == 128; }

// Argument checks of the split-KV entry points: nullptr when the call may go ahead, else what
// is wrong with it.  Everything a kernel assumes about shapes and alignment is checked here, on
// the host, before anything is launched.
static const char* check_decode(OMMX_DECODE_PARAMS) {
    (void)q_stride_b; (void)q_stride_h; (void)rt_stride; (void)rg_stride; (void)table_i64;
    (void)al_stride_b; (void)al_stride_h; (void)al_stride_s; (void)scale_bf16; (void)v_bf16;
    (void)k_scale; (void)v_scale;
    (void)sm_scale; (void)logit_cap; (void)stream; (void)err_flag;
    if (num_pages < 0 || num_group_slots < 0) return "num_pages / num_group_slots must be >= 0 (0 = not given)";
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv)
        return "q heads must be a positive multiple of kv heads";
    const int R = Hq / Hkv;
    if (!(R == 1 || R == 2 || R == 4 || R == 8) || !(D == 64 || D == 128))
        return "supported shapes are head_dim 64|128 and 1|2|4|8 q heads per kv head";
    if (!is_group_size(group_tokens) || !is_group_size(group_channels) || D % group_channels)
        return "group_tokens / group_channels must be 16, 32, 64 or 128";
    if (page_size <= 0 || group_tokens % page_size) return "page_size must divide the K group";
    if (packed_start_offset < 0 || packed_start_offset >= page_size || seg_group_base < 0)
        return "packed_start_offset must be in [0,page_size), seg_group_base >= 0";
    if (k_outliers < 0 || k_outliers > 16 || k_outliers > group_tokens || num_splits < 1 ||
        num_splits > 512 || (index_repr != 0 && index_repr != 1))
        return "k_outliers in [0,min(16,group_tokens)], num_splits in [1,512], index_repr 0|1";
    if ((reinterpret_cast<uintptr_t>(k_base) | reinterpret_cast<uintptr_t>(v_main) |
         reinterpret_cast<uintptr_t>(v_zp) | reinterpret_cast<uintptr_t>(k_index) |
         reinterpret_cast<uintptr_t>(k_oval) | reinterpret_cast<uintptr_t>(k_zp) |
         reinterpret_cast<uintptr_t>(k_ms) | reinterpret_cast<uintptr_t>(k_mc)) & 7)
        return "planes must be 8-byte aligned";
    // (plane pointers may be null: an empty cache is legal when every b_seq_len is zero, and then
    // no plane is read)
    if (!q || !b_seq_len || !attn_logits || !req_to_token || !req_to_group) return "null pointer";
    if ((k_outliers > 0 && (!k_index || !k_oval)) || (!k_ms != !k_mc)) return "outlier planes missing";
    return nullptr;
}

static DecodeArgs make_decode_args(OMMX_DECODE_PARAMS) {
    (void)D; (void)stream;
    return DecodeArgs{q, q_stride_b, q_stride_h, k_base, static_cast<const int8_t*>(k_scale), k_zp, k_ms, k_mc,
                      k_index, k_oval, v_main, static_cast<const int8_t*>(v_scale), v_zp, req_to_token, rt_stride,
                      req_to_group, rg_stride, table_i64, b_seq_len, attn_logits, al_stride_b, al_stride_h,
                      al_stride_s, B, Hq, Hkv, page_size, k_outliers, num_splits, sm_scale, logit_cap,
                      packed_start_offset, seg_group_base, index_repr, scale_bf16 ? 1 : 0,
                      group_tokens, group_channels, v_bf16 ? 1 : 0, num_pages, num_group_slots, err_flag};
}

static void set_error2(const char* where, const char* what) { g_error = std::string(where) + ": " + what; }

}  // namespace ommx

extern "C" int ommx_decode_splitkv(OMMX_DECODE_PARAMS) {
    using namespace ommx;
    if (const char* bad = check_decode(OMMX_DECODE_ARGS)) { set_error2("ommx_decode_splitkv", bad); return -1; }
    const DecodeArgs a = make_decode_args(OMMX_DECODE_ARGS);
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc = launch_decode_gqa4(a, D, Hq / Hkv, st);
    if (rc == 1) rc = launch_decode_fast(a, D, Hq / Hkv, st);
    if (rc == 1) rc = launch_decode_ref(a, D, Hq / Hkv, st);      // shapes the matrix-core kernel leaves out
    if (rc != 0) { set_error("ommx_decode_splitkv: no kernel for this shape"); return -1; }
    if (hipGetLastError() != hipSuccess) { set_error("ommx_decode_splitkv: launch failed"); return -2; }
    return 0;
}

// Same operator through the plain fp32 kernel only (cross-check entry used by tests).
extern "C" int ommx_decode_splitkv_ref(OMMX_DECODE_PARAMS) {
    using namespace ommx;
    if (const char* bad = check_decode(OMMX_DECODE_ARGS)) { set_error2("ommx_decode_splitkv_ref", bad); return -1; }
    const DecodeArgs a = make_decode_args(OMMX_DECODE_ARGS);
    if (launch_decode_ref(a, D, Hq / Hkv, static_cast<hipStream_t>(stream)) != 0) {
        set_error("ommx_decode_splitkv_ref: unsupported shape");
        return -1;
    }
    if (hipGetLastError() != hipSuccess) { set_error("ommx_decode_splitkv_ref: launch failed"); return -2; }
    return 0;
}

extern "C" int ommx_decode_combine(
    const float* attn_logits, int64_t al_stride_b, int64_t al_stride_h, int64_t al_stride_s,
    const uint16_t* q, int64_t q_stride_b, int64_t q_stride_h,
    const uint16_t* k_tail, const uint16_t* v_tail,
    int64_t kt_stride_b, int64_t kt_stride_t, int64_t kt_stride_h,
    int64_t vt_stride_b, int64_t vt_stride_t, int64_t vt_stride_h,
    const int32_t* b_tail_len, const int32_t* b_seq_len,
    float* o, int64_t o_stride_b, int64_t o_stride_h, float* lse, int64_t lse_stride_b,
    int B, int Hq, int Hkv, int D, int num_splits, int group_tokens, int tail_rows, float sm_scale,
    float logit_cap, void* stream) {
    using namespace ommx;
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || num_splits < 1 || !(D == 64 || D == 128) ||
        group_tokens < 16 || group_tokens > 128 || (group_tokens & (group_tokens - 1)) || tail_rows < 0) {
        set_error("ommx_decode_combine: bad shape");
        return -1;
    }
    if (!attn_logits || !o || !lse || !b_seq_len) { set_error("ommx_decode_combine: null pointer"); return -1; }
    if (b_tail_len && (!k_tail || !v_tail || !q)) {
        set_error("ommx_decode_combine: tail lengths given without tail rows");
        return -1;
    }
    if (b_tail_len && ((reinterpret_cast<uintptr_t>(k_tail) & 15) || kt_stride_b % 8 ||
                       kt_stride_t % 8 || kt_stride_h % 8)) {
        set_error("ommx_decode_combine: k_tail rows must be 16-byte aligned (strides multiples of 8)");
        return -1;
    }
    if (num_splits > 512) {
        set_error("ommx_decode_combine: at most 512 KV splits");
        return -1;
    }
    CombineArgs a{attn_logits, al_stride_b, al_stride_h, al_stride_s, q, q_stride_b, q_stride_h,
                  k_tail, v_tail, kt_stride_b, kt_stride_t, kt_stride_h,
                  vt_stride_b, vt_stride_t, vt_stride_h, b_tail_len, b_seq_len,
                  o, o_stride_b, o_stride_h, lse, lse_stride_b, B, Hq, Hkv, num_splits,
                  sm_scale, logit_cap, group_tokens, b_tail_len ? tail_rows : 0};
    if (launch_combine(a, D, static_cast<hipStream_t>(stream)) != 0) {
        set_error("ommx_decode_combine: unsupported head_dim");
        return -1;
    }
    if (hipGetLastError() != hipSuccess) { set_error("ommx_decode_combine: launch failed"); return -2; }
    return 0;
}

// bf16 residual ring: one new K/V row per request (kv_store_ops.py:63-68, kv_pool.py:407-419).
extern "C" int ommx_ring_write(
    const uint16_t* k, const uint16_t* v, int64_t k_stride_b, int64_t k_stride_h,
    int64_t v_stride_b, int64_t v_stride_h,
    uint16_t* k_hist, uint16_t* v_hist, int64_t hist_stride_req, int hist_rows,
    const int64_t* slots, const int64_t* pos, int64_t* pos_next,
    int B, int H, int D, int sink_rows, int ring_span, int32_t* err_flag, void* stream) {
    using namespace ommx;
    if (B <= 0 || H <= 0 || D <= 0 || hist_rows <= 0 || sink_rows < 0 || ring_span < 0) {
        set_error("ommx_ring_write: bad shape");
        return -1;
    }
    if (!k || !v || !k_hist || !v_hist || !pos) { set_error("ommx_ring_write: null pointer"); return -1; }
    if (ring_span > 0 && sink_rows + ring_span > hist_rows) {
        set_error("ommx_ring_write: sink_rows + ring_span exceeds the history rows");
        return -1;
    }
    RingArgs a{k_hist, v_hist, hist_stride_req, hist_rows, sink_rows, ring_span, H, D, slots, err_flag};
    launch_ring_write(a, k, v, k_stride_b, k_stride_h, v_stride_b, v_stride_h, pos, pos_next, B,
                      static_cast<hipStream_t>(stream));
    if (hipGetLastError() != hipSuccess) { set_error("ommx_ring_write: launch failed"); return -2; }
    return 0;
}

// Tail rows (sink + recent) of every request into the fixed tail buffers, plus the packed /
// tail lengths of the decode call (kv_pool.py:1048-1105, kv_store_ops.py:71-76).
extern "C" int ommx_tail_gather(
    const uint16_t* k_hist, const uint16_t* v_hist, int64_t hist_stride_req, int hist_rows,
    const int64_t* slots, const int64_t* seq, const int64_t* tail_idx,
    uint16_t* k_tail, uint16_t* v_tail, int32_t* b_tail_len, int32_t* b_seq_len,
    int B, int T, int H, int D, int sink_rows, int recent_rows, int group_tokens, int ring_span,
    int packed_lag, int32_t* err_flag, void* stream) {
    using namespace ommx;
    if (B <= 0 || T <= 0 || H <= 0 || D <= 0 || hist_rows <= 0 || sink_rows < 0 || ring_span < 0 ||
        recent_rows < 0 || group_tokens <= 0 || packed_lag < 0 || packed_lag > group_tokens) {
        set_error("ommx_tail_gather: bad shape");
        return -1;
    }
    if (!k_hist || !v_hist || !k_tail || !v_tail || (!seq && !tail_idx)) {
        set_error("ommx_tail_gather: null pointer (one of seq, tail_idx is required)");
        return -1;
    }
    if (seq && tail_idx) { set_error("ommx_tail_gather: pass seq or tail_idx, not both"); return -1; }
    if (ring_span > 0 && sink_rows + ring_span > hist_rows) {
        set_error("ommx_tail_gather: sink_rows + ring_span exceeds the history rows");
        return -1;
    }
    RingArgs a{const_cast<uint16_t*>(k_hist), const_cast<uint16_t*>(v_hist), hist_stride_req,
               hist_rows, sink_rows, ring_span, H, D, slots, err_flag};
    if (seq && ring_span > 0 && recent_rows + group_tokens - 1 + packed_lag > ring_span) {
        set_error("ommx_tail_gather: the ring is too short for recent_rows + a group + packed_lag");
        return -1;
    }
    if (seq && T < sink_rows + recent_rows + group_tokens - 1 + packed_lag) {
        // the tail of a request can hold that many rows (sink, recent, a group short of one token, the lag);
        // the kernel writes min(rows, T), sink rows first, so a shorter buffer would drop the newest tokens
        set_error("ommx_tail_gather: T is below sink_rows + recent_rows + group_tokens - 1 + packed_lag");
        return -1;
    }
    launch_tail_gather(a, seq, tail_idx, k_tail, v_tail, B, T, recent_rows, group_tokens,
                       packed_lag, b_tail_len, b_seq_len, static_cast<hipStream_t>(stream));
    if (hipGetLastError() != hipSuccess) { set_error("ommx_tail_gather: launch failed"); return -2; }
    return 0;
}

// ---- decode without a workspace argument ------------------------------------------------------
// The partial states of the splits live in a file-scope device array instead of a caller
// workspace, so the call allocates nothing.  Every GPU the library runs on holds its own copy of
// the array (at its own address) until the process ends; calls on one GPU share it, so two calls
// that overlap on one GPU (different streams) race.  Stage 1 writes every (request, head, split)
// state the combine reads, empty splits included, so nothing has to be cleared between calls.
#define OMMX_NOALLOC_SCRATCH_FLOATS (2u * 1024u * 1024u)     /* 8 MiB */
static __device__ __align__(256) float scratch[OMMX_NOALLOC_SCRATCH_FLOATS];

namespace ommx {
namespace {
constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices];        // device address of `scratch` per device, 0 = not asked yet
}  // namespace

// Device address of this device's copy of `scratch` (the array's name is only a host-side
// handle: kernels and copies need the address hipGetSymbolAddress returns).
static float* scratch_on_current_device(const char** why) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        *why = "cannot tell the current device";
        return nullptr;
    }
    float* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (p) return p;
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) {
        (void)hipGetLastError();
        *why = "hipGetSymbolAddress failed for the scratch array";
        return nullptr;
    }
    p = static_cast<float*>(sym);
    __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);
    return p;
}
}  // namespace ommx

extern "C" int ommx_decode_attention_noalloc(
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
    int num_pages, int num_group_slots, int32_t* err_flag, void* stream) {
    using namespace ommx;
    const char* where = "ommx_decode_attention_noalloc";
    if (B <= 0 || Hq <= 0 || D <= 0 || num_splits < 1 || num_splits > 512) {
        set_error2(where, "bad shape");
        return -1;
    }
    const int64_t al_stride_s = D + 1, al_stride_h = (int64_t)(num_splits + 1) * al_stride_s,
                  al_stride_b = (int64_t)Hq * al_stride_h;
    const int64_t need = (int64_t)B * al_stride_b;
    if (need > (int64_t)OMMX_NOALLOC_SCRATCH_FLOATS) {
        g_error = std::string(where) + ": B*Hq*(num_splits+1)*(D+1) = " + std::to_string(need) +
                  " floats of split states exceed the built-in scratch of " +
                  std::to_string(OMMX_NOALLOC_SCRATCH_FLOATS) +
                  " floats (8 MiB); use fewer splits or ommx_decode_splitkv + ommx_decode_combine "
                  "with a caller workspace";
        return -1;
    }
    const char* why = nullptr;
    float* ws = scratch_on_current_device(&why);
    if (!ws) { set_error2(where, why); return -3; }
    int rc = ommx_decode_splitkv(q, q_stride_b, q_stride_h, k_base, k_scale, k_zp, k_ms, k_mc, k_index,
                                 k_oval, v_main, v_scale, v_zp, req_to_token, rt_stride, req_to_group,
                                 rg_stride, table_i64, b_seq_len, ws, al_stride_b, al_stride_h,
                                 al_stride_s, B, Hq, Hkv, D, page_size, k_outliers, index_repr,
                                 scale_bf16, group_tokens, group_channels, v_bf16, num_splits,
                                 sm_scale, logit_cap, packed_start_offset, 0, num_pages, num_group_slots,
                                 err_flag, stream);
    if (rc != 0) return rc;
    return ommx_decode_combine(ws, al_stride_b, al_stride_h, al_stride_s, q, q_stride_b, q_stride_h,
                               k_tail, v_tail, kt_stride_b, kt_stride_t, kt_stride_h, vt_stride_b,
                               vt_stride_t, vt_stride_h, b_tail_len, b_seq_len, o, o_stride_b,
                               o_stride_h, lse, lse_stride_b, B, Hq, Hkv, D, num_splits, group_tokens,
                               tail_rows, sm_scale, logit_cap, stream);
}

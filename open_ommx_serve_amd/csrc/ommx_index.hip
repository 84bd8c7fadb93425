// Conversion between the three outlier-position planes of the K groups: flat bitmask
// (group_tokens / 8 bytes per vector), 7-bit position streams (ceil(7k/8) bytes) and the
// combinadic rank (ceil(log2 C(group_tokens, k) / 8) bytes, little endian), which is the storage
// floor.  All three name the same k positions of a vector (membership equivalence,
// ommx_gpu_serve/attention/pack.py:323-326); the rank of ascending positions p_1 < ... < p_k is
// sum_i C(p_i, i) (ommx_gpu_serve/attention/codec.py:146-180), and unranking is the greedy
// inverse from i = k down.  The reference ranks and unranks on the host with big integers, one
// vector at a time (pack.py:179-223); here one thread converts one vector.
#include "ommx_common.h"

namespace ommx {
namespace {

constexpr int MAX_POS = 128, MAX_K = 16;
struct Binom { uint64_t c[MAX_POS + 1][MAX_K + 1]; };
// Pascal's triangle, saturating (entries beyond 2^64 are never used: the host refuses ranks
// wider than 8 bytes, and every term C(p, i) of such a rank is at most the rank's bound)
constexpr Binom make_binom() {
    Binom b{};
    for (int n = 0; n <= MAX_POS; ++n) {
        b.c[n][0] = 1;
        for (int i = 1; i <= MAX_K; ++i) {
            if (n == 0) { b.c[n][i] = 0; continue; }
            const uint64_t x = b.c[n - 1][i - 1], y = b.c[n - 1][i];
            b.c[n][i] = (x > ~0ull - y) ? ~0ull : x + y;
        }
    }
    return b;
}
__device__ const Binom kBinom = make_binom();

// 128-bit values as two named halves: a dynamically indexed two-element array would live in
// scratch memory
struct U128 { uint64_t lo, hi; };
__device__ __forceinline__ void or_shifted(U128& v, uint64_t x, int bit) {     // v |= x << bit
    if (bit < 64) {
        v.lo |= x << bit;
        if (bit > 0) v.hi |= x >> (64 - bit);
    } else {
        v.hi |= x << (bit - 64);
    }
}
__device__ __forceinline__ uint32_t bits_at(const U128& v, int bit) {         // low 32 bits of v >> bit
    if (bit >= 64) return static_cast<uint32_t>(v.hi >> (bit - 64));
    uint64_t r = v.lo >> bit;
    if (bit > 32) r |= v.hi << (64 - bit);
    return static_cast<uint32_t>(r);
}
__device__ __forceinline__ U128 load_bytes(const uint8_t* s, int n) {
    U128 v{0, 0};
    for (int i = 0; i < n; ++i) or_shifted(v, s[i], 8 * i);
    return v;
}
__device__ __forceinline__ void store_bytes(uint8_t* d, int n, const U128& v) {
    for (int i = 0; i < n; ++i) d[i] = static_cast<uint8_t>(bits_at(v, 8 * i));
}

struct IndexArgs {
    const uint8_t* src;
    uint8_t* dst;
    const int32_t* groups;     // group slots to convert, or NULL: slots 0 .. n_groups-1
    int n_groups, vecs, gt, k, src_repr, dst_repr, src_bytes, dst_bytes;
    int32_t* err;
};

__global__ void __launch_bounds__(256) index_convert_kernel(IndexArgs a) {
    // the binomials this launch can touch, C(c, i) for c < group_tokens and i <= k, staged in LDS:
    // the unranking loop reads them at lane-dependent indices
    __shared__ uint64_t tab[MAX_POS * (MAX_K + 1)];
    const int tw = a.k + 1;
    if (a.src_repr == OMMX_INDEX_COMBINADIC || a.dst_repr == OMMX_INDEX_COMBINADIC) {
        for (int e = threadIdx.x; e < a.gt * tw; e += blockDim.x) tab[e] = kBinom.c[e / tw][e % tw];
        __syncthreads();
    }
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= static_cast<int64_t>(a.n_groups) * a.vecs) return;
    const int gi = static_cast<int>(t / a.vecs);
    const int64_t slot = a.groups ? a.groups[gi] : gi;
    const int64_t vec = slot * a.vecs + (t - static_cast<int64_t>(gi) * a.vecs);
    const uint8_t* s = a.src + vec * a.src_bytes;
    uint8_t* d = a.dst + vec * a.dst_bytes;
    // ---- positions of the vector as a 128-bit occupancy mask ------------------------
    U128 occ{0, 0};
    bool bad = false;
    const U128 w = load_bytes(s, a.src_bytes);
    if (a.src_repr == OMMX_INDEX_BITMAP) {
        occ = w;
    } else if (a.src_repr == OMMX_INDEX_RELIDX7) {
        for (int i = 0; i < a.k; ++i) {
            const int p = static_cast<int>(bits_at(w, 7 * i) & 127u);
            if (p >= a.gt) bad = true;
            else or_shifted(occ, 1, p);
        }
    } else {   // combinadic rank (at most 64 bits): greedy unranking, largest position first
        // One pass down the positions with the level i as lane state (every lane makes the same
        // group_tokens steps): position c is taken at level i iff C(c, i) still fits the rest,
        // which is the largest such c below the position taken before it.
        uint64_t rem = w.lo;
        int i = a.k;
        for (int c = a.gt - 1; c >= 0; --c) {
            const uint64_t b = tab[c * tw + i];
            if (i >= 1 && b <= rem) {
                rem -= b;
                or_shifted(occ, 1, c);
                --i;
            }
        }
        if (rem != 0 || i != 0) bad = true;
    }
    if (__popcll(occ.lo) + __popcll(occ.hi) != a.k) bad = true;   // a vector holds exactly k outliers
    if (bad) {
        if (a.err) atomicOr(a.err, OMMX_ERR_INDEX_PLANE);
        for (int i = 0; i < a.dst_bytes; ++i) d[i] = 0;
        return;
    }
    // ---- write the destination plane ---------------------------------------------------
    if (a.dst_repr == OMMX_INDEX_BITMAP) {
        store_bytes(d, a.dst_bytes, occ);
        return;
    }
    U128 out{0, 0};
    int i = 0;
    for (int half = 0; half < 2; ++half) {
        uint64_t m = half ? occ.hi : occ.lo;
        while (m) {
            const int p = 64 * half + __builtin_ctzll(m);
            m &= m - 1;
            if (a.dst_repr == OMMX_INDEX_RELIDX7) or_shifted(out, static_cast<uint64_t>(p), 7 * i);
            else out.lo += tab[p * tw + i + 1];
            ++i;
        }
    }
    store_bytes(d, a.dst_bytes, out);
}

// bytes per vector of an index plane; 0 = unsupported
int plane_bytes(int repr, int gt, int k) {
    if (repr == OMMX_INDEX_BITMAP) return (gt + 7) / 8;
    if (repr == OMMX_INDEX_RELIDX7) return (7 * k + 7) / 8;
    if (repr != OMMX_INDEX_COMBINADIC) return 0;
    // ceil(log2 C(gt, k)) bits; wider than 64 is refused
    const Binom b = make_binom();
    const uint64_t total = b.c[gt][k];
    if (total == ~0ull) return 0;
    int bits = 0;
    for (uint64_t v = total - 1; v; v >>= 1) ++bits;
    if (bits < 1) bits = 1;
    return (bits + 7) / 8;
}

}  // namespace
}  // namespace ommx

extern "C" int ommx_index_plane_bytes(int index_repr, int group_tokens, int k) {
    if (k <= 0 || k > ommx::MAX_K || group_tokens <= 0 || group_tokens > ommx::MAX_POS || k >= group_tokens)
        return 0;
    return ommx::plane_bytes(index_repr, group_tokens, k);
}

extern "C" int ommx_index_convert(const uint8_t* src, uint8_t* dst, const int32_t* groups, int n_groups,
                                  int vectors_per_group, int group_tokens, int k, int src_repr,
                                  int dst_repr, int32_t* err_flag, void* stream) {
    using namespace ommx;
    if (!src || !dst) { set_error("ommx_index_convert: null pointer"); return -1; }
    if (n_groups < 0 || vectors_per_group <= 0) { set_error("ommx_index_convert: bad shape"); return -1; }
    if (group_tokens % 8 != 0) { set_error("ommx_index_convert: group_tokens must be a multiple of 8"); return -1; }
    const int sb = ommx_index_plane_bytes(src_repr, group_tokens, k);
    const int db = ommx_index_plane_bytes(dst_repr, group_tokens, k);
    if (sb == 0 || db == 0) {
        set_error("ommx_index_convert: unsupported plane (1..16 outliers, group_tokens <= 128, rank <= 64 bits)");
        return -1;
    }
    if (n_groups == 0) return 0;
    IndexArgs a{src, dst, groups, n_groups, vectors_per_group, group_tokens, k, src_repr, dst_repr, sb, db, err_flag};
    const int64_t total = static_cast<int64_t>(n_groups) * vectors_per_group;
    const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
    hipLaunchKernelGGL(index_convert_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), a);
    if (hipGetLastError() != hipSuccess) { set_error("ommx_index_convert: launch failed"); return -2; }
    return 0;
}

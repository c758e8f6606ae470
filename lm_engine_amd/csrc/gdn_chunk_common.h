// Types and device helpers shared by the chunked-forward kernels of the gated delta rule.
#pragma once

#include "gdn_common.h"

namespace gdn {

constexpr int C = 64;  // chunk length
constexpr int GDN_CYCLE_BUDGET_SLOTS = 64;  // sampled workgroups of the measurement build
constexpr int GDN_LOCAL_CYCLE_SLOTS = 32;   // of them the chunk-local backward kernel uses two each (16 counters per workgroup)
constexpr int PREP_THREADS = 256;
constexpr int FRAG_BYTES = WAVE * 16;  // one MFMA operand fragment: 8 bf16 per lane

// head of q and k that value head h reads
__host__ __device__ inline int qk_head_of(int h, int qk_div) { return qk_div > 1 ? h / qk_div : h; }

struct ChunkParams {
    const bf16_t* q;
    const bf16_t* k;
    const bf16_t* v;
    const void* beta;
    const float* g;
    const float* h0;
    float* ht;
    bf16_t* o;
    const int32_t* cu_seqlens;  // packed sequences (B == 1), else NULL
    const int32_t* pad_lens;    // left-padded batch: prefix sums of the valid lengths, else NULL
    int32_t* chunk_off;  // [N + 1] prefix of chunks per sequence (packed input only)
    int32_t* seq_order;  // [N] the sequences by decreasing number of chunks (packed input only)
    uint8_t* rec;        // workspace records, [H][TC]
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    int64_t o_stride_b, o_stride_t, o_stride_h;
    int B, T, H, V, N;
    int qk_div;  // value heads per head of q and k (grouped value attention): head h reads q and k of head h / qk_div
    // Mirror reads (the reverse sweep of the backward pass on the scan without output): the sequence the scan walks is
    // the caller's sequence backwards, every chunk twice - chunk 2 r takes its rows of k from k and of v from v, chunk
    // 2 r + 1 from k2 and v2, both as tokens 64 (NT / 2 - 1 - r) + 63 - row of those tensors ([N, T / 2, H, .]).
    int mirror;
    int save_sliced;  // bf16 staged saves: [entry][V / 32 slices][rows][32] instead of [entry][rows][V]
    const bf16_t* k2;
    const bf16_t* v2;
    int64_t k2_stride_b, k2_stride_t, k2_stride_h;
    int64_t v2_stride_b, v2_stride_t, v2_stride_h;
    int NT;  // chunks per sequence (fixed-length input)
    int TC;  // chunk slots per head
    int beta_dtype;
    int l2norm;
    float scale;
    uint32_t rec_bytes, off_qs, off_ks, off_cs, off_p, off_eg;
    int scan_groups;  // workgroups per (sequence, head) in the scan kernel
    // training support: when set, the scan also writes the fp32 state every
    // chunk starts from, [N * H][save_nc][K][V], and V~ of every chunk, [N * H][save_nc][64][V]
    float* save_state;
    float* save_vnew;
    int save_nc;
    int save_every;    // only chunks c with c % save_every == 0 are saved, as entry c / save_every ...
    int save_reverse;  // ... or, when set, as entry save_nc - 1 - c / save_every
    const int32_t* row_order;  // left-padded rows of given records: the order in which the rows' chains are dealt out (or NULL)
    int save_state_bf16, save_vnew_bf16;  // that array is bf16 (the pointer then points at bf16 data); staged saves only
    int no_output;     // the scan writes no output (a sweep of the backward pass); staged saves only
    int records_given;  // the records are already in place: prepare is not run
    int32_t* ready;     // [H][TC] one flag per record, for the launch that runs prepare and scan together
    int fused;          // that launch was asked for (GDN_FLAG_FUSED_LAUNCH)
    int ready_clear;    // the caller vouches that the ready flags are zero (GDN_FLAG_READY_FLAGS_CLEAR)
    int32_t* err;         // error latch in the workspace header: set when a scan workgroup of that launch gave up waiting
    int32_t* err_caller;  // the caller's own error word (gdn_args::error_word) or NULL
    uint32_t spin_limit;  // polls of a ready flag before giving up
    int no_producers;     // GDN_FLAG_DEBUG_NO_PRODUCERS
    uint64_t* cycle_out;  // measurement build (GDN_CYCLE_BUDGET) only: where sampled waves of the half-slice scan report; else NULL
    int rec16;          // the fragments of T diag(beta) and P are laid out for v_mfma_f32_16x16x32_bf16 (the half-slice scan)
};

// The shapes the one-launch forward is used for: its scan workgroups (one per 64 columns of every chain, the chains rounded
// up to a multiple of 8) fill between 3/8 and 1/2 of the compute units.  With fewer chains the two-kernel path's scan, one
// slice per CU, is the faster one and prepare is short; with more, too few CUs are left for the producers.
// And the chains number at least 5/32 of the CUs (40 of 256).  Per chunk of a chain the one-launch scan (a pair of waves
// per slice, two slices per CU) is ~0.4 us slower than the half-slice scan of the two-kernel path, and what it saves is
// the prepare kernel, ~0.0115 us per chunk and chain: both grow with the sequence length, so the sign of the difference
// depends on the number of chains alone.  Measured at steady clocks: 64 chains (B = 4, H = 16, V = 128) 0.111 ms in one
// launch against 0.114 ms; 32 chains (H = 32, V = 256, T = 65536) 1.645 ms against 1.565 ms.
inline bool fused_launch_window(int64_t chains, int V, int num_cus) {
    const int64_t scan_wgs = (chains + 7) / 8 * 8 * (V / 64);
    return scan_wgs <= (int64_t)num_cus / 2 && scan_wgs >= (int64_t)num_cus * 3 / 8 && chains * 32 >= (int64_t)num_cus * 5;
}

// Kernel choice of the scan (plan_scan, gdn_chunk32.hip)
struct ScanPlan {
    int nw;             // 32-column slices per workgroup
    bool half;          // a slice is scanned by two waves of 16 columns (records in the 16x16x32 fragment order)
    bool staged_saves;  // a saving scan whose saves go through LDS and the store wave: only there bf16 saves exist
    bool no_output;     // the scan without output runs
};
// what a saving launch asks for (gdn_chunk_saves)
struct SaveRequest {
    bool no_output = false, has_state = true, has_vnew = true, state_bf16 = false, vnew_bf16 = false;
    int save_every = 1;
};
ScanPlan plan_scan(int K, int64_t chains, int V, bool packed, bool save, int records_given, int num_cus, const SaveRequest& req);

struct RecordLayout {
    uint32_t off_p, off_qs, off_ks, off_cs, off_eg, bytes;
};

// Record of one (head, chunk), the same for every K and V: the 6 non-zero fragments of T diag(beta) (T = (I + A)^-1)
// at 0, the 6 non-zero fragments of P, then three vectors of 64 fp32 row scales - of q at off_qs
// (e^{gamma} scale / |q|), of k for the state update at off_ks (e^{gamma_C - gamma} / |k|), of k S0 at off_cs
// (e^{gamma} / |k|) - and e^{gamma_C}.  q, k and v themselves are read from the caller's tensors by the scan, which
// forms V~ = T diag(beta) (V - diag(cs) K S0) itself: the record depends neither on V nor on the key dim.
inline RecordLayout record_layout(int K, int V) {
    (void)K, (void)V;
    RecordLayout r;
    r.off_p = 6 * FRAG_BYTES;
    r.off_qs = r.off_p + 6 * FRAG_BYTES;
    r.off_ks = r.off_qs + C * 4;
    r.off_cs = r.off_ks + C * 4;
    r.off_eg = r.off_cs + C * 4;
    r.bytes = (r.off_eg + 4 + 255u) & ~255u;
    return r;
}

// Where chunk slot `slot` of the grid lives: sequence, first token, valid length (0 = unused slot).
struct ChunkCoord {
    int n;
    int64_t b, t0;
    int len;
};

__device__ __forceinline__ ChunkCoord locate_chunk(const ChunkParams& p, int slot) {
    ChunkCoord cc;
    if (slot >= p.TC) {  // past the last slot (the item grid of prepare is rounded up): nothing there
        cc.n = 0, cc.b = 0, cc.t0 = 0, cc.len = 0;
        return cc;
    }
    if (p.cu_seqlens == nullptr) {
        cc.n = slot / p.NT;
        const int c = slot - cc.n * p.NT;
        cc.b = cc.n;
        // the last `len` tokens of the row (clamped: a malformed prefix must not send a load out of the row)
        const int len = p.pad_lens == nullptr ? p.T : min(max(p.pad_lens[cc.n + 1] - p.pad_lens[cc.n], 0), p.T);
        cc.t0 = (int64_t)(p.T - len) + (int64_t)c * C;
        cc.len = min(C, len - c * C);
        return cc;
    }
    cc.b = 0;
    if (slot >= p.chunk_off[p.N]) {
        cc.n = 0, cc.t0 = 0, cc.len = 0;
        return cc;
    }
    int lo = 0, hi = p.N;  // largest n with chunk_off[n] <= slot
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (p.chunk_off[mid] <= slot) lo = mid;
        else hi = mid;
    }
    cc.n = lo;
    const int c = slot - p.chunk_off[lo];
    int t0, len;
    packed_bounds(p.cu_seqlens, lo, p.T, t0, len);
    cc.t0 = (int64_t)t0 + (int64_t)c * C;
    cc.len = min(C, len - c * C);
    return cc;
}

__device__ __forceinline__ f32x4 mfma_bf16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ f32x4 mfma_f32(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 pack8(f32x4 lo, f32x4 hi) {
    bf16x8 r;
    r[0] = (bf16_t)lo[0], r[1] = (bf16_t)lo[1], r[2] = (bf16_t)lo[2], r[3] = (bf16_t)lo[3];
    r[4] = (bf16_t)hi[0], r[5] = (bf16_t)hi[1], r[6] = (bf16_t)hi[2], r[7] = (bf16_t)hi[3];
    return r;
}

typedef __attribute__((ext_vector_type(16))) float f32x16;

// v_mfma_f32_32x32x16_bf16:  A[i = l%32][k = 8 (l/32) + 0..7]   B[k = 8 (l/32) + 0..7][j = l%32]
//                            D[i = 8 (r/4) + 4 (l/32) + r%4][j = l%32],  r = 0..15 the register index
__device__ __forceinline__ f32x16 mfma32_bf16(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

}  // namespace gdn

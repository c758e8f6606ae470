// Chunked forward of the gated delta rule for gfx950 (bf16 MFMA, fp32 state), chunk C = 64: the host side.
//
// Replaces fla.ops.gated_delta_rule.chunk_gated_delta_rule as called at
// lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:197-209.
//
// Per chunk, with gamma = cumsum(g) inside the chunk, k^ / q^ the (optionally normalised) rows
// and S0 the state at chunk start:
//
//     A_ij = beta_i e^{gamma_i - gamma_j} (k^_i . k^_j)  (i > j)        T = (I + A)^-1
//     V~ = T diag(beta) (V - diag(e^gamma) K^ S0)
//     O  = diag(e^gamma scale) Q^ S0 + P V~,   P_ij = scale e^{gamma_i - gamma_j} (q^_i . k^_j)  (i >= j)
//     S_C = e^{gamma_C} S0 + K~^T V~,          K~_j = e^{gamma_C - gamma_j} k^_j
//
// Two steps, both in gdn_chunk32.hip (one launch each, or one launch for both: gdn_chunk_fused.hip):
//   prepare (parallel over every chunk and head): everything that does not depend on the state - K K^T, the
//       triangular inverse, P and the row scales - written to a workspace record per (head, chunk) as bf16 MFMA
//       operand fragments, in the register order the scan consumes them;
//   scan (serial over the chunks of a sequence, parallel over sequences, heads and column slices of V): a wave owns
//       a slice of the fp32 state as MFMA accumulators.
// This file: the workspace layout, the chunk offsets of packed batches, and the translation of the C arguments into
// the kernels' parameter block.

#include <type_traits>

#include "gdn_chunk_common.h"
#include "gdn_launch.h"

namespace gdn {

static int chunk_slots(const gdn_args& a) {
    const int nt = (a.T + C - 1) / C;
    const bool packed = a.cu_seqlens != nullptr && !(a.flags & GDN_FLAG_LEFT_PADDED);
    return packed ? a.T / C + a.N : a.B * nt;
}

// chunk offsets [N + 1] and the scan order of the sequences [N] (packed batches), then the error latch of the one-launch
// forward: the last 32-bit word of this region
static uint64_t chunk_off_bytes(const gdn_args& a) { return ((2 * (uint64_t)a.N + 2) * 4 + 255u) & ~(uint64_t)255u; }

bool chunk_shape_supported(const gdn_args& a) {
    if (a.dtype != GDN_BF16) return false;
    if (a.chunk != 0 && a.chunk != C) return false;
    if (a.K != 64 && a.K != 128 && a.K != 256) return false;
    if (a.V <= 0 || a.V % 32 != 0) return false;
    if (a.B <= 0 || a.T <= 0 || a.H <= 0 || a.N <= 0) return false;
    return true;
}

uint64_t chunk_record_bytes(const gdn_args& a) {
    return (uint64_t)a.H * chunk_slots(a) * record_layout(a.K, a.V).bytes;
}

// one int32 flag per record (used when prepare and scan run in one launch)
static uint64_t chunk_flag_bytes(const gdn_args& a) { return ((uint64_t)a.H * chunk_slots(a) * 4 + 255u) & ~(uint64_t)255u; }

uint64_t chunk_header_bytes(const gdn_args& a) { return chunk_off_bytes(a) + chunk_flag_bytes(a); }

uint64_t chunk_error_latch_offset(const gdn_args& a) { return chunk_off_bytes(a) - 4; }

uint64_t chunk_workspace_bytes(const gdn_args& a) {
    const RecordLayout r = record_layout(a.K, a.V);
    return chunk_off_bytes(a) + chunk_flag_bytes(a) + (uint64_t)a.H * chunk_slots(a) * r.bytes;
}

// ------------------------------------------------------------------------------------------
// chunk offsets of packed sequences: chunk_off[n] = sum_{m < n} ceil(len_m / C)
// ------------------------------------------------------------------------------------------
// Lengths are taken through packed_bounds, and the running total is capped at the number of record slots
// the workspace holds (`slots`): whatever cu_seqlens contains, no chunk gets a slot outside the workspace
// (sequences past the cap get none; a well-formed prefix never reaches it).
//
// order[r] = the sequence with the r-th most chunks (ties by index): the scan starts its chains in that order, so that the
// longest sequence of a ragged batch, which bounds the launch, is not the one that starts last.  Ranked by counting
// (N^2 / 256 comparisons per thread) for up to ORDER_MAX sequences; larger batches, whose many sequences even out by
// themselves, keep the order of the batch.
constexpr int ORDER_MAX = 1024;
__global__ __launch_bounds__(256) void chunk_offsets_kernel(const int32_t* __restrict__ cu, int32_t* __restrict__ off,
                                                            int32_t* __restrict__ order, int N, int total, int slots) {
    __shared__ int s_part[256];
    const int tid = threadIdx.x;
    const int per = (N + 255) / 256;
    const int begin = min(tid * per, N), end = min(begin + per, N);
    auto chunks_of = [&](int n) {
        int t0, len;
        packed_bounds(cu, n, total, t0, len);
        return (len + C - 1) / C;
    };
    int sum = 0;
    for (int n = begin; n < end; n++) sum = min(sum + chunks_of(n), slots);
    s_part[tid] = sum;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int i = 0; i < 256; i++) {
            const int x = s_part[i];
            s_part[i] = run;
            run = min(run + x, slots);
        }
        off[N] = run;
    }
    __syncthreads();
    int run = s_part[tid];
    for (int n = begin; n < end; n++) {
        off[n] = run;
        run = min(run + chunks_of(n), slots);
    }
    if (N > ORDER_MAX) {
        for (int n = tid; n < N; n += 256) order[n] = n;
        return;
    }
    __shared__ int s_cnt[ORDER_MAX];
    for (int n = tid; n < N; n += 256) s_cnt[n] = chunks_of(n);
    __syncthreads();
    for (int n = tid; n < N; n += 256) {
        const int mine = s_cnt[n];
        int rank = 0;
        for (int m = 0; m < N; m++) rank += (s_cnt[m] > mine || (s_cnt[m] == mine && m < n)) ? 1 : 0;
        order[rank] = n;  // the ranks are a permutation of 0 .. N - 1
    }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
int launch_chunk32(ChunkParams& p, int K, hipStream_t stream, hipEvent_t* events, int num_cus);  // gdn_chunk32.hip

bool chunk_saving_scan_is_staged(const gdn_args& a, const gdn_chunk_saves& saves) {
    if (!chunk_shape_supported(a)) return false;
    const bool packed = a.cu_seqlens != nullptr && !(a.flags & GDN_FLAG_LEFT_PADDED);
    SaveRequest req;
    req.no_output = saves.no_output != 0, req.has_state = saves.states != nullptr, req.has_vnew = saves.v_new != nullptr;
    req.state_bf16 = saves.states_dtype == GDN_BF16, req.vnew_bf16 = saves.v_new_dtype == GDN_BF16;
    req.save_every = saves.save_every > 0 ? saves.save_every : 1;
    return plan_scan(a.K, (int64_t)a.N * a.H, a.V, packed, true, saves.records_given, compute_units(), req).staged_saves;
}

bool chunk_runs_as_one_launch(const gdn_args& a) {
    if (!(a.flags & GDN_FLAG_FUSED_LAUNCH) || !chunk_shape_supported(a)) return false;
    if ((a.K != 64 && a.K != 128) || a.V % 64 != 0 || a.cu_seqlens != nullptr) return false;  // see chunk_fused_supported
    return fused_launch_window((int64_t)a.N * a.H, a.V, compute_units());
}

#ifdef GDN_CYCLE_BUDGET
// Measurement build only: a device buffer the sampled waves of the half-slice scan (and the sampled workgroups of the
// chunk-local backward kernel) report into (allocated on first use; this build is not the library proper and is free
// to), and its read-out.
uint64_t* cycle_buffer() {
    static uint64_t* buf = nullptr;
    if (buf == nullptr && hipMalloc(&buf, GDN_CYCLE_BUDGET_SLOTS * 8 * sizeof(uint64_t)) != hipSuccess) buf = nullptr;
    return buf;
}
int cycle_budget_read(uint64_t* host, int slots) {
    uint64_t* buf = cycle_buffer();
    if (buf == nullptr || slots > GDN_CYCLE_BUDGET_SLOTS) return GDN_ERR_WORKSPACE;
    if (hipError_t e = hipDeviceSynchronize(); e != hipSuccess) return (int)e;
    return (int)hipMemcpy(host, buf, (size_t)slots * 8 * sizeof(uint64_t), hipMemcpyDeviceToHost);
}
#endif

int launch_chunk_fwd(const gdn_args& a, hipStream_t stream, hipEvent_t* events, const gdn_chunk_saves* saves) {
    const RecordLayout r = record_layout(a.K, a.V);
    ChunkParams p;
    p.cycle_out = nullptr;
#ifdef GDN_CYCLE_BUDGET
    p.cycle_out = cycle_buffer();
    if (p.cycle_out != nullptr) (void)hipMemsetAsync(p.cycle_out, 0, GDN_CYCLE_BUDGET_SLOTS * 8 * sizeof(uint64_t), stream);
#endif
    p.q = static_cast<const bf16_t*>(a.q);
    p.k = static_cast<const bf16_t*>(a.k);
    p.v = static_cast<const bf16_t*>(a.v);
    p.beta = a.beta;
    p.g = a.g;
    p.h0 = a.h0;
    p.ht = a.ht;
    p.o = static_cast<bf16_t*>(a.o);
    const bool left_padded = (a.flags & GDN_FLAG_LEFT_PADDED) != 0;
    p.cu_seqlens = left_padded ? nullptr : a.cu_seqlens;
    p.pad_lens = left_padded ? a.cu_seqlens : nullptr;
    p.chunk_off = static_cast<int32_t*>(a.workspace);
    p.seq_order = p.chunk_off + a.N + 1;
    p.ready = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(a.workspace) + chunk_off_bytes(a));
    p.err = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(a.workspace) + chunk_error_latch_offset(a));
    p.err_caller = a.error_word;
    p.spin_limit = a.spin_limit > 0 ? (uint32_t)a.spin_limit : (1u << 22);
    p.no_producers = (a.flags & GDN_FLAG_DEBUG_NO_PRODUCERS) ? 1 : 0;
    p.rec = static_cast<uint8_t*>(a.workspace) + chunk_off_bytes(a) + chunk_flag_bytes(a);
    p.save_state = nullptr, p.save_vnew = nullptr, p.save_nc = 0, p.records_given = 0, p.save_every = 1, p.save_reverse = 0;
    p.save_state_bf16 = 0, p.save_vnew_bf16 = 0, p.no_output = 0;
    p.mirror = 0, p.k2 = nullptr, p.v2 = nullptr;
    p.row_order = saves != nullptr && saves->records_given && left_padded ? saves->row_order : nullptr;
    p.save_sliced = saves != nullptr && saves->sliced ? 1 : 0;
    p.k2_stride_b = p.k2_stride_t = p.k2_stride_h = p.v2_stride_b = p.v2_stride_t = p.v2_stride_h = 0;
    if (saves != nullptr && saves->mirror_reads) {
        p.mirror = 1, p.k2 = static_cast<const bf16_t*>(saves->k_odd), p.v2 = static_cast<const bf16_t*>(saves->v_odd);
        p.k2_stride_b = saves->k_odd_stride_b, p.k2_stride_t = saves->k_odd_stride_t, p.k2_stride_h = saves->k_odd_stride_h;
        p.v2_stride_b = saves->v_odd_stride_b, p.v2_stride_t = saves->v_odd_stride_t, p.v2_stride_h = saves->v_odd_stride_h;
    }
    if (saves != nullptr) {
        p.save_state = static_cast<float*>(saves->states), p.save_vnew = static_cast<float*>(saves->v_new), p.save_nc = saves->chunks_per_chain;
        p.save_state_bf16 = saves->states_dtype == GDN_BF16 ? 1 : 0, p.save_vnew_bf16 = saves->v_new_dtype == GDN_BF16 ? 1 : 0;
        p.no_output = saves->no_output ? 1 : 0;
        p.save_every = saves->save_every > 0 ? saves->save_every : 1, p.save_reverse = saves->save_reverse ? 1 : 0;
        p.records_given = saves->records_given;
        if (p.records_given) p.chunk_off = nullptr, p.seq_order = nullptr, p.ready = nullptr, p.err = nullptr, p.rec = static_cast<uint8_t*>(a.workspace);
    }
    p.q_stride_b = a.q_stride_b, p.q_stride_t = a.q_stride_t, p.q_stride_h = a.q_stride_h;
    p.k_stride_b = a.k_stride_b, p.k_stride_t = a.k_stride_t, p.k_stride_h = a.k_stride_h;
    p.v_stride_b = a.v_stride_b, p.v_stride_t = a.v_stride_t, p.v_stride_h = a.v_stride_h;
    p.o_stride_b = a.o_stride_b, p.o_stride_t = a.o_stride_t, p.o_stride_h = a.o_stride_h;
    p.B = a.B, p.T = a.T, p.H = a.H, p.V = a.V, p.N = a.N;
    p.qk_div = a.qk_heads > 0 ? a.H / a.qk_heads : 1;
    p.NT = (a.T + C - 1) / C;
    p.TC = chunk_slots(a);
    p.beta_dtype = a.beta_dtype;
    p.l2norm = (a.flags & GDN_FLAG_L2NORM) ? 1 : 0;
    p.scale = a.scale;
    p.rec_bytes = r.bytes, p.off_qs = r.off_qs, p.off_ks = r.off_ks, p.off_cs = r.off_cs, p.off_p = r.off_p;
    p.off_eg = r.off_eg;
    p.scan_groups = 1;
    p.fused = (a.flags & GDN_FLAG_FUSED_LAUNCH) ? 1 : 0;
    p.ready_clear = (a.flags & GDN_FLAG_READY_FLAGS_CLEAR) ? 1 : 0;

    auto mark = [&](int i) {
        if (events != nullptr) (void)hipEventRecord(events[i], stream);
    };
    mark(0);
    if (p.cu_seqlens != nullptr) {
        hipLaunchKernelGGL(chunk_offsets_kernel, dim3(1), dim3(256), 0, stream, p.cu_seqlens, p.chunk_off, p.seq_order, p.N, p.T, p.TC);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
    }
    mark(1);
    const int rc = launch_chunk32(p, a.K, stream, events, compute_units());
    mark(3);
    return rc;
}

}  // namespace gdn

// C ABI of libgdn_hip.so (declared in include/gdn_hip.h): argument validation and dispatch.
// Everything the host can see that could fault a kernel (shapes, strides, alignment, workspace size) is
// checked here before any launch.  The contents of cu_seqlens live on the device and are not: the kernels
// clamp them (packed_bounds, and the slot cap of chunk_offsets_kernel), so a malformed prefix gives wrong
// sequences but no access outside the caller's tensors or the workspace.

#include <hip/hip_runtime.h>

#include <mutex>

#include "gdn_hip.h"
#include "gdn_launch.h"

// Workspace of gdn_chunk_fwd_noalloc: device memory that belongs to the library's code object, so that the entry
// point has nothing to allocate.  Every device the library runs on holds its own copy, at its own address, until
// the process ends.  Host code never passes this name to a kernel (on the host it is a stand-in, not a device
// address): noalloc_scratch() below asks the runtime for the address once per device and hands that out.
static __device__ __align__(256) unsigned char scratch[GDN_NOALLOC_SCRATCH_BYTES];

#ifdef GDN_CYCLE_BUDGET
namespace gdn {
int cycle_budget_read(uint64_t* host, int slots);  // gdn_chunk.hip, measurement build only
}
#endif

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void* scratch_ptr[MAX_DEVICES] = {};

// Address of `scratch` on the calling thread's current device; looked up on the first call per device.
int noalloc_scratch(void** out) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return GDN_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        if (hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)); e != hipSuccess) return (int)e;
        if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
        scratch_ptr[dev] = ptr;
    }
    *out = scratch_ptr[dev];
    return GDN_OK;
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

int validate_common(const gdn_args* a) {
    if (a == nullptr) return GDN_ERR_NULL;
    if (!a->q || !a->k || !a->v || !a->o) return GDN_ERR_NULL;
    if (a->B <= 0 || a->T <= 0 || a->H <= 0 || a->K <= 0 || a->V <= 0 || a->N <= 0) return GDN_ERR_SHAPE;
    if (a->qk_heads < 0 || (a->qk_heads > 0 && a->H % a->qk_heads != 0)) return GDN_ERR_SHAPE;
    if (a->cu_seqlens != nullptr && !(a->flags & GDN_FLAG_LEFT_PADDED)) {
        if (a->B != 1) return GDN_ERR_VARLEN;
    } else if (a->N != a->B) {
        return GDN_ERR_SHAPE;
    }
    if ((a->flags & GDN_FLAG_LEFT_PADDED) && a->cu_seqlens == nullptr) return GDN_ERR_NULL;
    if (a->H > 65535 || a->N > 65535) return GDN_ERR_UNSUPPORTED;
    if (a->dtype != GDN_BF16 && a->dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->beta && a->beta_dtype != GDN_BF16 && a->beta_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->K != 64 && a->K != 128 && a->K != 256) return GDN_ERR_UNSUPPORTED;
    if (a->V % 32 != 0) return GDN_ERR_UNSUPPORTED;

    // rows are read and written with 16-byte accesses
    const int64_t elems16 = (a->dtype == GDN_BF16) ? 8 : 4;
    const int64_t strides[] = {a->q_stride_b, a->q_stride_t, a->q_stride_h, a->k_stride_b, a->k_stride_t,
                               a->k_stride_h, a->v_stride_b, a->v_stride_t, a->v_stride_h, a->o_stride_b,
                               a->o_stride_t, a->o_stride_h};
    for (int64_t s : strides)
        if (s < 0 || s % elems16 != 0) return GDN_ERR_ALIGN;
    if (a->q_stride_h < a->K || a->k_stride_h < a->K || a->v_stride_h < a->V || a->o_stride_h < a->V)
        return GDN_ERR_SHAPE;
    // the kernels address the 64 rows of a chunk with 32-bit byte offsets from the chunk's first row
    const int64_t token_strides[] = {a->q_stride_t, a->k_stride_t, a->v_stride_t, a->o_stride_t};
    for (int64_t s : token_strides)
        if (s > ((int64_t)1 << 24)) return GDN_ERR_UNSUPPORTED;
    if (!aligned(a->q, 16) || !aligned(a->k, 16) || !aligned(a->v, 16) || !aligned(a->o, 16)) return GDN_ERR_ALIGN;
    if ((a->h0 && !aligned(a->h0, 16)) || (a->ht && !aligned(a->ht, 16))) return GDN_ERR_ALIGN;
    if (a->g && !aligned(a->g, 4)) return GDN_ERR_ALIGN;
    if (a->cu_seqlens && !aligned(a->cu_seqlens, 4)) return GDN_ERR_ALIGN;
    if (a->h0 && a->ht && a->h0 == a->ht && !(a->flags & GDN_FLAG_STATE_INPLACE)) return GDN_ERR_SHAPE;
    return GDN_OK;
}

}  // namespace

extern "C" {

int gdn_abi_version(void) { return GDN_ABI_VERSION; }

const char* gdn_strerror(int status) {
    switch (status) {
        case GDN_OK: return "success";
        case GDN_ERR_NULL: return "a required pointer is NULL";
        case GDN_ERR_SHAPE: return "inconsistent or non-positive shape";
        case GDN_ERR_UNSUPPORTED:
            return "unsupported configuration (need K in {64,128,256}, V % 32 == 0, bf16/fp32; chunked forward: "
                   "bf16, chunk 64)";
        case GDN_ERR_ALIGN: return "pointer or stride not 16-byte aligned";
        case GDN_ERR_WORKSPACE:
            return "workspace missing or too small (gdn_chunk_fwd_noalloc: the shape needs more than its built-in scratch)";
        case GDN_ERR_VARLEN: return "cu_seqlens requires B == 1 (packed) or GDN_FLAG_LEFT_PADDED";
        case GDN_ERR_TIMEOUT:
            return "the one-launch chunked forward gave up waiting for a record of its prepare half; the outputs of that call are invalid";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown gdn status";
}

uint64_t gdn_workspace_bytes(const gdn_args* a) {
    if (a == nullptr || !gdn::chunk_shape_supported(*a)) return 0;
    return gdn::chunk_workspace_bytes(*a);
}

uint64_t gdn_workspace_header_bytes(const gdn_args* a) {
    if (a == nullptr || !gdn::chunk_shape_supported(*a)) return 0;
    return gdn::chunk_header_bytes(*a);
}

int gdn_chunk_fwd_is_one_launch(const gdn_args* a) { return a != nullptr && gdn::chunk_runs_as_one_launch(*a) ? 1 : 0; }

int gdn_recurrent_fwd(const gdn_args* a, void* stream) {
    const int rc = validate_common(a);
    if (rc != GDN_OK) return rc;
    return gdn::launch_recurrent(*a, static_cast<hipStream_t>(stream));
}

static int validate_chunk(const gdn_args* a) {
    const int rc = validate_common(a);
    if (rc != GDN_OK) return rc;
    if (!gdn::chunk_shape_supported(*a)) return GDN_ERR_UNSUPPORTED;
    const uint64_t need = gdn::chunk_workspace_bytes(*a);
    if (a->workspace == nullptr || a->workspace_bytes < need || !aligned(a->workspace, 256)) return GDN_ERR_WORKSPACE;
    return GDN_OK;
}

int gdn_chunk_fwd(const gdn_args* a, void* stream) {
    const int rc = validate_chunk(a);
    if (rc != GDN_OK) return rc;
    return gdn::launch_chunk_fwd(*a, static_cast<hipStream_t>(stream));
}

int gdn_chunk_fwd_status(const gdn_args* a, void* stream) {
    const int rc = validate_chunk(a);
    if (rc != GDN_OK) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (hipError_t e = hipStreamSynchronize(s); e != hipSuccess) return (int)e;
    int32_t latch = 0;
    uint8_t* ws = static_cast<uint8_t*>(a->workspace);
    if (hipError_t e = hipMemcpy(&latch, ws + gdn::chunk_error_latch_offset(*a), sizeof(latch), hipMemcpyDeviceToHost); e != hipSuccess) return (int)e;
    if (latch == 0) return GDN_OK;
    // every kernel of the failed call has ended: nobody sets a flag any more
    if (hipError_t e = hipMemsetAsync(ws, 0, gdn::chunk_header_bytes(*a), s); e != hipSuccess) return (int)e;
    if (hipError_t e = hipStreamSynchronize(s); e != hipSuccess) return (int)e;
    return GDN_ERR_TIMEOUT;
}

int gdn_chunk_fwd_noalloc(const gdn_args* a, void* stream) {
    int rc = validate_common(a);
    if (rc != GDN_OK) return rc;
    if (!gdn::chunk_shape_supported(*a)) return GDN_ERR_UNSUPPORTED;
    if (gdn::chunk_workspace_bytes(*a) > (uint64_t)GDN_NOALLOC_SCRATCH_BYTES) return GDN_ERR_WORKSPACE;
    void* ptr = nullptr;
    rc = noalloc_scratch(&ptr);
    if (rc != GDN_OK) return rc;
    // Nothing in the workspace has to start at zero: the offsets kernel and prepare write every word the
    // scan reads.  The same array serves every call on this device.
    gdn_args b = *a;
    b.flags &= ~GDN_FLAG_READY_FLAGS_CLEAR;  // where the flags lie in the array depends on the shape: records of another call may have been there
    b.workspace = ptr;
    b.workspace_bytes = (uint64_t)GDN_NOALLOC_SCRATCH_BYTES;
    return gdn::launch_chunk_fwd(b, static_cast<hipStream_t>(stream));
}

int gdn_chunk_fwd_saving(const gdn_args* a, const gdn_chunk_saves* saves, void* stream) {
    if (saves == nullptr) return GDN_ERR_NULL;
    const int rc = validate_common(a);
    if (rc != GDN_OK) return rc;
    if (!gdn::chunk_shape_supported(*a)) return GDN_ERR_UNSUPPORTED;
    if (saves->states == nullptr && saves->v_new == nullptr) return GDN_ERR_NULL;
    if ((saves->states && !aligned(saves->states, 16)) || (saves->v_new && !aligned(saves->v_new, 16))) return GDN_ERR_ALIGN;
    if (saves->chunks_per_chain <= 0) return GDN_ERR_SHAPE;  // chunks beyond it are computed but not saved
    uint64_t need = gdn::chunk_workspace_bytes(*a);
    if (saves->records_given < 0 || saves->records_given > 2) return GDN_ERR_SHAPE;
    if (saves->records_given == 1 && a->K > 128) return GDN_ERR_UNSUPPORTED;  // K = 256 scans on half-slice waves only
    if (saves->records_given) {
        // records are given for batches of rows: fixed-length, or left-padded with whole chunks per row
        if (a->cu_seqlens != nullptr && (!(a->flags & GDN_FLAG_LEFT_PADDED) || saves->mirror_reads)) return GDN_ERR_VARLEN;
        if (saves->row_order != nullptr && !aligned(saves->row_order, 4)) return GDN_ERR_ALIGN;
        need = gdn::chunk_record_bytes(*a);
    }
    if (a->workspace == nullptr || a->workspace_bytes < need || !aligned(a->workspace, 256)) return GDN_ERR_WORKSPACE;
    if ((saves->states_dtype != GDN_F32 && saves->states_dtype != GDN_BF16) || (saves->v_new_dtype != GDN_F32 && saves->v_new_dtype != GDN_BF16))
        return GDN_ERR_UNSUPPORTED;
    if ((saves->states_dtype == GDN_BF16 || saves->v_new_dtype == GDN_BF16) && !gdn::chunk_saving_scan_is_staged(*a, *saves))
        return GDN_ERR_UNSUPPORTED;
    if (saves->sliced) {  // bf16 saves through the staging variant only
        if ((saves->states && saves->states_dtype != GDN_BF16) || (saves->v_new && saves->v_new_dtype != GDN_BF16)) return GDN_ERR_UNSUPPORTED;
        if (!gdn::chunk_saving_scan_is_staged(*a, *saves)) return GDN_ERR_UNSUPPORTED;
    }
    if (saves->mirror_reads) {
        // only the scan without output reads that way
        if (!saves->records_given || !saves->no_output || a->K < 128 || !gdn::chunk_saving_scan_is_staged(*a, *saves)) return GDN_ERR_UNSUPPORTED;
        if (saves->k_odd == nullptr || saves->v_odd == nullptr) return GDN_ERR_NULL;
        if (!aligned(saves->k_odd, 16) || !aligned(saves->v_odd, 16)) return GDN_ERR_ALIGN;
        if (a->T % 128 != 0) return GDN_ERR_SHAPE;
        const int64_t odd_strides[] = {saves->k_odd_stride_b, saves->k_odd_stride_t, saves->k_odd_stride_h,
                                       saves->v_odd_stride_b, saves->v_odd_stride_t, saves->v_odd_stride_h};
        for (int64_t s : odd_strides)
            if (s < 0 || s % 8 != 0) return GDN_ERR_ALIGN;
        if (saves->k_odd_stride_t > (1 << 24) || saves->v_odd_stride_t > (1 << 24)) return GDN_ERR_UNSUPPORTED;
    }
    return gdn::launch_chunk_fwd(*a, static_cast<hipStream_t>(stream), nullptr, saves);
}

int gdn_chunk_fwd_saving_is_staged(const gdn_args* a, const gdn_chunk_saves* saves) {
    return a != nullptr && saves != nullptr && gdn::chunk_saving_scan_is_staged(*a, *saves) ? 1 : 0;
}

int gdn_chunk_bwd_local(const gdn_chunk_local_args* a, void* stream) {
    if (a == nullptr) return GDN_ERR_NULL;
    const void* needed[] = {a->v_new, a->states, a->dstates, a->gamma, a->beta, a->y_mirror != nullptr ? a->y_mirror : a->y_chunks,
                            a->dq_out, a->dk_out, a->dv_out, a->dg_out, a->dbeta_out, a->q_raw, a->k_raw, a->v_raw, a->dout_raw};
    for (const void* x : needed)
        if (x == nullptr) return GDN_ERR_NULL;
        else if (!aligned(x, 16)) return GDN_ERR_ALIGN;
    if (a->saves_dtype != GDN_BF16 && a->saves_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->dstates_dtype != GDN_BF16 && a->dstates_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->saves_sliced && (a->saves_dtype != GDN_BF16 || a->dstates_dtype != GDN_BF16 || a->y_chunks == nullptr)) return GDN_ERR_UNSUPPORTED;
    if (a->H <= 0 || a->NC <= 0 || a->chunks % ((int64_t)a->H * a->NC) != 0) return GDN_ERR_SHAPE;
    if (a->seq_start != nullptr && (a->seq_len == nullptr || a->T_rows <= 0)) return GDN_ERR_SHAPE;
    const int64_t raw_strides[] = {a->q_stride_b, a->q_stride_t, a->q_stride_h, a->k_stride_b, a->k_stride_t, a->k_stride_h,
                                   a->v_stride_b, a->v_stride_t, a->v_stride_h, a->dout_stride_b, a->dout_stride_t, a->dout_stride_h};
    for (int64_t st : raw_strides)
        if (st < 0 || st % 8 != 0) return GDN_ERR_ALIGN;
    if ((a->rq == nullptr) != (a->rk == nullptr)) return GDN_ERR_NULL;
    if (a->rq != nullptr && (!aligned(a->rq, 4) || !aligned(a->rk, 4))) return GDN_ERR_ALIGN;
    if (!(a->scale > 0.f)) return GDN_ERR_SHAPE;
    if (a->chunks <= 0 || a->chunks > 0x7fffffff) return GDN_ERR_SHAPE;
    if (!gdn::chunk_bwd_local_supported(*a)) return GDN_ERR_UNSUPPORTED;
    return gdn::launch_chunk_bwd_local(*a, static_cast<hipStream_t>(stream));
}

int gdn_chunk_bwd_prepare(const gdn_chunk_bwd_prepare_args* a, void* stream) {
    if (a == nullptr) return GDN_ERR_NULL;
    const void* ptrs[] = {a->q, a->k, a->dout, a->gamma, a->beta_packed, a->rq, a->rk, a->v_mirror, a->records};
    for (const void* x : ptrs) {
        if (x == nullptr) return GDN_ERR_NULL;
        if (!aligned(x, 16)) return GDN_ERR_ALIGN;
    }
    if (a->k_mirror == nullptr && a->seq_start != nullptr) return GDN_ERR_VARLEN;  // no reversed copies: whole-chunk batches only
    if (a->k_mirror != nullptr && !aligned(a->k_mirror, 16)) return GDN_ERR_ALIGN;
    if (a->N <= 0 || a->T <= 0 || a->H <= 0 || a->N > 65535 || a->H > 65535) return GDN_ERR_SHAPE;
    if (!gdn::chunk_bwd_prepare_supported(*a)) return GDN_ERR_UNSUPPORTED;
    if (a->beta && a->beta_dtype != GDN_BF16 && a->beta_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (!(a->scale > 0.f)) return GDN_ERR_SHAPE;
    const int64_t strides[] = {a->q_stride_b, a->q_stride_t, a->q_stride_h, a->k_stride_b, a->k_stride_t, a->k_stride_h,
                               a->dout_stride_b, a->dout_stride_t, a->dout_stride_h};
    for (int64_t s : strides)
        if (s < 0 || s % 8 != 0) return GDN_ERR_ALIGN;
    if ((int64_t)a->N * a->H * (a->seq_start != nullptr ? a->NC : a->T / 64) > 0x7fffffff) return GDN_ERR_UNSUPPORTED;
    if (!aligned(a->records, 256) || a->records_bytes < gdn::chunk_bwd_record_bytes(*a)) return GDN_ERR_WORKSPACE;
    if (a->records_fwd != nullptr) {
        if (a->seq_start != nullptr) return GDN_ERR_VARLEN;  // the forward's records are laid out for whole-chunk batches
        if (!aligned(a->records_fwd, 256) || a->records_fwd_bytes < gdn::chunk_bwd_record_bytes(*a) / 2) return GDN_ERR_WORKSPACE;
    }
    return gdn::launch_chunk_bwd_prepare(*a, static_cast<hipStream_t>(stream));
}

int gdn_causal_conv1d_bwd(const gdn_conv_bwd_args* a, void* stream) {
    if (a == nullptr) return GDN_ERR_NULL;
    if (!a->x || !a->dy || !a->weight || !a->dx || !a->dweight_partial || !a->dbias_partial) return GDN_ERR_NULL;
    if (a->B <= 0 || a->S <= 0 || a->C <= 0) return GDN_ERR_SHAPE;
    if (a->dtype != GDN_BF16 && a->dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    const int vec = 2;  // channels per thread
    if (a->C % vec != 0 || a->kernel_size < 2 || a->kernel_size > 4) return GDN_ERR_UNSUPPORTED;
    if (a->w_dtype != GDN_BF16 && a->w_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->activation != GDN_ACT_NONE && a->activation != GDN_ACT_SILU) return GDN_ERR_UNSUPPORTED;
    if (!aligned(a->x, 8) || !aligned(a->dy, 8) || !aligned(a->dx, 8)) return GDN_ERR_ALIGN;
    const int64_t strides[] = {a->x_stride_b, a->x_stride_s, a->dy_stride_b, a->dy_stride_s};
    for (int64_t s : strides)
        if (s < 0 || s % vec != 0) return GDN_ERR_ALIGN;
    if (a->tokens_per_block < 8 || a->tokens_per_block > 4096) return GDN_ERR_SHAPE;
    if ((int64_t)a->B * ((a->S + a->tokens_per_block - 1) / a->tokens_per_block) > 65535) return GDN_ERR_UNSUPPORTED;  // one grid row per block
    return gdn::launch_conv_bwd(*a, static_cast<hipStream_t>(stream));
}

#ifdef GDN_CYCLE_BUDGET
// Measurement build only (not declared in gdn_hip.h, not part of libgdn_hip.so): after a chunked forward that ran the
// half-slice scan, the cycles wave 0 of every 16th scan workgroup spent in each group of its chunk loop, summed over its
// chunks: out[slot * 8 + 0..5] = K S0 | S0^T q^T | T' X | k^T V~ | V~^T P^T | between chunks, out[slot * 8 + 6] = chunks.
// After a gdn_chunk_bwd_local call the same buffer holds that kernel's report instead (read it with slots = 64): 32 sampled
// workgroups, out[w * 16 + 0..14] = the cycles of the kernel's steps (bench.py's LOCAL_GROUPS), out[w * 16 + 15] = slabs per chunk.
int gdn_cycle_budget_read(uint64_t* out, int slots) { return gdn::cycle_budget_read(out, slots); }
#endif

int gdn_chunk_fwd_profile(const gdn_args* a, void* stream, float* kernel_ms) {
    if (kernel_ms == nullptr) return GDN_ERR_NULL;
    int rc = validate_chunk(a);
    if (rc != GDN_OK) return rc;
    hipEvent_t events[GDN_CHUNK_KERNELS + 1];
    int created = 0;
    for (; created <= GDN_CHUNK_KERNELS; created++)
        if (hipError_t e = hipEventCreate(&events[created]); e != hipSuccess) {
            rc = (int)e;
            break;
        }
    if (rc == GDN_OK) rc = gdn::launch_chunk_fwd(*a, static_cast<hipStream_t>(stream), events);
    if (rc == GDN_OK) rc = (int)hipEventSynchronize(events[GDN_CHUNK_KERNELS]);
    for (int i = 0; rc == GDN_OK && i < GDN_CHUNK_KERNELS; i++) {
        kernel_ms[i] = 0.f;
        if (i == 0 && (a->cu_seqlens == nullptr || (a->flags & GDN_FLAG_LEFT_PADDED))) continue;
        rc = (int)hipEventElapsedTime(&kernel_ms[i], events[i], events[i + 1]);
    }
    for (int i = 0; i < created; i++) (void)hipEventDestroy(events[i]);
    return rc;
}

}  // extern "C"

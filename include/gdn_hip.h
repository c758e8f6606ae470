/*
 * gdn_hip.h — C ABI of libgdn_hip.so: the gated delta-rule sequence mixer for gfx950.
 *
 * The reference reaches this path through a Python import seam, not an FFI:
 *   from fla.ops.gated_delta_rule import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule
 *   (lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:24-25)
 * and calls both with keywords q, k, v, g, beta, scale, initial_state, output_final_state,
 * cu_seqlens, use_qk_l2norm_in_kernel (module.py:197-222).  The entry points below are what a
 * binding for those two functions needs; every pointer is a DEVICE pointer owned by the
 * caller.  The library holds no state, never allocates, frees or synchronises (the measurement
 * aid gdn_chunk_fwd_profile excepted), and launches asynchronously on the stream it is given
 * (current device of the calling thread).
 *
 * Return value of every int-returning entry point: 0 on success, a negative gdn_status on
 * rejected arguments, a positive hipError_t if a launch failed.
 */
#ifndef GDN_HIP_H
#define GDN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GDN_ABI_VERSION 2

typedef enum gdn_dtype { GDN_BF16 = 0, GDN_F32 = 1 } gdn_dtype;

typedef enum gdn_status {
    GDN_OK = 0,
    GDN_ERR_NULL = -1,        /* a required pointer is NULL */
    GDN_ERR_SHAPE = -2,       /* B, T, H, K, V, N inconsistent or non-positive */
    GDN_ERR_UNSUPPORTED = -3, /* head dims / dtype / chunk size this build has no kernel for */
    GDN_ERR_ALIGN = -4,       /* pointer or stride not aligned as the kernels require */
    GDN_ERR_WORKSPACE = -5,   /* workspace missing or smaller than gdn_workspace_bytes() */
    GDN_ERR_VARLEN = -6,      /* cu_seqlens given with B != 1 */
    GDN_ERR_TIMEOUT = -7      /* gdn_chunk_fwd_status: the one-launch forward gave up waiting for a record; outputs invalid */
} gdn_status;

enum {
    GDN_FLAG_L2NORM = 1,        /* normalise q and k rows in-kernel: x / sqrt(sum x^2 + 1e-6) */
    GDN_FLAG_STATE_INPLACE = 2, /* decode: ht == h0 is allowed and expected */
    GDN_FLAG_LEFT_PADDED = 4,   /* cu_seqlens describes a left-padded batch, see gdn_args */
    GDN_FLAG_FUSED_LAUNCH = 8,  /* gdn_chunk_fwd: run prepare and scan as one launch when the shape allows it (fixed-length
                                   batch, K <= 128, V a multiple of 64, N * H * V / 64 between 3/8 and 1/2 of the CUs: where
                                   it is the faster way; other shapes run as without the flag); results stay within the
                                   same parity gates but are not bit-identical to the two-kernel path */
    GDN_FLAG_READY_FLAGS_CLEAR = 16, /* gdn_chunk_fwd: the caller keeps this workspace between calls and every byte of it was
                                   zero before its first use.  The one-launch forward keeps one ready flag per record
                                   in the workspace; it clears them itself before it starts (a small kernel of its own)
                                   unless this flag promises that they are clear.  Every call that returns success
                                   leaves them clear again, with or without the flag, so a workspace that is used for
                                   nothing else, by calls of one shape on one stream, keeps the promise by itself. */
    GDN_FLAG_RECORDS_16X16 = 32, /* gdn_chunk_bwd_prepare: write the operand fragments of the mirror problem's records in
                                   the lane order of the 16x16x32 MFMA, for gdn_chunk_fwd_saving with records_given = 2 */
    GDN_FLAG_SKIP_EMPTY_CHUNKS = 128, /* gdn_chunk_bwd_prepare with seq_start / seq_len: chunk slots past the end of their
                                       * sequence (other than a sequence's first slot) get no records and no rows of the
                                       * mirror problem - for a mirror scan that walks every row over its own length
                                       * (gdn_chunk_fwd_saving with records_given on a left-padded batch) */
    GDN_FLAG_DEBUG_NO_PRODUCERS = 64, /* test aid for the one-launch forward: its prepare workgroups return at once, so that
                                   the scan's bounded wait runs out (with a small args->spin_limit) and the error path can be
                                   exercised while every kernel still ends normally; outputs are invalid */
};

/*
 * One call = one forward of the operator over all sequences and heads.
 *
 *   q, k   [B, T, H, K]   element strides q_stride_{b,t,h}, last dim contiguous
 *   v, o   [B, T, H, V]   element strides v_/o_stride_{b,t,h}, last dim contiguous
 *   g      [B, T, H] fp32 contiguous, log-decay (<= 0), or NULL for the ungated rule
 *   beta   [B, T, H] contiguous in beta_dtype, or NULL for beta == 1
 *   h0     [N, H, K, V] fp32 contiguous or NULL (zero state)
 *   ht     [N, H, K, V] fp32 contiguous or NULL (final state not written)
 *   cu_seqlens  int32 [N + 1] with a leading 0 (packed sequences, then B must be 1), or NULL
 *               (then N must equal B).  With GDN_FLAG_LEFT_PADDED the batch stays [B, T, ...], N must
 *               equal B, and cu_seqlens holds the prefix sums of the valid lengths: sequence b is the
 *               last cu_seqlens[b+1] - cu_seqlens[b] tokens of row b (what the reference gets from
 *               compute_cu_seqlens_and_max_seqlen_from_attention_mask, sequence_packing.py:18-22, and
 *               then packs and unpacks around the operator, :25-93); o is written at valid tokens only.
 *
 * Replaces the argument list of both fla calls at gated_deltanet/module.py:198-222.
 */
typedef struct gdn_args {
    const void *q;
    const void *k;
    const void *v;
    const void *beta;
    const float *g;
    const float *h0;
    float *ht;
    void *o;
    const int32_t *cu_seqlens;
    void *workspace;
    uint64_t workspace_bytes;

    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    int64_t o_stride_b, o_stride_t, o_stride_h;

    int32_t B, T, H, K, V, N;
    int32_t chunk;      /* chunk length of the chunked forward; this build supports 64 (0 = default) */
    int32_t dtype;      /* gdn_dtype of q, k, v, o */
    int32_t beta_dtype; /* gdn_dtype of beta */
    int32_t flags;      /* GDN_FLAG_* */
    float scale;        /* multiplies q (after optional normalisation) */
    int32_t spin_limit; /* one-launch forward: polls of a record's ready flag before the scan gives up (0 = default, 2^22:
                           seconds); see gdn_chunk_fwd_status */
    int32_t qk_heads;   /* heads of q and k when fewer than H (grouped value attention, gated_deltanet/module.py:175-177:
                           value head h reads q and k of head h / (H / qk_heads), what repeat_interleave would copy
                           there); must divide H.  0 = H */
    int32_t reserved;
    int32_t *error_word; /* optional, may be NULL: an int32 the GPU can write (device memory, or pinned host memory, which a
                           caller can read without synchronising); the one-launch forward stores 1 there when it gives up
                           waiting.  Never cleared by the library. */
} gdn_args;

/* Version of this header the library was built from; a binding checks it equals GDN_ABI_VERSION. */
int gdn_abi_version(void);

/* Human-readable text for a value returned by the functions below (gdn_status or hipError_t). */
const char *gdn_strerror(int status);

/*
 * Bytes of device scratch gdn_chunk_fwd needs for these shapes (only the shape fields of
 * `args` are read).  The caller allocates it and passes it in args->workspace.  Returns 0
 * for unsupported shapes (gdn_chunk_fwd then reports why).
 */
uint64_t gdn_workspace_bytes(const gdn_args *args);

/*
 * The leading bytes of the workspace that GDN_FLAG_READY_FLAGS_CLEAR promises to be zero (chunk offsets, the
 * error latch and the ready flags); the records behind them need no initialisation.  0 for unsupported shapes.
 */
uint64_t gdn_workspace_header_bytes(const gdn_args *args);

/*
 * Chunked forward over full sequences (bf16 q/k/v/o, fp32 state, chunk 64):
 * replaces fla.ops.gated_delta_rule.chunk_gated_delta_rule as called at
 * gated_deltanet/module.py:197-209.  `stream` is a hipStream_t.
 */
int gdn_chunk_fwd(const gdn_args *args, void *stream);

/*
 * 1 when gdn_chunk_fwd would run these arguments as one launch (prepare and scan together) on the calling thread's
 * current device, else 0.  Reads the shape fields, dtype, flags and whether cu_seqlens is NULL; no pointer is followed.
 */
int gdn_chunk_fwd_is_one_launch(const gdn_args *args);

/*
 * Error report of the one-launch forward (GDN_FLAG_FUSED_LAUNCH; no counterpart in the reference, whose Triton
 * kernels are separate launches).  Its scan workgroups wait, with a bounded number of polls, for records that
 * prepare workgroups of the same launch write.  A scan workgroup whose wait runs out latches an error word in
 * the workspace header (and stores 1 to args->error_word when that is set), stops writing its outputs and runs
 * to its end, so the launch always terminates; o and ht of that call are then invalid.  This function waits
 * for `stream`, reads the latch of args->workspace (same shape fields as the gdn_chunk_fwd call) and returns
 * GDN_OK or GDN_ERR_TIMEOUT; in the latter case it also zeroes the workspace header (latch and ready flags,
 * which such a launch leaves in no defined state), so the workspace can be used again with
 * GDN_FLAG_READY_FLAGS_CLEAR.  It blocks the calling thread.
 */
int gdn_chunk_fwd_status(const gdn_args *args, void *stream);

/*
 * gdn_chunk_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  args->workspace and
 * args->workspace_bytes are ignored: the chunk records go to a scratch array that is part of the library's
 * device code (GDN_NOALLOC_SCRATCH_BYTES per device the library runs on, held until the process ends), and the
 * call makes no hipMalloc, hipFree or other allocating call.  Shapes with gdn_workspace_bytes(args) above that
 * size are rejected with GDN_ERR_WORKSPACE.  Results are bit-identical to gdn_chunk_fwd's.  Every call on a
 * device shares that device's array: calls that overlap on one device (different streams or threads) race;
 * calls on one stream are ordered and safe.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress), which may load the code object: make that call outside any capture.
 */
#define GDN_NOALLOC_SCRATCH_BYTES (64u << 20)
int gdn_chunk_fwd_noalloc(const gdn_args *args, void *stream);

/*
 * Token-by-token recurrence with the state tile held in registers; T may be any length and
 * q/k/v may be bf16 or fp32.  With T == 1 this is the decode step: one read and one write
 * of the fp32 state, in place when GDN_FLAG_STATE_INPLACE is set and ht == h0.
 * Replaces fla.ops.gated_delta_rule.fused_recurrent_gated_delta_rule as called at
 * gated_deltanet/module.py:210-222.  `stream` is a hipStream_t.
 */
int gdn_recurrent_fwd(const gdn_args *args, void *stream);

/*
 * Training support.  The reference differentiates through chunk_gated_delta_rule (chunk mode is asserted
 * while training, gated_deltanet/module.py:194-209); a backward pass needs the state every chunk starts
 * from and the chunk's V~ (the values written into the state), which gdn_chunk_fwd does not keep.
 * gdn_chunk_fwd_saving is gdn_chunk_fwd with a scan that also writes them, fp32:
 *     states [N * H][chunks_per_chain][K][V]     chain n * H + h, chunk c of its sequence
 *     v_new  [N * H][chunks_per_chain][64][V]    rows past the end of a sequence are not meaningful
 * Either may be NULL.  Only chunks c with c % save_every == 0 are saved (save_every <= 0 means 1), as entry
 * e = c / save_every, or as entry chunks_per_chain - 1 - e when save_reverse != 0; entries outside
 * [0, chunks_per_chain) are computed but not saved.
 * With records_given != 0 the prepare kernel is skipped: args->workspace then holds the chunk records
 * themselves, [H][B * ceil(T / 64)] records in the layout prepare writes (fixed-length batches only;
 * g, beta and the l2norm flag are not used, the records carry every scale).  records_given = 1: the twelve
 * operand fragments of a record are in the lane order of the 32x32x16 MFMA (K <= 128 only; the scan runs
 * whole-slice waves, 1 or 4 slices per workgroup).  records_given = 2: they are in the lane order of the
 * 16x16x32 MFMA (any K, required for K = 256); the scan then runs one slice per workgroup on two half-slice
 * waves, which is the faster kernel as long as N * H * V / 32 does not exceed the number of compute units.
 * The backward pass of this package runs its reverse sweep over the chunks that way.
 * states_dtype, v_new_dtype: GDN_F32, or GDN_BF16 (the pointer is then a bf16 array of the same shape).  bf16 saves
 * need the variant of the scan that stages its saves through LDS, which gdn_chunk_fwd_saving_is_staged reports for
 * the same arguments and saves (one column slice per workgroup, and K <= 128; or K = 256 with no_output, bf16 or no
 * v_new, and states that are bf16 or asked for with save_every >= 2); GDN_ERR_UNSUPPORTED otherwise.
 * no_output != 0: the caller does not need args->o (a sweep that is run for its saves); where a variant of the scan
 * without the products that only serve the output exists (staged saves, K >= 128) it runs and args->o, which must
 * still be a valid buffer, is left unwritten; elsewhere the flag changes nothing.
 * mirror_reads != 0 (records_given and no_output set, the scan without output: staged saves, K >= 128; else
 * GDN_ERR_UNSUPPORTED): the sequence of T tokens that the scan walks is a sequence of T / 2 tokens read backwards with
 * every chunk taken twice - the reverse sweep of the backward pass over gdn_chunk_bwd_prepare's mirror problem without
 * its reversed copies.  Row i of chunk 2 r is token 64 (T/128 - 1 - r) + 63 - i of args->k and args->v, row i of chunk
 * 2 r + 1 that token of k_odd and v_odd; all four are [N, T / 2, H, .] bf16 with element strides (args' for k and v).
 * sliced != 0 (bf16 saves through the staging variant only; GDN_ERR_UNSUPPORTED otherwise): states and v_new are laid
 * out by 32-column slice, [N * H][chunks_per_chain][V / 32][K or 64][32]: what one scan workgroup saves of a chunk is
 * then one contiguous block (whole 128-byte lines from one CU instead of 64-byte halves of lines from several), which
 * gdn_chunk_bwd_local reads with saves_sliced.
 * records_given with a left-padded batch (GDN_FLAG_LEFT_PADDED, args->cu_seqlens the prefix sums of the rows' valid lengths,
 * which must be multiples of 64; not with mirror_reads): row n is scanned over its last tokens only, its records lie at
 * the slots of those tokens (the last ones of the row), and with save_reverse the row's last saved chunk goes to entry 0
 * of ITS entries whatever the row's length.  row_order (then only; NULL = as they lie): the rows in the order in which
 * their chains are dealt out to the XCDs and started, best longest first - a ragged batch takes as long as the XCD with
 * the most chunks.
 * mirror_reads: T / 64 must be even.  The twelve operand fragments of every odd chunk are read from the record of chunk 1 of the chain
 * (in the mirror problem they are the same for all odd chunks: T' = I, P = 0); an odd chunk's own record supplies its
 * row scales and e^{gamma_C} only.
 */
typedef struct gdn_chunk_saves {
    void *states;
    void *v_new;
    int32_t chunks_per_chain;
    int32_t records_given;
    int32_t save_every;
    int32_t save_reverse;
    int32_t states_dtype; /* gdn_dtype of states */
    int32_t v_new_dtype;  /* gdn_dtype of v_new */
    int32_t no_output;
    int32_t mirror_reads;
    int32_t sliced;
    int32_t reserved;
    const void *k_odd, *v_odd;
    int64_t k_odd_stride_b, k_odd_stride_t, k_odd_stride_h;
    int64_t v_odd_stride_b, v_odd_stride_t, v_odd_stride_h;
    const int32_t *row_order; /* [N] or NULL */
} gdn_chunk_saves;
int gdn_chunk_fwd_saving(const gdn_args *args, const gdn_chunk_saves *saves, void *stream);
/* 1 when gdn_chunk_fwd_saving would run these arguments (shape fields, flags, cu_seqlens NULL or not; every field of
 * saves, its two pointers only as NULL or not) on the scan that stages its saves through LDS, on the calling thread's
 * current device; else 0. */
int gdn_chunk_fwd_saving_is_staged(const gdn_args *args, const gdn_chunk_saves *saves);

/*
 * Training support, second part: the chunk-local gradients, one workgroup per (sequence, head, chunk), once
 * the two sweeps over the chunks (gdn_chunk_fwd_saving, forward and mirrored) have delivered per chunk the
 * state it starts from, the gradient of the state it ends with, V~ and Y = T^T dV~.  Chunk index
 * = (n * H + h) * NC + c; per-chunk arrays are contiguous and chunk-major:
 *     v_new         [chunks][64][V]   V~, in saves_dtype (what gdn_chunk_fwd_saving wrote)
 *     states        [chunks][K][V]    the state a chunk starts from, in saves_dtype
 *     dstates       [chunks][K][V]    the gradient of the state it ends with, in dstates_dtype (fp32 or bf16)
 *     gamma, beta   [chunks][64]      prefix sum of g inside the chunk, beta (fp32; from gdn_chunk_bwd_prepare)
 *     rq, rk        [chunks][64]      1 / sqrt(|q|^2 + 1e-6), likewise for k, when q and k were normalised
 *                                     (the l2norm flag of the forward); both NULL otherwise
 *     y_mirror      bf16 [N, 2 * NC * 64, H, V]: the output of the scan over the mirror problem of
 *                   gdn_chunk_bwd_prepare (Y at its even chunks, tokens reversed); or NULL and
 *     y_chunks      bf16 [chunks][64][V]: the V~ that scan saved at its even chunks (save_every = 2, save_reverse,
 *                   bf16 saves, no output): Y of chunk (n, h, c) with its tokens in reverse order
 *     q_raw, k_raw, v_raw, dout_raw   the caller's bf16 q, k, v, dO, [N, NC * 64, H, D] with element strides
 * Outputs, in the caller's layout, contiguous: dq_out, dk_out [N, NC * 64, H, K] and dv_out [N, NC * 64, H, V]
 * (bf16; the gradients with respect to q and k themselves, through the scale and the normalisation), dg_out and
 * dbeta_out fp32 [N, NC * 64, H] (dg_out is the gradient with respect to g: the reverse prefix sum of the gradient
 * with respect to gamma inside the chunk).
 * K = 64, 128 or 256 and V a multiple of 64 (GDN_ERR_UNSUPPORTED otherwise).  Counterpart upstream: the chunk-local
 * kernels of fla's backward of chunk_gated_delta_rule, reached from gated_deltanet/module.py:197-209 under autograd.
 */
typedef struct gdn_chunk_local_args {
    const void *v_new, *states, *dstates;
    const float *gamma, *beta, *rq, *rk;
    int32_t saves_dtype; /* gdn_dtype of v_new and states */
    float scale;
    int64_t chunks;
    int32_t K, V;
    const void *y_mirror, *y_chunks;
    void *dq_out, *dk_out, *dv_out;
    float *dg_out, *dbeta_out;
    int32_t H, NC;
    const void *q_raw, *k_raw, *v_raw, *dout_raw;
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    int64_t dout_stride_b, dout_stride_t, dout_stride_h;
    /* packed or left-padded batches: sequence n starts at token seq_start[n] (a flat index over the
     * rows of the caller's tensors, T_rows tokens per row) and has seq_len[n] tokens; its chunks c * 64 >= seq_len[n]
     * are skipped, tokens past its end are not written.  NULL: sequence n is row n, NC * 64 tokens. */
    const int32_t *seq_start, *seq_len;
    int32_t T_rows;
    int32_t dstates_dtype; /* gdn_dtype of dstates */
    int32_t saves_sliced;  /* v_new, states, dstates and y_chunks are laid out by 32-column slice, [chunks][V / 32][rows][32]
                              (gdn_chunk_saves.sliced); all of them bf16 then */
    int32_t reserved;
} gdn_chunk_local_args;
int gdn_chunk_bwd_local(const gdn_chunk_local_args *args, void *stream);

/*
 * Training support, third part: everything the backward needs per chunk before its two sweeps (batches of
 * whole chunks: T a multiple of 64, one sequence per row; other batches through seq_start / seq_len below;
 * bf16 q, k, dout as [N, T, H, D] with element
 * strides; K = 64, 128 or 256 and V a multiple of 64, GDN_ERR_UNSUPPORTED otherwise).  One workgroup per (sequence, head, chunk) writes
 *   - gamma, beta_packed, rq, rk: fp32 [N H T/64][64], operands of gdn_chunk_bwd_local;
 *   - the reverse sweep as a forward scan over 2 T tokens per sequence ("mirror" problem: tokens in reverse
 *     order, chunk c becomes chunks 2 r and 2 r + 1, r = T/64 - 1 - c): k_mirror [N, 2 T, H, K] and
 *     v_mirror [N, 2 T, H, V] (bf16, contiguous) and the chunk records [H][N * 2 T/64], records_bytes >=
 *     H * N * 2 T/64 * 13312, for gdn_chunk_fwd_saving with records_given (k_mirror also in the place of q).
 *     With k_mirror == NULL (batches of whole chunks only) no reversed copies are written: v_mirror is then
 *     [N, T, H, V] and receives P^T dO, the rows of v of the even chunks, in the caller's token order, for a scan with
 *     gdn_chunk_saves.mirror_reads (k = the caller's k, v = this array, k_odd = the caller's q, v_odd = dout); of the
 *     odd chunks' records only chunk 1 of every chain then carries its operand fragments, the others their scales.
 *     The scan's output at the even chunks is Y = T^T dV~ (reversed), the states it saves there are the
 *     gradients of the chunks' final states, its final state is the gradient of the initial state.
 * flags: GDN_FLAG_L2NORM, GDN_FLAG_RECORDS_16X16, GDN_FLAG_SKIP_EMPTY_CHUNKS.  g (fp32 [N, T, H]) and beta ([N, T, H], beta_dtype) may be NULL (0 and 1).
 */
typedef struct gdn_chunk_bwd_prepare_args {
    const void *q, *k, *dout;
    const float *g;
    const void *beta;
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t dout_stride_b, dout_stride_t, dout_stride_h;
    int32_t N, T, H, K, V;
    int32_t beta_dtype;
    int32_t flags;
    float scale;
    float *gamma, *beta_packed, *rq, *rk;
    void *k_mirror, *v_mirror, *records;
    uint64_t records_bytes;
    /* packed or left-padded batches: as in gdn_chunk_local_args, with T the tokens per row of q, k, dout (N need not
     * be their number of rows) and NC the chunks per sequence of the packed arrays and of the mirror problem
     * (>= ceil(max seq_len / 64)); T / 64 is read as NC when seq_start is NULL */
    const int32_t *seq_start, *seq_len;
    int32_t NC;
    int32_t reserved;
    /* optional (whole-chunk batches only: seq_start NULL): the records of the forward pass itself, [H][N * T/64] as
     * gdn_chunk_fwd's prepare step writes them (fragment order as chosen by GDN_FLAG_RECORDS_16X16), for a forward
     * sweep through gdn_chunk_fwd_saving with records_given (q, k, v are then the caller's own tensors);
     * records_fwd_bytes >= H * N * T/64 * 13312 */
    void *records_fwd;
    uint64_t records_fwd_bytes;
} gdn_chunk_bwd_prepare_args;
int gdn_chunk_bwd_prepare(const gdn_chunk_bwd_prepare_args *args, void *stream);

/*
 * Measurement aid, no counterpart in the reference: runs exactly what gdn_chunk_fwd runs, with a
 * HIP event recorded on `stream` before and after every kernel, waits for the last one and
 * returns each kernel's duration in milliseconds in kernel_ms[GDN_CHUNK_KERNELS], in launch
 * order: [0] chunk offsets of packed sequences (0 when cu_seqlens is NULL), [1] prepare, [2] scan.
 * Unlike every other entry point it creates events and blocks the calling thread.
 */
#define GDN_CHUNK_KERNELS 3
int gdn_chunk_fwd_profile(const gdn_args *args, void *stream, float *kernel_ms);

/*
 * Depthwise causal convolution over the token axis, the step right before the operator in the layer
 * (q, k, v are slices of its output): replaces DepthwiseCausalConvolution.forward,
 * lm_engine/modeling_utils/depthwise_causal_convolution.py:103-241, in all three of its modes
 * (fresh prefill :157-197, one-token update :199-231, multi-token continuation :232-246), i.e. the
 * causal_conv1d_fn / causal_conv1d_update calls and their torch restatements there.
 *
 *   y[b, s, c] = act(bias[c] + sum_j weight[c, j] * xx[b, s - (kernel_size - 1) + j, c]) * mask[b, s]
 *   xx = input_state (positions -(kernel_size-1) .. -1, zeros when NULL) followed by x * mask
 *   final_state[b, c, :] = the last kernel_size - 1 positions of xx        (:53-64)
 *
 *   x, y          [B, S, C]  element strides *_stride_b, *_stride_s, channels contiguous; y must not overlap x
 *   weight        [C, kernel_size] contiguous in w_dtype (nn.Conv1d's [C, 1, kernel_size])
 *   bias          [C] in w_dtype, or NULL
 *   input_state   [B, C, kernel_size - 1] contiguous in dtype, or NULL
 *   mask          [B, S] contiguous in dtype, or NULL  (the reference's 0/1 padding mask, :28-37)
 *   final_state   [B, C, kernel_size - 1] contiguous in dtype, or NULL (not written)
 *
 * kernel_size 2..4, C a multiple of 8 (bf16) or 4 (fp32), rows, weight and bias 16-byte aligned;
 * w_dtype equals dtype or is fp32.
 */
typedef enum gdn_activation { GDN_ACT_NONE = 0, GDN_ACT_SILU = 1 } gdn_activation;

typedef struct gdn_conv_args {
    const void *x;
    const void *weight;
    const void *bias;
    const void *input_state;
    const void *mask;
    void *y;
    void *final_state;
    int64_t x_stride_b, x_stride_s;
    int64_t y_stride_b, y_stride_s;
    int32_t B, S, C, kernel_size;
    int32_t dtype;      /* gdn_dtype of x, y, input_state, final_state, mask */
    int32_t w_dtype;    /* gdn_dtype of weight and bias */
    int32_t activation; /* gdn_activation */
    int32_t reserved;
} gdn_conv_args;

int gdn_causal_conv1d_fwd(const gdn_conv_args *args, void *stream);

/*
 * Backward of gdn_causal_conv1d_fwd (what autograd computes through
 * DepthwiseCausalConvolution.forward, depthwise_causal_convolution.py:103-241, when the layer trains):
 * given dy [B, S, C] (element strides) it recomputes the pre-activation from x and writes dx [B, S, C]
 * (contiguous), dstate [B, C, kernel_size - 1] (NULL when there was no input_state), both in dtype, and, per
 * block of tokens_per_block (8 .. 4096) tokens of a row, the partial sums of the gradients of weight and bias:
 * dweight_partial [B * ceil(S / tokens_per_block)][C][kernel_size] and dbias_partial [same][C], fp32, which
 * the caller adds up over the first dim.  C even; x, dy, dx 8-byte aligned, strides even.  The gradient flowing
 * into final_state is the caller's to add (it lands on the last kernel_size - 1 rows of dx or on dstate).
 */
typedef struct gdn_conv_bwd_args {
    const void *x, *dy, *weight, *bias, *input_state, *mask;
    void *dx, *dstate;
    float *dweight_partial, *dbias_partial;
    int64_t x_stride_b, x_stride_s;
    int64_t dy_stride_b, dy_stride_s;
    int32_t B, S, C, kernel_size;
    int32_t w_dtype;    /* gdn_dtype of weight and bias */
    int32_t activation; /* gdn_activation */
    int32_t tokens_per_block;
    int32_t dtype;      /* gdn_dtype of x, dy, input_state, mask, dx, dstate (bf16 or fp32) */
} gdn_conv_bwd_args;
int gdn_causal_conv1d_bwd(const gdn_conv_bwd_args *args, void *stream);

/*
 * The operator's scalar inputs from the layer's projections, one pass:
 *   g    = -exp(A_log[h]) * softplus(a + dt_bias[h])     fp32   SoftplusDecayGate.forward with
 *          final_exponential=False, lm_engine/modeling_utils/softplus_decay_gate/module.py:69-96
 *   beta = beta_scale * sigmoid(b)                       dtype  gated_deltanet/module.py:179-181
 *          (beta_scale 2 when allow_neg_eigval, else 1)
 * a, b: [tokens, H] with element strides a_stride / b_stride between tokens (slices of one projection);
 * A_log, dt_bias: [H] fp32; g: [tokens, H] fp32 contiguous; beta: [tokens, H] contiguous in dtype.
 */
typedef struct gdn_gate_args {
    const void *a;
    const void *b;
    const float *A_log;
    const float *dt_bias;
    float *g;
    void *beta;
    int64_t a_stride, b_stride;
    int64_t tokens;
    int32_t H;
    int32_t dtype; /* gdn_dtype of a, b, beta */
    float beta_scale;
    int32_t reserved;
} gdn_gate_args;

int gdn_gates_fwd(const gdn_gate_args *args, void *stream);

/*
 * Backward of gdn_gates_fwd (autograd through SoftplusDecayGate.forward, softplus_decay_gate/module.py:69-96, and
 * `beta = b.sigmoid()`, gated_deltanet/module.py:179-181, when the layer trains): given dg (fp32) and dbeta (dtype),
 * both [tokens, H] contiguous, it writes da and db ([tokens, H] contiguous, dtype) and the partial sums of the
 * gradients of A_log and dt_bias left by each of its `partial_blocks` workgroups (1 .. 65535; a few per compute
 * unit), dA_log_partial and ddt_bias_partial, fp32 [partial_blocks][H], which the caller adds up over the first dim.
 */
typedef struct gdn_gate_bwd_args {
    const void *a, *b;
    const float *A_log, *dt_bias;
    const float *dg;
    const void *dbeta;
    void *da, *db;
    float *dA_log_partial, *ddt_bias_partial;
    int64_t a_stride, b_stride;
    int64_t tokens;
    int32_t H;
    int32_t dtype; /* gdn_dtype of a, b, dbeta, da, db */
    float beta_scale;
    int32_t partial_blocks;
} gdn_gate_bwd_args;
int gdn_gates_bwd(const gdn_gate_bwd_args *args, void *stream);

/*
 * What the layer does to the operator's output before the output projection, one pass:
 *   y = rmsnorm(o * silu(gate)) * weight   over the V columns of every (token, head)
 * gated_deltanet/module.py:238-242 (`o = o * silu(g)`, `o = self.o_norm(o)`), RMSNorm of
 * lm_engine/modeling_utils/normalization.py:69-124: x / sqrt(mean(x^2) + eps) * weight.
 * o, y: [tokens, H, V] with element strides *_stride_t between tokens; gate: same shape with
 * gate_stride_t (a slice of a projection), or NULL (no gating); weight: [V] in w_dtype or NULL.
 * V a multiple of 8, at most 512; 16-byte aligned rows.
 */
typedef struct gdn_norm_args {
    const void *o;
    const void *gate;
    const void *weight;
    void *y;
    int64_t o_stride_t, gate_stride_t, y_stride_t;
    int64_t tokens;
    int32_t H, V;
    int32_t dtype;   /* gdn_dtype of o, gate, y */
    int32_t w_dtype; /* gdn_dtype of weight */
    float eps;
    int32_t reserved;
} gdn_norm_args;

int gdn_gated_rmsnorm_fwd(const gdn_norm_args *args, void *stream);

/*
 * Backward of gdn_gated_rmsnorm_fwd (autograd through `o = o * silu(g)`, `o = self.o_norm(o)`,
 * module.py:238-242, when the layer trains): given dy [tokens, H, V] (contiguous) it writes d_o and, with a
 * gate, d_gate (both [tokens, H, V] contiguous, dtype of o), and the partial sums of the gradient of weight
 * left by each of its `partial_blocks` workgroups, dweight_partial [partial_blocks][V] fp32, which the
 * caller adds up (also when weight is NULL).
 */
typedef struct gdn_norm_bwd_args {
    const void *o, *gate, *weight, *dy;
    void *d_o, *d_gate;
    float *dweight_partial;
    int64_t o_stride_t, gate_stride_t;
    int64_t tokens;
    int32_t H, V;
    int32_t dtype, w_dtype;
    float eps;
    int32_t partial_blocks;
} gdn_norm_bwd_args;
int gdn_gated_rmsnorm_bwd(const gdn_norm_bwd_args *args, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GDN_HIP_H */

// Chunked forward of the gated delta rule (K = 64, 128, 256): the kernels.  Whole-slice waves work on
// v_mfma_f32_32x32x16_bf16 (K <= 128), half-slice waves on v_mfma_f32_16x16x32_bf16 (K <= 128 when a slice has a
// CU to itself, and K = 256 always).
//
// Two kernels (prepare: what does not depend on the state, written as MFMA operand fragments to a workspace
// record per (head, chunk); scan: the serial pass over the chunks of a sequence with the state held in MFMA
// accumulators; gdn_chunk.hip holds the host side), with the WY form's T pulled out:
//     V~ = U - W S0 = T diag(beta) (V - diag(cs) K S0),      cs = e^{gamma} / |k|
// so the record holds T diag(beta) and P only, prepare never touches V, and the scan works from the
// caller's q, k and v.  Further:
//
//   * a wave of the scan owns a K x 32 slice of the state; operand fragments are laid out for
//     the 32x32x16 shape;
//   * the scan stages everything a chunk needs in an LDS double buffer filled by dedicated loader waves,
//     hands its output to a dedicated store wave, and keeps its compute waves free of memory instructions;
//   * prepare is persistent: a workgroup walks over (chunk, head) items and loads q, k of
//     the next item into registers while it computes the current one;
//   * the triangular inverse runs its block products on bf16 MFMA with operands split into
//     hi + lo halves (error ~2^-16, far below the final bf16 rounding of T), and transposed
//     operands come from ds_read_tr16_b64 instead of 2-byte gathers.
//
// 32x32x16 layouts (wave64, l = lane, h = l / 32):
//   A[i = l%32][k = 8 h + 0..7]    B[k = 8 h + 0..7][j = l%32]
//   D[i = 8 (r/4) + 4 h + r%4][j = l%32]   for accumulator register r = 0..15
//
// Reduction order: a D tile reused as B (or A) operand gives, for the 16-row slab s of the tile
// (s = 0, 1), registers 8 s .. 8 s + 7, i.e. MFMA rows 16 s + 4 h + 0..3 and 16 s + 8 + 4 h + 0..3.
// The state keeps its rows (key dim) and its columns in the order slice_col (bits 2 and 3 of the
// index within a 32-block swapped): MFMA row i of a state tile is key column slice_col(i), so the 8
// entries a lane half contributes per slab are the 8 consecutive key columns 16 s + 8 h + 0..7.
// So the scan uses q and k straight from their row-major rows.  (The token index, where it is the
// reduction index - of T' X, K^T V~ and P V~ - keeps the MFMA order; the T' and P fragments and the scan's
// transposing LDS reads of k are built to match.)
//
// Record:
//   T' = T diag(beta)   6 fragments      A fragments of V~ = T' X, rows = tokens: (token tile 0; X slabs 0, 1),
//                                        (token tile 1; X slabs 0..3); the zero quarter above the diagonal is not stored
//   P                   6 fragments      B fragments of O^T += V~^T P^T: (query tile 0; key slabs 0, 1),
//                                        (query tile 1; key slabs 0..3); P[i < 32][j >= 32] = 0 is not stored
//   64 fp32 row scales of q (e^{gamma} scale / |q|), 64 of k for the state update (e^{gamma_C - gamma} / |k|),
//   64 of k for K S0 (e^{gamma} / |k|), e^{gamma_C}

#include <type_traits>

#include "gdn_chunk32_common.h"
#include "gdn_chunk_prepare32.h"
#include "gdn_launch.h"

namespace gdn {

// ------------------------------------------------------------------------------------------
// prepare as a kernel of its own: persistent workgroups of four waves, three per CU
// ------------------------------------------------------------------------------------------
template <int K>
__global__ __launch_bounds__(PREP_THREADS, (K > 128 ? 1 : 3)) void chunk_prepare32_kernel(const ChunkParams p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[prepare32_lds_bytes<K>()];
    // Work items: (chunk slot, head), the slots rounded up to a multiple of 8.  Workgroup i runs on XCD i % 8 and
    // takes items i, i + grid, ... with the grid a multiple of 8, so w % 8 names the XCD.  That digit goes into
    // the slot number and the heads rotate with the rest: every XCD works on all heads.  The rows of one head
    // lie a whole token row (a multiple of 2 KiB) apart, so they fall on few channels of an XCD's L2; an XCD
    // that only ever sees one or two heads would send all its q, k, v traffic there.
    const uint32_t items = (uint32_t)((p.TC + 7) / 8) * 8u * (uint32_t)p.H;  // the launcher rejects more than 2^31
    if (blockIdx.x >= items) return;
    const uint32_t H = (uint32_t)p.H;
    auto item_of = [H](uint32_t w, int& h, int& slot) {
        const uint32_t j = w / 8u, jh = j / H;
        h = (int)(j - jh * H);
        slot = (int)(jh * 8u + w % 8u);
    };
    const uint32_t rounds = (items - blockIdx.x + gridDim.x - 1) / gridDim.x;
    chunk_prepare32_body<K, 1, false>(p, lds, item_of, items, blockIdx.x, gridDim.x, rounds, nullptr, 0);
}

// ------------------------------------------------------------------------------------------
// scan
//
// A workgroup works on one (sequence, head) chain and NW of its 32-column slices: NW compute
// waves, each owning a K x 32 slice of the fp32 state as MFMA accumulators, 4 loader waves and
// (NW < 4) one output wave.
//
// Per chunk, with S0 the state at its start (gamma, beta, T = (I + A)^-1 and P as in prepare):
//     X   = V - diag(cs) K S0            cs = e^{gamma} / |k|
//     V~  = T diag(beta) X               (the WY form U - W S0 with T pulled out: the record needs no W, no U)
//     O   = diag(qs) Q S0 + P V~         qs = e^{gamma} scale / |q|
//     S   = e^{gamma_C} S0 + K^T diag(ks) V~      ks = e^{gamma_C - gamma} / |k|
// Everything a chunk needs - the 12 operand fragments T diag(beta) | P of its record, the chunk's rows of q and k
// and this workgroup's columns of v straight from the caller's tensors, three vectors of row scales and
// e^{gamma_C} - goes through a double buffer in LDS: during chunk c the loaders move the data of chunk c + 1
// global -> registers -> LDS and already have chunks c + 2 and c + 3 in flight in a second register buffer.
// One workgroup barrier per chunk hands the halves over.  The memory instructions are kept out of the compute
// waves on purpose: a wave that issues a load or a store while the CU's vector-memory queue is full stalls
// until there is room, and with one compute wave per SIMD that stall is a stall of the matrix pipe.
//
// A compute wave runs the 60 MFMAs of a chunk (K = 128) as one unrolled schedule, reading each fragment from
// LDS a few MFMAs before its use; all other per-chunk work is cut into pieces placed between MFMAs that do not
// depend on them (ScanSchedule).  O is accumulated transposed (operands swapped) and the slice's columns are
// held in slice_col order, so a lane ends up with 8 consecutive columns of one token (16 bytes).
//
// The slices of a chain sit in workgroups on one XCD and read the same lines at the same time, so those come
// out of HBM once per chain.  What bounds the kernel when every CU has a workgroup is the rate at which a CU
// gets lines that were not in its L2 yet when asked for (~15 - 20 B/clk per CU, whatever the number of waves
// asking).
// ------------------------------------------------------------------------------------------
constexpr int SCAN_LOADERS = 4;

// Waves of a scan workgroup.  The hardware deals the waves of a workgroup round over the four SIMDs (wave w runs on
// SIMD w % 4), and a wave that shares a SIMD with a compute wave takes instruction-issue slots from it (measured:
// the loader on the compute wave's SIMD ran twice as long as the other three, and the compute wave waited for it).
// So with fewer than four compute waves the waves that land on their SIMDs get the light jobs:
//   NW = 1:  0 compute | 1 2 3 loaders | 4 output store | 5 loader
//   NW = 2:  0 1 compute | 2 3 loaders | 4 output store | 5 exits at once | 6 7 loaders
//   NW = 4:  0..3 compute | 4..7 loaders (each compute wave shares with one loader; no output wave)
//   NW = 1, HALF:  0 1 compute (16 columns each) | the rest as for NW = 2
__host__ __device__ constexpr int scan_waves(int nw, bool half = false) { return nw == 1 && !half ? 6 : 8; }

// Order of the MFMAs of one chunk in the scan's compute wave, and where its side work goes.
//
// MFMAs ("ops"):  K S0 (NSF) | O^T = S0^T q^T (NQF) | V~ = T' X (6) | S += k^T V~' (NKF) | O^T += V~^T P^T (6).
// The fourth group runs token slabs 0, 1 of every key tile before slabs 2, 3, so that the second token tile of V~,
// finished last, is needed late.
//
// Everything else (X = V - diag(cs) K S0 and its bf16 copy, decay of the state, bf16 repacking of V~ and of the new
// state, the row scales, hand-over of the output) is cut into pieces of four to twelve vector instructions.  A piece
// has a window: the first op at which its inputs exist (an MFMA result is taken two ops after the MFMA was issued)
// and the op that needs its result.  A lone wave issues an instruction every four to five cycles and an MFMA
// occupies the matrix pipe for 33, so more than about six instructions between two MFMAs idle the pipe: the pieces
// are spread one per op, earliest deadline first, as far as their windows allow.
template <int K>
struct ScanScheduleRules {
    static constexpr int KD = K / 32, KS16 = K / 16;
    static constexpr int NSF = 2 * KS16, NQF = 2 * KS16, NTF = 6, NKF = 4 * KD, NPF = 6;
    static constexpr int NOPS = NSF + NQF + NTF + NKF + NPF;
    static constexpr int LA = 6;
    static constexpr int OP_Q = NSF, OP_T = OP_Q + NQF, OP_K = OP_T + NTF, OP_P = OP_K + NKF, OP_BAR = NOPS - LA;
    static constexpr int AHEAD = 2;  // scales and rows of v are read this many ops before their piece
    static_assert(OP_BAR >= OP_P, "the scales and v of this chunk are used before the barrier");

    // op j of the fourth group -> key tile, token slab
    static constexpr int k_tile(int j) { return (j % (2 * KD)) / 2; }
    static constexpr int k_slab(int j) { return 2 * (j / (2 * KD)) + j % 2; }
    // op j of the third group -> token tile of V~, slab of X (fragment j of the record)
    static constexpr int t_tile(int j) { return j < 2 ? 0 : 1; }
    static constexpr int t_slab(int j) { return j < 2 ? j : j - 2; }

    // pieces: X (4 registers) | output hand-over (half a tile) | q row scale (4 registers) | decay (4 registers) |
    // scaled V~ (half a fragment) | plain V~ (a fragment) | new state (a fragment) | X as operand (a fragment)
    static constexpr int N_XC = 8, N_OUT = 4, N_AS = 8, N_DEC = 4 * KD, N_VS = 8, N_VB = 4, N_SB = 2 * KD, N_XB = 4;
    static constexpr int P_XC = 0, P_OUT = P_XC + N_XC, P_AS = P_OUT + N_OUT, P_DEC = P_AS + N_AS, P_VS = P_DEC + N_DEC,
                         P_VB = P_VS + N_VS, P_SB = P_VB + N_VB, P_XB = P_SB + N_SB, NPIECES = P_XB + N_XB;

    struct Window {
        int first, end;  // the piece runs before the MFMA of an op in [first, end)
    };
    static constexpr Window window(int pc) {
        if (pc < P_OUT) {  // K S0 of tile tt is complete after op KS16 (tt + 1) - 1; T' X overwrites tile 1 at its third op
            const int tt = (pc - P_XC) / 4;
            return {KS16 * (tt + 1) + 1, OP_T + 2 * tt};
        }
        if (pc < P_AS) return {1, OP_Q + KS16 * ((pc - P_OUT) / 2)};  // the previous chunk's tile, before q overwrites it
        if (pc < P_DEC) {
            const int tt = (pc - P_AS) / 4;
            const int end = OP_P + 2 * tt;
            return {OP_Q + KS16 * (tt + 1) + 1, end < OP_BAR ? end : OP_BAR};
        }
        if (pc < P_VS) return {0, OP_K + 2 * ((pc - P_DEC) / 4)};
        if (pc < P_VB) {  // V~ tile 0 is complete after the second op of T' X, tile 1 after the sixth
            const int x = (pc - P_VS) / 2;
            return {OP_T + (x / 2 == 0 ? 2 : 6) + 1, x < 2 ? OP_K + x : OP_K + NKF / 2 + (x - 2)};
        }
        if (pc < P_SB) return {OP_T + ((pc - P_VB) / 2 == 0 ? 2 : 6) + 1, OP_P};
        if (pc < P_XB) return {OP_K + NKF / 2 + 2 * ((pc - P_SB) / 2) + 3, NOPS};
        const int tt = (pc - P_XB) / 2;  // after the two X pieces of its half tile (checked in make)
        return {KS16 * (tt + 1) + 2, OP_T + 2 * tt};
    }

    struct Table {
        int op[NPIECES];
        bool ok;
    };
    static constexpr Table make() {
        Table t{};
        bool done[NPIECES] = {};
        int left = NPIECES;
        t.ok = true;
        for (int op = 0; op < NOPS; op++) {
            const int quota = (left + (NOPS - op) - 1) / (NOPS - op);
            for (int n = 0;; n++) {
                int best = -1;
                for (int pc = 0; pc < NPIECES; pc++)
                    if (!done[pc] && window(pc).first <= op && (best < 0 || window(pc).end < window(best).end)) best = pc;
                if (best < 0) break;
                if (n >= quota && window(best).end > op + 1) break;
                if (window(best).end <= op) t.ok = false;  // window missed
                t.op[best] = op, done[best] = true, left--;
            }
        }
        if (left != 0) t.ok = false;
        // a half tile of X is packed after its two pieces (within an op the pieces run in index order: X before the pack)
        for (int i = 0; i < N_XB; i++)
            if (t.op[P_XB + i] < t.op[P_XC + 2 * i] || t.op[P_XB + i] < t.op[P_XC + 2 * i + 1]) t.ok = false;
        // a ring register (rings of four) is refilled only after the piece four places earlier has used it
        for (int i = 4; i < N_VS; i++)
            if (t.op[P_VS + i] - AHEAD <= t.op[P_VS + i - 4]) t.ok = false;
        for (int i = 4; i < N_XC; i++)
            if (t.op[P_XC + i] - AHEAD <= t.op[P_XC + i - 4]) t.ok = false;
        for (int i = 0; i < N_VS; i++)
            if (t.op[P_VS + i] - AHEAD < 0) t.ok = false;
        return t;
    }
};

template <int K>
struct ScanSchedule : ScanScheduleRules<K> {
    static constexpr typename ScanScheduleRules<K>::Table TABLE = ScanScheduleRules<K>::make();
    static_assert(TABLE.ok, "no placement of the side work satisfies the windows");
    static constexpr int op_of(int pc) { return TABLE.op[pc]; }
};

// Schedule of the half-slice scan (HALF, see the kernel): the same five groups on v_mfma_f32_16x16x32_bf16, whose
// tiles are 16 tokens or 16 keys by this wave's 16 columns: K S0 (K/32 slabs x 4 token tiles) | O^T (as many) |
// V~ = T' X (6) | S += k^T V~' (2 token slabs x K/16 key tiles) | O^T += V~^T P^T (6).  Within a group consecutive
// MFMAs go to different accumulators (the instruction has 4 passes: a dependent one right behind it would wait).
// The pieces are half as large as in the whole-slice schedule; placement is the same earliest-deadline walk.  With
// MFMAs this short an op can be over in 16 cycles, so results are taken DIST ops after their MFMA and LDS data
// LA ops (operand fragments) or AHEAD ops (scales, rows of v) after the read was issued.
// NOOUT: a scan that only carries the state and V~ (the sweeps of the backward pass): the two groups that form the output
// and the pieces that serve them are left out.
template <int K, bool NOOUT = false>
struct Scan16Rules {
    static constexpr int KS = K / 32, KT = K / 16;
    static constexpr int NSF = 4 * KS, NQF = NOOUT ? 0 : 4 * KS, NTF = 6, NKF = 2 * KT, NPF = NOOUT ? 0 : 6;
    static constexpr int NOPS = NSF + NQF + NTF + NKF + NPF;
    static constexpr int LA = 10;
    static constexpr int OP_Q = NSF, OP_T = OP_Q + NQF, OP_K = OP_T + NTF, OP_P = OP_K + NKF, OP_BAR = NOPS - LA;
    static constexpr int AHEAD = 4, DIST = 3;

    // op j of the first two groups -> token tile, key slab: tiles 0 and 1 alternate through all slabs, then tiles 2 and 3
    // (X of the first two tiles can then be formed while the products of the other two run)
    static constexpr int s_tile(int j) { return 2 * (j / (2 * KS)) + j % 2; }
    static constexpr int s_slab(int j) { return (j % (2 * KS)) / 2; }
    static constexpr int s_last(int tt) { return (tt / 2) * 2 * KS + 2 * (KS - 1) + tt % 2; }  // last op of tile tt
    static constexpr int s_begin(int tt) { return (tt / 2) * 2 * KS + tt % 2; }                // and its first
    // op j of the third and fifth group -> token tile (16 tokens), slab of 32 reduction tokens: the non-zero blocks of a
    // lower triangular 64 x 64 matrix, (0,0) (1,0) (2,0) (3,0) (2,1) (3,1); fragment (tile, slab) is number
    // t_frag(j) of the record, where they are stored tile by tile
    static constexpr int t_tile(int j) { return j < 4 ? j : j - 2; }
    static constexpr int t_slab(int j) { return j < 4 ? 0 : 1; }
    static constexpr int t_frag(int j) { return j < 2 ? j : j == 2 ? 2 : j == 3 ? 4 : j == 4 ? 3 : 5; }
    static constexpr int t_first(int tt) { return tt; }                   // first op of tile tt ...
    static constexpr int t_last(int tt) { return tt < 2 ? tt : tt + 2; }  // ... and its last
    static constexpr int s_first(int s) { return s == 0 ? 0 : 4; }        // first op that reads slab s
    static constexpr int k_tile(int j) { return j % KT; }
    static constexpr int k_slab(int j) { return j / KT; }

    // pieces: X of a token tile | X of a slab as operand | previous output tile to LDS | q row scale of a tile |
    // decay of a state tile | scaled V~ of a token tile (half an operand) | plain V~ of a slab | new state slab
    static constexpr int N_XC = 4, N_XB = 2, N_OUT = NOOUT ? 0 : 4, N_AS = NOOUT ? 0 : 4, N_DEC = KT, N_VS = 4, N_VB = NOOUT ? 0 : 2, N_SB = KS;
    static constexpr int P_XC = 0, P_XB = P_XC + N_XC, P_OUT = P_XB + N_XB, P_AS = P_OUT + N_OUT, P_DEC = P_AS + N_AS,
                         P_VS = P_DEC + N_DEC, P_VB = P_VS + N_VS, P_SB = P_VB + N_VB, NPIECES = P_SB + N_SB;
    struct Window {
        int first, end;
    };
    static constexpr int before_barrier(int op) { return op < OP_BAR ? op : OP_BAR; }
    static constexpr Window window(int pc) {
        if (pc < P_XB) {
            const int tt = pc - P_XC;
            return {s_last(tt) + DIST, OP_T + s_first(tt / 2)};
        }
        if (pc < P_OUT) {
            const int s = pc - P_XB;
            return {s_last(2 * s + 1) + DIST, OP_T + s_first(s)};
        }
        if (pc < P_AS) return {DIST - 1, OP_Q + s_begin(pc - P_OUT)};  // (the last MFMA of the previous chunk was its last op)
        if (pc < P_DEC) {
            const int it = pc - P_AS;
            return {OP_Q + s_last(it) + DIST, before_barrier(OP_P + t_first(it))};
        }
        if (pc < P_VS) return {OP_Q, before_barrier(OP_K + (pc - P_DEC))};
        if (pc < P_VB) {
            const int tt = pc - P_VS;
            return {OP_T + t_last(tt) + DIST, before_barrier(OP_K + KT * (tt / 2))};
        }
        if (pc < P_SB) {
            const int s = pc - P_VB;
            return {OP_T + t_last(2 * s + 1) + DIST, OP_P + s_first(s)};
        }
        // The new state slab, from the tiles 2 s and 2 s + 1 that the last group finishes; without the output groups
        // behind it the last slabs no longer fit this chunk: they are packed at the start of the next one, before the
        // first MFMA that takes them (op 2 s of K S0; the loop is entered with all slabs packed, so chunk 0 packs them twice)
        const int s = pc - P_SB;
        const int first = OP_K + KT + 2 * s + 1 + DIST;
        if (NOOUT && first >= NOPS) return {first - NOPS, 2 * s};
        return {first, NOPS};
    }
    struct Table {
        int op[NPIECES];
        bool ok;
    };
    static constexpr Table make() {
        Table t{};
        bool done[NPIECES] = {};
        int left = NPIECES;
        t.ok = true;
        for (int op = 0; op < NOPS; op++) {
            const int quota = (left + (NOPS - op) - 1) / (NOPS - op);
            for (int n = 0;; n++) {
                int best = -1;
                for (int pc = 0; pc < NPIECES; pc++)
                    if (!done[pc] && window(pc).first <= op && (best < 0 || window(pc).end < window(best).end)) best = pc;
                if (best < 0) break;
                if (n >= quota && window(best).end > op + 1) break;
                if (window(best).end <= op) t.ok = false;  // window missed
                t.op[best] = op, done[best] = true, left--;
            }
        }
        if (left != 0) t.ok = false;
        // a slab of X is packed after the X of both its tiles (within an op the pieces run in index order)
        for (int s = 0; s < N_XB; s++)
            if (t.op[P_XB + s] < t.op[P_XC + 2 * s] || t.op[P_XB + s] < t.op[P_XC + 2 * s + 1]) t.ok = false;
        // what a piece reads of this chunk's half of the stage is read before the barrier; the decay and the row scale
        // of q use values that the barrier op replaces
        for (int i = 0; i < N_VS; i++)
            if (t.op[P_VS + i] - AHEAD < 0 || t.op[P_VS + i] >= OP_BAR) t.ok = false;
        for (int i = 0; i < N_XC; i++)
            if (t.op[P_XC + i] - AHEAD < 0 || t.op[P_XC + i] >= OP_BAR) t.ok = false;
        for (int i = 0; i < N_DEC; i++)
            if (t.op[P_DEC + i] >= OP_BAR) t.ok = false;
        for (int i = 0; i < N_AS; i++)
            if (t.op[P_AS + i] >= OP_BAR) t.ok = false;
        return t;
    }
};

template <int K, bool NOOUT = false>
struct Scan16Schedule : Scan16Rules<K, NOOUT> {
    static constexpr typename Scan16Rules<K, NOOUT>::Table TABLE = Scan16Rules<K, NOOUT>::make();
    static_assert(TABLE.ok, "no placement of the side work satisfies the windows");
    static constexpr int op_of(int pc) { return TABLE.op[pc]; }
};

// NT: the loaders use non-temporal loads.  Right when no other workgroup reads the same lines (one workgroup per
// chain; measured 7 % faster at 1024 chains), wrong when column groups share them through the L2 (8 % slower).
//
// HALF (one slice per workgroup): the slice has two waves, each with 16 of its columns, on v_mfma_f32_16x16x32_bf16.
// A wave has the same number of MFMAs and operand reads as a whole-slice wave but half the accumulators, so half the
// vector work on them (decay, X, the bf16 copies), and the two halves need nothing from each other.  The records must
// hold the fragments of T diag(beta) and P in the layout of that instruction (ChunkParams::rec16).
//
// NOOUT (with SAVE and HALF, K <= 128): the scan writes no output and skips the products that form it; what it saves (the
// state every chunk starts from, V~) is all it is run for.  The loaders still stage the whole record and the rows of q.
template <int K, int NW, bool NT = false, bool SAVE = false, bool HALF = false, bool NOOUT = false>
__global__ __launch_bounds__(scan_waves(NW, HALF) * WAVE) void chunk_scan32_kernel(const ChunkParams p) {
    static_assert(!HALF || NW == 1, "the half-slice scan has one slice per workgroup");
    static_assert(!NOOUT || (SAVE && HALF && K >= 128), "the scan without output is the saving half-slice scan at K = 128 or 256");
    // K = 256: two stage halves with the rows of q and k do not fit the LDS.  The rows of q, which a chunk needs for
    // one group of MFMAs only, then get a single buffer and a second workgroup barrier per chunk ("barrier Q"), passed
    // by a compute wave once it holds the last fragment of q: the loaders write the next chunk's rows of q between
    // that barrier and the one at the end of the chunk.
    // Without output (NOOUT) no row of q is staged at all: K = 256 then fits two stage halves, needs no barrier Q, and has
    // room for the staging of the saves.
    constexpr bool HASQ = !NOOUT;
    constexpr bool QS = K > 128 && HASQ;
    static_assert(K <= 128 || HALF, "K = 256 runs as half slices");
    constexpr int NL = SCAN_LOADERS;
    // a separate wave writes the output (see below); with four compute waves the LDS has no room for its staging
    constexpr bool OS = NW < 4;
    constexpr int KD = K / 32;    // 32-row tiles of the state
    constexpr int KS16 = K / 16;  // 16-wide slabs over the key dim
    // One half of the stage: [T diag(beta) 6 | P 6] (the head of the record) | the chunk's 64 rows of this
    // workgroup's columns of v | of q | of k, row-major, copied from the caller's tensors | 64 row scales of q |
    // of k for the state update | of k S0 | e^{gamma_C}
    constexpr int SHARED_FRAGS = 12;
    constexpr int SHARED_BYTES = SHARED_FRAGS * FRAG_BYTES;
    constexpr int VROW = 64 * NW;                    // bytes per row of v held by this workgroup (32 columns per compute wave)
    constexpr int VLD = VROW + 16;                   // bytes per staged row of v
    constexpr int V_UNITS = C * VROW / FRAG_BYTES;   // 1 KiB pieces of the v rows: 1024 / VROW whole rows each
    constexpr int QLD = 2 * K + 16;                  // bytes per staged row of q / k (16 bytes of padding against bank conflicts)
    constexpr int Q_UNITS = C * 2 * K / FRAG_BYTES;  // 1 KiB pieces of the q rows: 512 / K whole rows each; as many for k
    constexpr int V_OFF = SHARED_BYTES;
    constexpr int Q_OFF = V_OFF + C * VLD;                 // not part of the stage halves when QS
    constexpr int K_OFF = (QS || !HASQ) ? Q_OFF : Q_OFF + C * QLD;
    constexpr int QS_OFF = K_OFF + C * QLD;
    constexpr int KS_OFF = QS_OFF + C * 4;
    constexpr int CS_OFF = KS_OFF + C * 4;
    constexpr int EG_OFF = CS_OFF + C * 4;
    constexpr int STAGE_BYTES = EG_OFF + 16;
    constexpr int NF = SHARED_FRAGS / NL;  // fragment slots per loader wave
    constexpr int NV = V_UNITS / NL;       // v row slots per loader wave
    constexpr int NQ = (HASQ ? 2 : 1) * Q_UNITS / NL;   // q / k row slots per loader wave
    constexpr int NLOAD = NF + NV + NQ;    // 1 KiB moves per loader wave and chunk
    static_assert(SHARED_FRAGS % NL == 0 && V_UNITS % NL == 0 && (2 * Q_UNITS) % NL == 0, "the pieces must divide over the loader waves");
    constexpr int OSTAGE_BYTES = (OS && !NOOUT) ? NW * 2 * C * 64 : 16;
    static_assert(2 * STAGE_BYTES + (QS ? C * QLD : 0) + OSTAGE_BYTES <= 160 * 1024, "stage exceeds LDS");

    __shared__ __attribute__((aligned(16))) uint8_t stage[2][STAGE_BYTES];
    __shared__ __attribute__((aligned(16))) uint8_t qstage[QS ? C * QLD : 16];  // the single buffer of q rows (QS)
    __shared__ __attribute__((aligned(16))) uint8_t ostage[OSTAGE_BYTES];
    // LSAVE (the saving half-slice scan, K <= 128): the compute waves leave the state a chunk starts from and V~ in LDS, as
    // rows of the slice's 32 fp32 columns, and the store wave writes them out in whole 128-byte lines.  Stores from the
    // compute waves themselves are 64-byte halves of those lines from two waves, and a store that waits for room in the
    // memory queue stalls the wave that feeds the matrix pipe.  Two buffers each, by chunk parity.  (K = 256 has no LDS
    // left for them and stores from its compute waves.)
    // K = 256 (NOOUT only) has half of that room: its states are staged in one buffer when they are fp32 - the launcher
    // asks for them at every second chunk at most then, so the store wave is done with a state before the next one is
    // staged - and in two when they are bf16; its V~ is bf16.
    constexpr bool LSAVE = SAVE && HALF && (K <= 128 || NOOUT);
    constexpr bool LSAVE_NARROW = LSAVE && K > 128;
    constexpr int SROW = 32 * 4;  // bytes per staged row of fp32
    // bf16 saves are staged TRANSPOSED, [32 columns][K + 8 keys] (V~: [32 columns][64 + 8 tokens]): a compute-wave lane holds
    // four consecutive keys (tokens) of one column, so it stages them with one 8-byte write instead of four 2-byte ones
    // (48 LDS writes per chunk became 12: the staging was 1,660 of the 4,030 cycles of a saving chunk step), and the
    // store wave turns them back into rows with the transposing LDS load on its way out.
    constexpr int SCOL = (K + 8) * 2, VCOL = (C + 8) * 2;  // bytes per staged column
    constexpr int SSTAGE_HALF = LSAVE ? (LSAVE_NARROW ? 32 * SCOL : K * SROW) : 8;
    constexpr int VSTAGE_HALF = LSAVE ? (LSAVE_NARROW ? 32 * VCOL : C * SROW) : 8;
    static_assert(32 * SCOL <= K * SROW && 32 * VCOL <= C * SROW, "the transposed bf16 staging fits the fp32 one");
    __shared__ __attribute__((aligned(16))) uint8_t sstage_raw[2 * SSTAGE_HALF];
    __shared__ __attribute__((aligned(16))) uint8_t vstage_raw[2 * VSTAGE_HALF];
    static_assert(!LSAVE || 2 * STAGE_BYTES + OSTAGE_BYTES + 2 * SSTAGE_HALF + 2 * VSTAGE_HALF <= 160 * 1024, "the staging of the saves exceeds LDS");
    // staging buffer of the state chunk c starts from / of its V~ (narrow fp32 states: a single buffer, see above)
    auto sstage_of = [&](int c) -> uint8_t* { return sstage_raw + ((LSAVE_NARROW && !p.save_state_bf16) ? 0 : (c & 1) * SSTAGE_HALF); };
    auto vstage_of = [&](int c) -> uint8_t* { return vstage_raw + (c & 1) * VSTAGE_HALF; };
    // entry of the save arrays that chunk c goes to, or -1; with save_reverse the chain's last saved chunk goes to entry 0
    // (save_last: the entry of its first one - save_nc - 1 unless the chain is a shorter row of a left-padded batch of
    // given records, set below)
    int save_last = p.save_nc - 1;
    auto save_entry = [&](int c) -> int {
        if (c % p.save_every != 0 || c / p.save_every >= p.save_nc) return -1;
        return p.save_reverse ? save_last - c / p.save_every : c / p.save_every;
    };

    const int lane = threadIdx.x % WAVE;
    const int wave = threadIdx.x / WAVE;
    const int l32 = lane % 32, lh = lane / 32;

    // workgroup -> (sequence-head chain, column group); the groups of a chain stay on one XCD (id % 8)
    // so that the lines they share are fetched into a single L2
    const int id = blockIdx.x;
    const int xcd = id % 8, rest = id / 8;
    const int vgroup = rest % p.scan_groups;
    const int per_xcd = (p.N * p.H + 7) / 8;
    int n, h;
    const int32_t* const order = p.cu_seqlens != nullptr ? p.seq_order : p.row_order;  // (row_order: left-padded rows of given records)
    if (order == nullptr) {
        // XCD x takes the chains x * per_xcd .. : consecutive chains are different heads
        const int chain = xcd * per_xcd + rest / p.scan_groups;
        if (rest / p.scan_groups >= per_xcd || chain >= p.N * p.H) return;  // whole workgroup
        n = chain / p.H, h = chain % p.H;
    } else {
        // Packed batches: the chains in the order (sequence by decreasing length, head) are dealt out eight at a time, one
        // per XCD, and workgroups start in the order of their ids: the longest chains first.  The deal is rotated from
        // one eight to the next, so that an XCD does not keep getting the same heads (rows of one head lie a whole
        // token row apart and fall on few channels of its L2).
        const int i = rest / p.scan_groups;
        const int rank = 8 * i + ((xcd - i) % 8 + 8) % 8;
        if (i >= per_xcd || rank >= p.N * p.H) return;  // whole workgroup
        n = order[rank / p.H], h = rank % p.H;
    }
    const int chain = n * p.H + h;

    int slot_begin, slot_end;
    int64_t b, seq_t0, seq_len;
    if (p.cu_seqlens == nullptr) {
        seq_len = p.pad_lens == nullptr ? p.T : min(max(p.pad_lens[n + 1] - p.pad_lens[n], 0), p.T);  // the last seq_len tokens of row n
        slot_begin = n * p.NT, slot_end = slot_begin + (int)((seq_len + C - 1) / C);
        b = n, seq_t0 = p.T - seq_len;
    } else {
        slot_begin = p.chunk_off[n], slot_end = p.chunk_off[n + 1];
        int t0, len;
        packed_bounds(p.cu_seqlens, n, p.T, t0, len);
        b = 0, seq_t0 = t0, seq_len = min(len, (slot_end - slot_begin) * C);
    }
    const int nchunks = slot_end - slot_begin;
    // Given records of a left-padded batch lie at the slots of the tokens they cover, the last ones of the row; and a
    // reverse save counts from the row's own last chunk.
    const bool padded_given = p.records_given && p.pad_lens != nullptr;
    if (padded_given) save_last = min(p.save_nc, (nchunks + p.save_every - 1) / p.save_every) - 1;
    const uint8_t* rec = p.rec + ((int64_t)h * p.TC + slot_begin + (padded_given ? p.NT - nchunks : 0)) * p.rec_bytes;

    // output staging: [compute wave][chunk parity][64 tokens][64 bytes], the four 16-byte pieces of a row
    // XOR-swizzled with (row / 4) % 4 so that both sides access it without bank conflicts
    auto ostage_at = [&](int w, int parity, int row, int piece) -> uint8_t* {
        return ostage + ((w * 2 + parity) * C + row) * 64 + ((piece ^ ((row >> 2) & 3)) << 4);
    };
    // role of this wave (see scan_waves)
    const bool is_store = OS && wave == 4;
    constexpr bool EIGHT = NW == 2 || HALF;  // the wave layout of two compute waves
    const bool is_loader = NW == 4 ? wave >= 4 : EIGHT ? (wave == 2 || wave == 3 || wave >= 6) : (wave >= 1 && wave != 4);
    if (EIGHT && wave == 5) return;
    if (is_store) {
        // ------------------------------ output store ------------------------------
        // The compute waves leave the bf16 output tile of chunk c in LDS while they work on chunk c + 1; this
        // wave writes it out after the next barrier.  A store that waits for queue space then stalls here and
        // not in the wave that feeds the matrix pipe.
        const int row0 = lane / 4, piece = lane % 4;
        bf16_t* og = p.o + b * p.o_stride_b + (seq_t0 + row0) * p.o_stride_t + (int64_t)h * p.o_stride_h +
                     32 * (vgroup * NW) + 8 * piece;
        auto flush = [&](int c) {  // output of chunk c
            const int valid = (int)min((int64_t)C, seq_len - (int64_t)c * C);
#pragma unroll
            for (int w = 0; w < NW; w++) {
                bf16x8 rows[4];
#pragma unroll
                for (int i = 0; i < 4; i++)
                    rows[i] = *reinterpret_cast<const bf16x8*>(ostage_at(w, c & 1, row0 + 16 * i, piece));
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (row0 + 16 * i < valid)
                        __builtin_nontemporal_store(rows[i], reinterpret_cast<bf16x8*>(og + ((int64_t)c * C + 16 * i) * p.o_stride_t + 32 * w));
            }
        };
        // LSAVE, bf16 saves: staged as [32 columns][ld rows]; out as rows of 32 columns (64 bytes): lane group `piece`
        // (16 lanes) takes columns 8 piece .. + 7 of 16 consecutive rows through two transposing loads (4 columns x 16 rows
        // each), so an instruction writes 16 rows of 64 bytes, 4 lanes per row
        // (save_sliced: slice by slice, a slice's rows of 64 bytes one after the other - what a workgroup saves of a chunk
        // is one contiguous block: element (row, column) at (column / 32) rows 32 + row 32 + column % 32)
        auto flush_rows16 = [&](const uint8_t* staged, int ld, bf16_t* dst, int rows) {  // dst: row 0, column 0 of this slice
            const int l16 = lane % 16, piece = lane / 16;
            const bf16_t* const m = reinterpret_cast<const bf16_t*>(staged);
            for (int r = 0; r < rows; r += 64) {
                bf16x8 x[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const bf16x4 lo = lds_read_tr4x16<false>(m, ld, 8 * piece, r + 16 * i, l16);
                    const bf16x4 hi = lds_read_tr4x16<false>(m, ld, 8 * piece + 4, r + 16 * i, l16);
#pragma unroll
                    for (int e = 0; e < 4; e++) x[i][e] = lo[e], x[i][4 + e] = hi[e];
                }
#pragma unroll
                for (int i = 0; i < 4; i++)
                {
                    const int row = r + 16 * i + l16;
                    bf16_t* const at = p.save_sliced ? dst + row * 32 + 8 * piece : dst + (int64_t)row * p.V + 8 * piece;
                    __builtin_nontemporal_store(x[i], reinterpret_cast<bf16x8*>(at));
                }
            }
        };
        // LSAVE: rows of 32 fp32 columns, 8 lanes per row, 8 rows per instruction
        auto flush_rows = [&](const uint8_t* staged, float* dst, int rows) {  // dst: row 0, column 0 of this slice
            const int r0 = lane / 8, piece = lane % 8;
            for (int r = 0; r < rows; r += 32) {
                f32x4 x[4];
#pragma unroll
                for (int i = 0; i < 4; i++) x[i] = *reinterpret_cast<const f32x4*>(staged + (r + 8 * i + r0) * SROW + 16 * piece);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    __builtin_nontemporal_store(x[i], reinterpret_cast<f32x4*>(dst + (int64_t)(r + 8 * i + r0) * p.V + 4 * piece));
            }
        };
        auto flush_state = [&](int c) {  // the state chunk c starts from
            if constexpr (LSAVE) {
                const int entry = save_entry(c);
                if (p.save_state != nullptr && entry >= 0) {
                    const int64_t at = ((int64_t)chain * p.save_nc + entry) * K * p.V + (p.save_sliced ? K * 32 * vgroup : 32 * vgroup);
                    if (p.save_state_bf16) flush_rows16(sstage_of(c), SCOL / 2, reinterpret_cast<bf16_t*>(p.save_state) + at, K);
                    else flush_rows(sstage_of(c), p.save_state + at, K);
                }
            }
        };
        auto flush_vnew = [&](int c) {  // V~ of chunk c
            if constexpr (LSAVE) {
                const int entry = save_entry(c);
                if (p.save_vnew != nullptr && entry >= 0) {
                    const int64_t at = ((int64_t)chain * p.save_nc + entry) * C * p.V + (p.save_sliced ? C * 32 * vgroup : 32 * vgroup);
                    if (p.save_vnew_bf16) flush_rows16(vstage_of(c), VCOL / 2, reinterpret_cast<bf16_t*>(p.save_vnew) + at, C);
                    else flush_rows(vstage_of(c), p.save_vnew + at, C);
                }
            }
        };
        __syncthreads();
#ifdef GDN_CYCLE_BUDGET
        uint64_t store_wait = 0;  // cycles this wave spends at the chunks' barriers (slot 7 of the report)
#endif
        for (int c = 0; c < nchunks; c++) {
            if constexpr (QS) __syncthreads();  // barrier Q
#ifdef GDN_CYCLE_BUDGET
            const uint64_t w0 = __builtin_readcyclecounter();
#endif
            __syncthreads();  // the state of chunk c, V~ and the output of chunk c - 1 are staged
#ifdef GDN_CYCLE_BUDGET
            store_wait += __builtin_readcyclecounter() - w0;
#endif
            flush_state(c);
            if (c > 0) {
                if constexpr (!NOOUT) flush(c - 1);
                flush_vnew(c - 1);
            }
        }
#ifdef GDN_CYCLE_BUDGET
        if (p.cycle_out != nullptr && lane == 0 && blockIdx.x % 16 == 0 && blockIdx.x / 16 < GDN_CYCLE_BUDGET_SLOTS)
            p.cycle_out[(blockIdx.x / 16) * 8 + 7] = store_wait;
#endif
        __syncthreads();
        if (nchunks > 0) {
            if constexpr (!NOOUT) flush(nchunks - 1);
            flush_vnew(nchunks - 1);
        }
        return;
    }
    if (is_loader) {
        // ------------------------------ loader ------------------------------
        // loader number 0..3, wave-uniform: unit numbers and bases stay scalar
        const int lw = __builtin_amdgcn_readfirstlane(NW == 4 ? wave - 4 : EIGHT ? (wave < 4 ? wave - 2 : wave - 4) : (wave < 4 ? wave - 1 : 3));
        // Slots 0 .. NF - 1 of this wave move record fragments lw * NF + (rotated slot), the next NV slots 1 KiB
        // pieces of the v rows, the last NQ slots pieces of the q and k rows.  Which kind a slot is, is known at
        // compile time, so there is no branch in these loops (a branch makes the compiler wait for every load in
        // flight).  The rotation by column group lets the workgroups of a chain ask for different lines at any
        // one time: a line's memory latency is then paid by one of them instead of being waited out by all.
        const int rot_f = vgroup % NF;
        const int rot_q = vgroup % NQ;
        auto frag_of = [&](int i) { return lw * NF + (i + rot_f < NF ? i + rot_f : i + rot_f - NF); };   // i < NF
        auto vunit_of = [&](int i) { return lw * NV + i; };                                              // i < NV
        // (QS: the first NQ / 2 slots of every wave are rows of q, the others rows of k, so that every wave writes its
        // share of q after barrier Q; no rotation, so that a slot's place is the wave's first unit plus a constant)
        constexpr int NQH = NQ / 2;
        auto qunit_of = [&](int i) {  // i < NQ
            if constexpr (QS) {
                return (i < NQH ? 0 : Q_UNITS) + lw * NQH + i % NQH;
            } else {
                return lw * NQ + (i + rot_q < NQ ? i + rot_q : i + rot_q - NQ);
            }
        };
        // rows of q, k: lane -> (row within the unit, 16-byte piece); likewise for v
        constexpr int Q_ROWS = C / Q_UNITS, Q_PIECES = WAVE / Q_ROWS;
        constexpr int V_ROWS = C / V_UNITS, V_PIECES = WAVE / V_ROWS;
        const int q_row = lane / Q_PIECES, q_piece = lane % Q_PIECES;
        const int v_row = lane / V_PIECES, v_piece = lane % V_PIECES;
        const int hqk = qk_head_of(h, p.qk_div);
        const bf16_t* const qg = p.q + b * p.q_stride_b + seq_t0 * p.q_stride_t + (int64_t)hqk * p.q_stride_h + q_piece * 8;
        const bf16_t* const kg = p.k + b * p.k_stride_b + seq_t0 * p.k_stride_t + (int64_t)hqk * p.k_stride_h + q_piece * 8;
        const bf16_t* const vg = p.v + b * p.v_stride_b + seq_t0 * p.v_stride_t + (int64_t)h * p.v_stride_h + 32 * (vgroup * NW) + v_piece * 8;
        // two register buffers: while one chunk is written to LDS, younger ones are in flight
        bf16x8 buf0[NLOAD], buf1[NLOAD];
        // lanes 0..63: row scales of token `lane` (of q, of k for the state update, of k S0), and e^{gamma_C}
        struct Scalars {
            float qs, ks, cs, eg;
        };
        Scalars sc0 = {0.f, 0.f, 0.f, 0.f}, sc1 = {0.f, 0.f, 0.f, 0.f};
        // (QS: wave-uniform 64-bit base of the chunk + 32-bit per-lane byte offset formed at the load, so that no
        // per-slot 64-bit lane addresses stay live: with 20 slots per buffer they would not fit the registers)
        const bf16_t* const qg0 = p.q + b * p.q_stride_b + seq_t0 * p.q_stride_t + (int64_t)hqk * p.q_stride_h;
        const bf16_t* const kg0 = p.k + b * p.k_stride_b + seq_t0 * p.k_stride_t + (int64_t)hqk * p.k_stride_h;
        const bf16_t* const vg0 = p.v + b * p.v_stride_b + seq_t0 * p.v_stride_t + (int64_t)h * p.v_stride_h + 32 * (vgroup * NW);
        // mirror reads (scan without output only): the odd chunks' tensors, and the token a row stands for
        const bool mirror = NOOUT && p.mirror != 0;
        const bf16_t* const kg2 = mirror ? p.k2 + b * p.k2_stride_b + (int64_t)h * p.k2_stride_h + q_piece * 8 : kg;
        const bf16_t* const vg2 = mirror ? p.v2 + b * p.v2_stride_b + (int64_t)h * p.v2_stride_h + 32 * (vgroup * NW) + v_piece * 8 : vg;
        auto src_of = [&](int c, int i) -> const uint8_t* {
            // (mirror reads: selects, not branches - a branch in these loops makes the compiler wait for the loads in flight)
            const bool odd = mirror && (c & 1);
            // the operand fragments of the odd chunks of a mirror problem (T' = I, P = 0) are the same for every chunk:
            // only chunk 1 of a chain carries them, the row scales come from the chunk's own record (load_scalars)
            if (i < NF) return rec + ((int64_t)(odd ? 1 : c) * p.rec_bytes + (int64_t)frag_of(i) * FRAG_BYTES) + lane * 16;
            const int row0_tok = ((nchunks >> 1) - 1 - (c >> 1)) * C + C - 1;  // mirror reads: the token of row 0
            if constexpr (QS) {
                const int last = (int)min((int64_t)C, seq_len - (int64_t)c * C) - 1;  // wave-uniform
                if (i < NF + NV) {
                    const uint32_t off = (uint32_t)min(vunit_of(i - NF) * V_ROWS + v_row, last) * ((uint32_t)p.v_stride_t * 2u) + (uint32_t)v_piece * 16u;
                    return reinterpret_cast<const uint8_t*>(vg0 + (int64_t)c * C * p.v_stride_t) + off;
                }
                // row of this lane in the wave's first unit; hidden from the optimiser at every use, or the offsets of
                // all slots are formed ahead of the loop and held in registers
                int row0 = lw * NQH * Q_ROWS + q_row;
                asm volatile("" : "+v"(row0));
                const bool is_k = i - NF - NV >= NQH;
                const uint32_t stride = (uint32_t)(is_k ? p.k_stride_t : p.q_stride_t) * 2u;
                const uint32_t off = (uint32_t)min(row0 + ((i - NF - NV) % NQH) * Q_ROWS, last) * stride + (uint32_t)q_piece * 16u;
                return reinterpret_cast<const uint8_t*>((is_k ? kg0 : qg0) + (int64_t)c * C * (is_k ? p.k_stride_t : p.q_stride_t)) + off;
            }
            // a row past the end of the sequence (tail chunk) is read from the last token instead: never used
            if (i < NF + NV) {
                const int row = vunit_of(i - NF) * V_ROWS + v_row;
                const int tok = mirror ? row0_tok - row : min(c * C + row, (int)seq_len - 1);
                return reinterpret_cast<const uint8_t*>((odd ? vg2 : vg) + (int64_t)tok * (odd ? p.v2_stride_t : p.v_stride_t));
            }
            // units 0 .. Q_UNITS - 1 are rows of q, the rest rows of k (wave-uniform choice); without q all are rows of k
            const int u = qunit_of(i - NF - NV);
            const bool is_k = !HASQ || u >= Q_UNITS;
            const int row = ((is_k && HASQ) ? u - Q_UNITS : u) * Q_ROWS + q_row;
            const int tok = mirror ? row0_tok - row : min(c * C + row, (int)seq_len - 1);
            return reinterpret_cast<const uint8_t*>((is_k ? (odd ? kg2 : kg) : qg) + (int64_t)tok * (is_k ? (odd ? p.k2_stride_t : p.k_stride_t) : p.q_stride_t));
        };
        auto dst_of = [&](uint8_t* st, int i) -> uint8_t* {
            if (i < NF) return st + frag_of(i) * FRAG_BYTES + lane * 16;
            if (i < NF + NV) return st + V_OFF + (vunit_of(i - NF) * V_ROWS + v_row) * VLD + v_piece * 16;
            if constexpr (QS) {
                // the lane's place in the wave's first unit plus a compile-time constant
                const int lane_off = (lw * NQH * Q_ROWS + q_row) * QLD + q_piece * 16;
                const int slot_off = ((i - NF - NV) % NQH) * Q_ROWS * QLD;
                if (i - NF - NV < NQH) return qstage + lane_off + slot_off;
                return st + K_OFF + lane_off + slot_off;
            } else {
                return st + Q_OFF + (qunit_of(i - NF - NV) * Q_ROWS + q_row) * QLD + q_piece * 16;  // the k rows follow the q rows
            }
        };
        // every loader wave carries the scales (identical values, identical LDS writes)
        auto load_scalars = [&](Scalars& sc, int c) {
            const uint8_t* r = rec + (int64_t)c * p.rec_bytes;
            sc.qs = reinterpret_cast<const float*>(r + p.off_qs)[lane];
            sc.ks = reinterpret_cast<const float*>(r + p.off_ks)[lane];
            sc.cs = reinterpret_cast<const float*>(r + p.off_cs)[lane];
            sc.eg = *reinterpret_cast<const float*>(r + p.off_eg);
        };
        auto fetch = [&](const uint8_t* src) -> bf16x8 {
            if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(src));
            else return *reinterpret_cast<const bf16x8*>(src);
        };
        auto load = [&](bf16x8(&buf)[NLOAD], Scalars& sc, int c) {
#pragma unroll
            for (int i = 0; i < NLOAD; i++) buf[i] = fetch(src_of(c, i));
            load_scalars(sc, c);
        };
        // write chunk c to LDS and refill each register with chunk c2 right behind its write, so the
        // LDS-write and the vector-memory queues fill together
        // (QS: the rows of q, slots NF + NV .. NF + NV + NQH - 1, go last, after barrier Q when `barrier_q` is set)
        auto store_and_reload = [&](bf16x8(&buf)[NLOAD], Scalars& sc, int c, int c2, auto reload_tag, auto barrier_q_tag) {
            constexpr bool reload = decltype(reload_tag)::value;
            constexpr bool barrier_q = decltype(barrier_q_tag)::value;
            uint8_t* dst = stage[c & 1];
            reinterpret_cast<float*>(dst + QS_OFF)[lane] = sc.qs;
            reinterpret_cast<float*>(dst + KS_OFF)[lane] = sc.ks;
            reinterpret_cast<float*>(dst + CS_OFF)[lane] = sc.cs;
            if (lane == 0) *reinterpret_cast<float*>(dst + EG_OFF) = sc.eg;
#pragma unroll
            for (int i = 0; i < NLOAD; i++) {
                if (QS && i >= NF + NV && i < NF + NV + NQH) continue;
                *reinterpret_cast<bf16x8*>(dst_of(dst, i)) = buf[i];
                if constexpr (reload) buf[i] = fetch(src_of(c2, i));
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (QS) {
                if constexpr (barrier_q) __syncthreads();  // barrier Q: the compute waves have read the rows of q in the buffer
#pragma unroll
                for (int i = NF + NV; i < NF + NV + NQH; i++) {
                    *reinterpret_cast<bf16x8*>(dst_of(dst, i)) = buf[i];
                    if constexpr (reload) buf[i] = fetch(src_of(c2, i));
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if constexpr (reload) load_scalars(sc, c2);
        };
        constexpr std::true_type yes{};
        constexpr std::false_type no{};
        // chunks 0 (-> LDS now), 1 and 2 (in flight); even chunks use buf0, odd ones buf1
        if (nchunks > 0) {
            load(buf0, sc0, 0);
            if (nchunks > 1) load(buf1, sc1, 1);
            if (nchunks > 2) store_and_reload(buf0, sc0, 0, 2, yes, no);
            else store_and_reload(buf0, sc0, 0, 0, no, no);
        }
        __syncthreads();  // stage[0] holds chunk 0
        // Barrier of iteration c: the compute waves are done with stage[c & 1] and chunk c + 1 is in the
        // other half.  Before it: write chunk c + 1 (its half was released by the barrier of iteration
        // c - 1) and refill the freed registers with chunk c + 3.
        int c = 0;
        // (QS: every iteration has barrier Q as well: inside store_and_reload, or on its own when nothing is left to write)
        for (; c + 4 < nchunks; c += 2) {  // steady state: straight-line code, both reloads exist
            store_and_reload(buf1, sc1, c + 1, c + 3, yes, yes);
            __syncthreads();
            store_and_reload(buf0, sc0, c + 2, c + 4, yes, yes);
            __syncthreads();
        }
        for (; c < nchunks; c += 2) {  // the last (at most four) chunks
            if (c + 1 < nchunks) {
                if (c + 3 < nchunks) store_and_reload(buf1, sc1, c + 1, c + 3, yes, yes);
                else store_and_reload(buf1, sc1, c + 1, 0, no, yes);
            } else if constexpr (QS) {
                __syncthreads();
            }
            __syncthreads();
            if (c + 1 < nchunks) {
                if (c + 2 < nchunks) store_and_reload(buf0, sc0, c + 2, 0, no, yes);
                else if constexpr (QS) __syncthreads();
                __syncthreads();
            }
        }
        if (OS) __syncthreads();  // the hand-over of the last output tile
        return;
    }

    if constexpr (HALF) {
        // ------------------------------ compute (HALF) ------------------------------
        // Lane (j, g) = (lane % 16, lane / 16).  Operands of the 16x16x32 MFMA: A[j][8 g + 0..7], B[8 g + 0..7][j]; its
        // accumulator: D[4 g + r][j], r = 0..3.  This wave owns the 16 columns c0 + j of the slice.
        //   state tile t (K / 16 of them), register r: key 32 (t / 2) + 8 g + 4 (t % 2) + r.  Tiles 2 s and 2 s + 1 together
        //     hand a lane the 8 consecutive keys 32 s + 8 g + 0..7: one operand register set, usable as B of K S0 (rows
        //     of k are read as they lie) and as A of O^T = S0^T q^T.
        //   token tile tt of K S0, X, V~ (16 tokens each), register r: token 16 tt + 4 g + r.  Tiles 2 s and 2 s + 1 hand
        //     over the tokens 32 s + 4 g + 0..3 and 32 s + 16 + 4 g + 0..3: the reduction order of every fragment of
        //     T diag(beta), P and k^T that multiplies them.
        //   O^T tile it, register r: column c0 + 4 g + r of token 16 it + j.
        typedef Scan16Schedule<K, NOOUT> SCH;
        constexpr int NOPS = SCH::NOPS, OP_Q = SCH::OP_Q, OP_T = SCH::OP_T, OP_K = SCH::OP_K, OP_P = SCH::OP_P, OP_BAR = SCH::OP_BAR;
        constexpr int LA = SCH::LA, KS = SCH::KS, KT = SCH::KT;
        const int j16 = lane % 16, g = lane / 16;
        const int half = wave;  // 0 or 1
        const int c0 = 32 * vgroup + 16 * half;
        auto out_tile = [&](const f32x4& acc, int parity, int it) {  // 4 columns of token 16 it + j to the output staging
            bf16x4 o4;
#pragma unroll
            for (int e = 0; e < 4; e++) o4[e] = (bf16_t)acc[e];
            *reinterpret_cast<bf16x4*>(ostage_at(0, parity, 16 * it + j16, 2 * half + g / 2) + 8 * (g % 2)) = o4;
        };
        f32x4 S[KT];
        auto st_key = [&](int t, int r) { return 32 * (t / 2) + 8 * g + 4 * (t % 2) + r; };
        const int64_t st_off = ((int64_t)n * p.H + h) * K * p.V + c0 + j16;
#pragma unroll
        for (int t = 0; t < KT; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) S[t][r] = p.h0 != nullptr ? p.h0[st_off + (int64_t)st_key(t, r) * p.V] : 0.f;

        auto lds_frag = [&](const uint8_t* st, auto opc) -> bf16x8 {
            constexpr int op = decltype(opc)::value;
            if constexpr (op < OP_T) {  // rows of k (A of K S0) or of q (B of S0^T q^T): token tile, 32-key slab
                constexpr int jj = op < OP_Q ? op : op - OP_Q, sl = SCH::s_slab(jj), tt = SCH::s_tile(jj);
                const uint8_t* rows = op < OP_Q ? st + K_OFF : QS ? qstage : st + Q_OFF;
                return *reinterpret_cast<const bf16x8*>(rows + (16 * tt + j16) * QLD + (32 * sl + 8 * g) * 2);
            } else if constexpr (op >= OP_K && op < OP_P) {
                // k^T: row j of key tile t is key 32 (t / 2) + 8 (j / 4) + 4 (t % 2) + j % 4; tokens 32 s + 4 g + 0..3 and
                // 32 s + 16 + 4 g + 0..3.  Two transposing loads; lane (4 r' + q) supplies keys base + 8 q + 0..3 of token row r'.
                constexpr int sl = SCH::k_slab(op - OP_K), t = SCH::k_tile(op - OP_K);
                const bf16_t* km = reinterpret_cast<const bf16_t*>(st + K_OFF) + (32 * sl + 4 * g + j16 / 4) * (QLD / 2) + 32 * (t / 2) + 4 * (t % 2) + 8 * (j16 % 4);
                const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)km);
                const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(km + 16 * (QLD / 2)));
                const bf16x4 a4 = __builtin_bit_cast(bf16x4, a), b4 = __builtin_bit_cast(bf16x4, b);
                bf16x8 r;
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = a4[e], r[4 + e] = b4[e];
                return r;
            } else {
                constexpr int f = op < OP_K ? SCH::t_frag(op - OP_T) : 6 + SCH::t_frag(op - OP_P);  // T' | P are contiguous in the stage
                return reinterpret_cast<const bf16x8*>(st)[f * WAVE + lane];
            }
        };
        auto lds_eg = [&](const uint8_t* st) -> float { return *reinterpret_cast<const float*>(st + EG_OFF); };
        auto lds_qs = [&](const uint8_t* st, int it) -> float { return reinterpret_cast<const float*>(st + QS_OFF)[16 * it + j16]; };
        auto pack4x2 = [](const f32x4& a, const f32x4& b) {
            bf16x8 r;
#pragma unroll
            for (int e = 0; e < 4; e++) r[e] = (bf16_t)a[e], r[4 + e] = (bf16_t)b[e];
            return r;
        };

        f32x4 accv[4], vt[4], acco[4];
        bf16x8 sb[KS], xb[2], vb[2], vbs[2], fnext[LA];
        f32x4 ksr[4], csr[4];
        bf16x4 xvr[4];
        float egc, qsc[4];
#pragma unroll
        for (int it = 0; it < 4; it++)
#pragma unroll
            for (int r = 0; r < 4; r++) acco[it][r] = 0.f;

        __syncthreads();  // stage[0] holds chunk 0
        egc = lds_eg(stage[0]);
        if constexpr (!NOOUT) {
#pragma unroll
            for (int it = 0; it < 4; it++) qsc[it] = lds_qs(stage[0], it);
        }
        static_for<0, LA>([&](auto i) { fnext[decltype(i)::value] = lds_frag(stage[0], i); });
#pragma unroll
        for (int sl = 0; sl < KS; sl++) sb[sl] = pack4x2(S[2 * sl], S[2 * sl + 1]);

#ifdef GDN_CYCLE_BUDGET
        // Measurement build (python -m lm_engine_amd.build --cycle-budget): the shader clock is read where one group of
        // MFMAs of the chunk ends and the next begins, and the cycles of each group, side work included, are added up
        // over the chunks: [K S0 | O^T = S0^T q^T | V~ = T' X | S += k^T V~ | O^T += V~^T P^T | from the last MFMA of a chunk
        // to the first of the next].  Every reading waits for the wave's LDS reads in flight, which costs the measured
        // loop a few hundred cycles per chunk.
        uint64_t cyc[6] = {0, 0, 0, 0, 0, 0};
        uint64_t cyc_t0 = __builtin_readcyclecounter();
        auto cyc_tick = [&](int group) {
            const uint64_t t1 = __builtin_readcyclecounter();
            cyc[group] += t1 - cyc_t0;
            cyc_t0 = t1;
            __builtin_amdgcn_sched_barrier(0);
        };
#endif
        for (int c = 0; c < nchunks; c++) {
            const uint8_t* st = stage[c & 1];
            const uint8_t* stn = stage[(c + 1) & 1];
            if constexpr (SAVE) {
                // the state this chunk starts from, for the backward pass (one wave-uniform base plus one per-lane
                // byte offset, as in the whole-slice scan)
                if constexpr (LSAVE) {
                    // into this chunk's staging buffer (read by the store wave after this chunk's barrier, written again two
                    // chunks on, after the next chunk's barrier)
                    if (p.save_state != nullptr && save_entry(c) >= 0) {
                        if (p.save_state_bf16) {
                            // column 16 half + j16, keys 32 (t / 2) + 4 (t % 2) + 8 g + 0..3 of tile t: one 8-byte write
                            uint8_t* const base = sstage_of(c) + (16 * half + j16) * SCOL + (8 * g) * 2;
#pragma unroll
                            for (int t = 0; t < KT; t++) {
                                bf16x4 x;
                                x.x = (bf16_t)S[t][0], x.y = (bf16_t)S[t][1], x.z = (bf16_t)S[t][2], x.w = (bf16_t)S[t][3];
                                *reinterpret_cast<bf16x4*>(base + (32 * (t / 2) + 4 * (t % 2)) * 2) = x;
                            }
                        } else {
                            uint8_t* const base = sstage_of(c) + (8 * g) * SROW + (16 * half + j16) * 4;
#pragma unroll
                            for (int t = 0; t < KT; t++)
#pragma unroll
                                for (int r = 0; r < 4; r++) *reinterpret_cast<float*>(base + (32 * (t / 2) + 4 * (t % 2) + r) * SROW) = S[t][r];
                        }
                    }
                } else if (p.save_state != nullptr && c % p.save_every == 0 && c / p.save_every < p.save_nc) {
                    const int entry = p.save_reverse ? save_last - c / p.save_every : c / p.save_every;
                    char* base = reinterpret_cast<char*>(p.save_state + ((int64_t)chain * p.save_nc + entry) * K * p.V);
                    const uint32_t lane_off = (uint32_t)((8 * g) * p.V + c0 + j16) * 4u;
                    const uint32_t row_bytes = (uint32_t)p.V * 4u;
#pragma unroll
                    for (int t = 0; t < KT; t++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            *reinterpret_cast<float*>(base + (size_t)((32 * (t / 2) + 4 * (t % 2) + r) * row_bytes) + lane_off) = S[t][r];
                }
            }
            bf16x8 fr[NOPS];
#pragma unroll
            for (int i = 0; i < LA; i++) fr[i] = fnext[i];
            __builtin_amdgcn_sched_barrier(0);

            auto run_piece = [&](auto pcc) {
                constexpr int pc = decltype(pcc)::value;
                if constexpr (pc < SCH::P_XB) {  // X = V - diag(cs) (K S0), token tile tt
                    constexpr int tt = pc - SCH::P_XC;
#pragma unroll
                    for (int e = 0; e < 4; e++) accv[tt][e] = (float)xvr[tt][e] - csr[tt][e] * accv[tt][e];
                } else if constexpr (pc < SCH::P_OUT) {
                    constexpr int sl = pc - SCH::P_XB;
                    xb[sl] = pack4x2(accv[2 * sl], accv[2 * sl + 1]);
                } else if constexpr (pc < SCH::P_AS) {  // output tile `it` of the previous chunk: 4 columns of token 16 it + j
                    constexpr int it = pc - SCH::P_OUT;
                    if (c > 0) out_tile(acco[it], (c - 1) & 1, it);
                } else if constexpr (pc < SCH::P_DEC) {
                    constexpr int it = pc - SCH::P_AS;
#pragma unroll
                    for (int e = 0; e < 4; e++) acco[it][e] *= qsc[it];
                } else if constexpr (pc < SCH::P_VS) {
                    constexpr int t = pc - SCH::P_DEC;
#pragma unroll
                    for (int e = 0; e < 4; e++) S[t][e] *= egc;
                } else if constexpr (pc < SCH::P_VB) {  // V~ of token tile tt with its rows scaled for the state update
                    constexpr int tt = pc - SCH::P_VS;
#pragma unroll
                    for (int e = 0; e < 4; e++) vbs[tt / 2][4 * (tt % 2) + e] = (bf16_t)(vt[tt][e] * ksr[tt][e]);
                } else if constexpr (pc < SCH::P_SB) {
                    constexpr int sl = pc - SCH::P_VB;
                    vb[sl] = pack4x2(vt[2 * sl], vt[2 * sl + 1]);
                } else {
                    constexpr int sl = pc - SCH::P_SB;
                    sb[sl] = pack4x2(S[2 * sl], S[2 * sl + 1]);
                    pin_regs(sb[sl]);
                }
            };

            static_for<0, NOPS>([&](auto opc) {
                constexpr int op = decltype(opc)::value;
#ifdef GDN_CYCLE_BUDGET
                if constexpr (op == 0) cyc_tick(5);
                else if constexpr (op == OP_Q && !NOOUT) cyc_tick(0);
                else if constexpr (op == OP_T) cyc_tick(NOOUT ? 0 : 1);
                else if constexpr (op == OP_K) cyc_tick(2);
                else if constexpr (op == OP_P && !NOOUT) cyc_tick(3);
#endif
                if constexpr (op + LA < NOPS) fr[op + LA] = lds_frag(st, std::integral_constant<int, (op + LA < NOPS ? op + LA : 0)>{});
                if constexpr (op == OP_BAR) {
#ifdef GDN_CYCLE_BUDGET
                    if constexpr (NOOUT) cyc_tick(3);  // (the scan without output has groups 1 and 4 to spare: 4 = the wait at the barrier)
#endif
                    __syncthreads();  // this wave is done with chunk c's half; chunk c + 1 is in the other one
#ifdef GDN_CYCLE_BUDGET
                    if constexpr (NOOUT) cyc_tick(4);
#endif
                    egc = lds_eg(stn);
                    if constexpr (!NOOUT) {
#pragma unroll
                        for (int it = 0; it < 4; it++) qsc[it] = lds_qs(stn, it);
                    }
                }
                if constexpr (QS && op == OP_T) {
                    // Barrier Q.  The MFMA before this point took the last fragment of q, and LDS reads return in order:
                    // no read of the q buffer is outstanding, so the barrier needs no wait for the reads still in flight.
                    static_assert(OP_T < OP_BAR && OP_Q >= LA, "barrier Q comes first and the prefetch across the chunk barrier holds no q");
                    __builtin_amdgcn_s_barrier();
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (op >= OP_BAR) fnext[op >= OP_BAR ? op - OP_BAR : 0] = lds_frag(stn, std::integral_constant<int, (op >= OP_BAR ? op - OP_BAR : 0)>{});
                static_for<0, SCH::N_VS>([&](auto ic) {
                    constexpr int i = decltype(ic)::value;
                    if constexpr (SCH::op_of(SCH::P_VS + i) - SCH::AHEAD == op)
                        ksr[i] = *reinterpret_cast<const f32x4*>(st + KS_OFF + (16 * i + 4 * g) * 4);
                });
                static_for<0, SCH::N_XC>([&](auto ic) {
                    constexpr int i = decltype(ic)::value;
                    if constexpr (SCH::op_of(SCH::P_XC + i) - SCH::AHEAD == op) {
                        csr[i] = *reinterpret_cast<const f32x4*>(st + CS_OFF + (16 * i + 4 * g) * 4);
                        xvr[i] = lds_read_tr4x16<false>(reinterpret_cast<const bf16_t*>(st + V_OFF), VLD / 2, 16 * i + 4 * g, 16 * half, j16);
                    }
                });
                static_for<0, SCH::NPIECES>([&](auto pcc) {
                    if constexpr (SCH::op_of(decltype(pcc)::value) == op) run_piece(pcc);
                });

                const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                if constexpr (op < OP_Q) {  // K S0
                    constexpr int sl = SCH::s_slab(op), tt = SCH::s_tile(op);
                    accv[tt] = mfma_bf16(fr[op], sb[sl], sl == 0 ? zero : accv[tt]);
                } else if constexpr (op < OP_T) {  // O^T = S0^T q^T, scaled per token by a later piece
                    constexpr int jj = op - OP_Q, sl = SCH::s_slab(jj), it = SCH::s_tile(jj);
                    acco[it] = mfma_bf16(sb[sl], fr[op], sl == 0 ? zero : acco[it]);
                } else if constexpr (op < OP_K) {  // V~ = T' X
                    constexpr int jj = op - OP_T, tt = SCH::t_tile(jj), sl = SCH::t_slab(jj);
                    vt[tt] = mfma_bf16(fr[op], xb[sl], sl == 0 ? zero : vt[tt]);
                } else if constexpr (op < OP_P) {  // S = e^{gamma_C} S + k^T (row-scaled V~)
                    constexpr int sl = SCH::k_slab(op - OP_K), t = SCH::k_tile(op - OP_K);
                    S[t] = mfma_bf16(fr[op], vbs[sl], S[t]);
                } else {  // O^T += V~^T P^T
                    constexpr int jj = op - OP_P, it = SCH::t_tile(jj), sl = SCH::t_slab(jj);
                    acco[it] = mfma_bf16(vb[sl], fr[op], acco[it]);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
#ifdef GDN_CYCLE_BUDGET
            cyc_tick(NOOUT ? 3 : 4);
#endif
            if constexpr (SAVE) {
                // V~ of this chunk: tile tt, register r holds token 16 tt + 4 g + r of this lane's column
                if constexpr (LSAVE) {
                    // after this chunk's barrier: the store wave takes it after the next one (or the last)
                    if (p.save_vnew != nullptr && save_entry(c) >= 0) {
                        if (p.save_vnew_bf16) {
                            // column 16 half + j16, tokens 16 tt + 4 g + 0..3: one 8-byte write per tile
                            uint8_t* const base = vstage_of(c) + (16 * half + j16) * VCOL + (4 * g) * 2;
#pragma unroll
                            for (int tt = 0; tt < 4; tt++) {
                                bf16x4 x;
                                x.x = (bf16_t)vt[tt][0], x.y = (bf16_t)vt[tt][1], x.z = (bf16_t)vt[tt][2], x.w = (bf16_t)vt[tt][3];
                                *reinterpret_cast<bf16x4*>(base + (16 * tt) * 2) = x;
                            }
                        } else {
                            uint8_t* const base = vstage_of(c) + (4 * g) * SROW + (16 * half + j16) * 4;
#pragma unroll
                            for (int tt = 0; tt < 4; tt++)
#pragma unroll
                                for (int r = 0; r < 4; r++) *reinterpret_cast<float*>(base + (16 * tt + r) * SROW) = vt[tt][r];
                        }
                    }
                } else if (p.save_vnew != nullptr && c % p.save_every == 0 && c / p.save_every < p.save_nc) {
                    const int entry = p.save_reverse ? save_last - c / p.save_every : c / p.save_every;
                    char* base = reinterpret_cast<char*>(p.save_vnew + ((int64_t)chain * p.save_nc + entry) * C * p.V);
                    const uint32_t lane_off = (uint32_t)((4 * g) * p.V + c0 + j16) * 4u;
                    const uint32_t row_bytes = (uint32_t)p.V * 4u;
#pragma unroll
                    for (int tt = 0; tt < 4; tt++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            *reinterpret_cast<float*>(base + (size_t)((16 * tt + r) * row_bytes) + lane_off) = vt[tt][r];
                }
            }
#ifdef GDN_CYCLE_BUDGET
            if constexpr (NOOUT) cyc_tick(1);  // 1 = staging V~ for the store wave (5 then holds the state's staging)
#endif
        }
#ifdef GDN_CYCLE_BUDGET
        // wave 0 of every 16th workgroup reports: [workgroup / 16][6 groups | chunks]
        if (p.cycle_out != nullptr && wave == 0 && lane == 0 && blockIdx.x % 16 == 0 && blockIdx.x / 16 < GDN_CYCLE_BUDGET_SLOTS) {
            uint64_t* out = p.cycle_out + (blockIdx.x / 16) * 8;
#pragma unroll
            for (int i = 0; i < 6; i++) out[i] = cyc[i];
            out[6] = (uint64_t)nchunks;
        }
#endif
        if constexpr (!NOOUT) {
            if (nchunks > 0) {
#pragma unroll
                for (int it = 0; it < 4; it++) out_tile(acco[it], (nchunks - 1) & 1, it);
            }
        }
        __syncthreads();  // the store wave writes the last output tile
        if (p.ht != nullptr) {
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) p.ht[st_off + (int64_t)st_key(t, r) * p.V] = S[t][r];
        }
        return;
    }

    // ------------------------------ compute ------------------------------
    const int tn = vgroup * NW + wave;  // 32-column tile of V owned by this wave (the launcher makes NW divide V / 32)
    // State tile td, register r: MFMA row i = 8 (r/4) + 4 h + r%4 holds state row 32 td + slice_col(i)
    // = 32 td + 16 (r/8) + 8 h + 4 ((r/4) % 2) + r%4, column 32 tn + slice_col(l32).  With the rows of a 16-block
    // in that order, the 8 reduction entries a lane half feeds per 16-row slab are 8 consecutive key columns:
    // q and k are used straight from their row-major rows.
    f32x16 S[KD];
    const int64_t st_off = ((int64_t)n * p.H + h) * K * p.V + (int64_t)(8 * lh) * p.V + 32 * tn + slice_col(l32);
    auto st_row = [](int td, int r) { return 32 * td + 16 * (r / 8) + 4 * ((r / 4) % 2) + r % 4; };
#pragma unroll
    for (int td = 0; td < KD; td++)
#pragma unroll
        for (int r = 0; r < 16; r++) S[td][r] = 0.f;
    if (p.h0 != nullptr) {
#pragma unroll
        for (int td = 0; td < KD; td++)
#pragma unroll
            for (int r = 0; r < 16; r++) S[td][r] = p.h0[st_off + (int64_t)st_row(td, r) * p.V];
    }
    // O^T tile tt, register r: token 32 tt + l32, column 32 tn + 16 (r/8) + 8 h + r%8 (slice_col order)
    bf16_t* og = p.o + b * p.o_stride_b + (seq_t0 + l32) * p.o_stride_t + (int64_t)h * p.o_stride_h + 32 * tn + 8 * lh;
    const int64_t og_step = (int64_t)C * p.o_stride_t;

    // MFMA schedule of one chunk: K S0 | q | T' X | k^T | P; the side work sits between the MFMAs at the ops
    // ScanSchedule<K> assigns.
    typedef ScanSchedule<K> SCH;
    constexpr int NOPS = SCH::NOPS, OP_Q = SCH::OP_Q, OP_T = SCH::OP_T, OP_K = SCH::OP_K, OP_P = SCH::OP_P, OP_BAR = SCH::OP_BAR;
    constexpr int LA = SCH::LA;  // LDS reads are issued this many MFMAs ahead of their use
    const int l16 = lane % 16, g16 = l32 / 16;
    auto lds_frag = [&](const uint8_t* st, auto opc) -> bf16x8 {
        constexpr int op = decltype(opc)::value;
        if constexpr (op < OP_T) {
            // rows of k (A operand of K S0) or of q (B operand of S0^T q^T): token tile tt, 16-column slab s,
            // 8 consecutive key columns per lane half
            constexpr int j = op < OP_Q ? op : op - OP_Q, s = j % KS16, tt = j / KS16;
            return *reinterpret_cast<const bf16x8*>(st + (op < OP_Q ? K_OFF : Q_OFF) + (32 * tt + l32) * QLD + (16 * s + 8 * lh) * 2);
        } else if constexpr (op >= OP_K && op < OP_P) {
            // k^T, key tile td (rows in state order), token slab s: tokens 16 s + 4 h + 0..3 and 16 s + 8 + 4 h + 0..3
            // of key column 32 td + slice_col(l32), through the transposing LDS load
            constexpr int s = SCH::k_slab(op - OP_K), td = SCH::k_tile(op - OP_K);
            const bf16_t* km = reinterpret_cast<const bf16_t*>(st + K_OFF);
            const bf16x4 a = lds_read_tr4x16<true>(km, QLD / 2, 16 * s + 4 * lh, 32 * td + 16 * g16, l16);
            const bf16x4 b = lds_read_tr4x16<true>(km, QLD / 2, 16 * s + 8 + 4 * lh, 32 * td + 16 * g16, l16);
            bf16x8 r;
#pragma unroll
            for (int e = 0; e < 4; e++) r[e] = a[e], r[4 + e] = b[e];
            return r;
        } else {
            constexpr int f = op < OP_K ? op - OP_T : 6 + (op - OP_P);  // T' | P are contiguous in the stage
            return reinterpret_cast<const bf16x8*>(st)[f * WAVE + lane];
        }
    };
    auto lds_eg = [&](const uint8_t* st) -> float { return *reinterpret_cast<const float*>(st + EG_OFF); };
    auto lds_qs = [&](const uint8_t* st, int tt) -> float { return reinterpret_cast<const float*>(st + QS_OFF)[32 * tt + l32]; };

    f32x16 accv[2], acco[2];
    bf16x8 sb[KS16], xb[4], vb[4], vbs[4], fnext[LA];  // xb: X, vb: V~, vbs: V~ with its rows scaled for the state update
    f32x4 ksr[4], csr[4];                              // row scales on their way to the pieces that use them
    bf16x4 xvr[4];                                     // and rows of v
    float egc, qsc[2];  // e^{gamma_C} and this lane's two row scales of q (tokens l32 and 32 + l32)

    __syncthreads();  // stage[0] holds chunk 0

    // what the tail of a chunk does for the next one, for chunk 0
    egc = lds_eg(stage[0]);
    qsc[0] = lds_qs(stage[0], 0), qsc[1] = lds_qs(stage[0], 1);
    static_for<0, LA>([&](auto i) { fnext[decltype(i)::value] = lds_frag(stage[0], i); });
#pragma unroll
    for (int s = 0; s < KS16; s++) sb[s] = pack8_16(S[s / 2], s % 2, 1.f);

    int valid_prev = 0;  // tokens of the previous chunk, whose output is still in acco
    for (int c = 0; c < nchunks; c++) {
        const uint8_t* st = stage[c & 1];
        const uint8_t* stn = stage[(c + 1) & 1];
        const int valid = (int)min((int64_t)C, seq_len - (int64_t)c * C);
        if constexpr (SAVE) {
            // the state this chunk starts from, for the backward pass (stores from a compute wave: this variant
            // is not the one the forward is timed on)
            // (one wave-uniform base per store plus one per-lane byte offset: 64-bit per-lane addresses for
            // all of them would not fit the register file)
            if (p.save_state != nullptr && c % p.save_every == 0 && c / p.save_every < p.save_nc) {
                const int entry = p.save_reverse ? save_last - c / p.save_every : c / p.save_every;
                char* base = reinterpret_cast<char*>(p.save_state + ((int64_t)chain * p.save_nc + entry) * K * p.V);
                const uint32_t lane_off = (uint32_t)((8 * lh) * p.V + 32 * tn + slice_col(l32)) * 4u;
                const uint32_t row_bytes = (uint32_t)p.V * 4u;
#pragma unroll
                for (int td = 0; td < KD; td++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        *reinterpret_cast<float*>(base + (size_t)(st_row(td, r) * row_bytes) + lane_off) = S[td][r];
            }
        }
        bf16x8 fr[NOPS];
#pragma unroll
        for (int i = 0; i < LA; i++) fr[i] = fnext[i];
        __builtin_amdgcn_sched_barrier(0);

        // one piece of side work (pc: index into ScanSchedule's piece list)
        auto run_piece = [&](auto pcc) {
            constexpr int pc = decltype(pcc)::value;
            if constexpr (pc >= SCH::P_XC && pc < SCH::P_XC + SCH::N_XC) {
                // X = V - diag(cs) (K S0), registers 4 q4 .. 4 q4 + 3 of tile tt: tokens 32 tt + 8 q4 + 4 h + 0..3 of
                // this lane's column; the second piece of a half tile also packs it as an operand of T' X
                constexpr int i = pc - SCH::P_XC, tt = i / 4, q4 = i % 4;
#pragma unroll
                for (int e = 0; e < 4; e++) accv[tt][4 * q4 + e] = (float)xvr[i % 4][e] - csr[i % 4][e] * accv[tt][4 * q4 + e];
            } else if constexpr (pc >= SCH::P_XB) {
                constexpr int i = pc - SCH::P_XB;  // X as operand of T' X
                xb[i] = pack8_16(accv[i / 2], i % 2, 1.f);
            } else if constexpr (pc >= SCH::P_OUT && pc < SCH::P_OUT + SCH::N_OUT) {
                // output tile tt of the previous chunk, registers 8 half .. 8 half + 7
                constexpr int i = pc - SCH::P_OUT, tt = i / 2, half = i % 2;
                if (OS) {
                    if (c > 0)
                        *reinterpret_cast<bf16x8*>(ostage_at(wave, (c - 1) & 1, 32 * tt + l32, 2 * half + lh)) =
                            pack8_16(acco[tt], half, 1.f);
                } else if (32 * tt + l32 < valid_prev) {
                    *reinterpret_cast<bf16x8*>(og - og_step + (int64_t)(32 * tt) * p.o_stride_t + 16 * half) =
                        pack8_16(acco[tt], half, 1.f);
                }
            } else if constexpr (pc >= SCH::P_AS && pc < SCH::P_AS + SCH::N_AS) {
                // O^T = (q S0)^T so far: its columns (tokens) take the row scale of q before the P terms are added
                constexpr int i = pc - SCH::P_AS, tt = i / 4, q4 = i % 4;
#pragma unroll
                for (int e = 0; e < 4; e++) acco[tt][4 * q4 + e] *= qsc[tt];
            } else if constexpr (pc >= SCH::P_DEC && pc < SCH::P_DEC + SCH::N_DEC) {
                // decay of the state (its bf16 copy for this chunk is already in sb)
                constexpr int i = pc - SCH::P_DEC, td = i / 4, q4 = i % 4;
#pragma unroll
                for (int e = 0; e < 4; e++) S[td][4 * q4 + e] *= egc;
            } else if constexpr (pc >= SCH::P_VS && pc < SCH::P_VS + SCH::N_VS) {
                // V~ as operand of k^T V~: each row (token) scaled by e^{gamma_C - gamma} / |k|; half a fragment
                constexpr int i = pc - SCH::P_VS, x = i / 2, sub = i % 2, tt = x / 2, half = x % 2;
#pragma unroll
                for (int e = 0; e < 4; e++) vbs[x][4 * sub + e] = (bf16_t)(accv[tt][8 * half + 4 * sub + e] * ksr[i % 4][e]);
            } else if constexpr (pc >= SCH::P_VB && pc < SCH::P_VB + SCH::N_VB) {
                constexpr int i = pc - SCH::P_VB;  // V~ as operand of P V~
                vb[i] = pack8_16(accv[i / 2], i % 2, 1.f);
            } else {
                // the new state tile as operand of the next chunk; pinned here, or the compiler moves all of them
                // behind the last MFMA of the loop
                constexpr int i = pc - SCH::P_SB;
                sb[i] = pack8_16(S[i / 2], i % 2, 1.f);
                pin_regs(sb[i]);
            }
        };

        static_for<0, NOPS>([&](auto opc) {
            constexpr int op = decltype(opc)::value;
            // ---- operand reads: this chunk until the barrier, the next one after it ----
            if constexpr (op + LA < NOPS) fr[op + LA] = lds_frag(st, std::integral_constant<int, (op + LA < NOPS ? op + LA : 0)>{});
            if constexpr (op == OP_BAR) {
                __syncthreads();  // this wave is done with chunk c's half; chunk c + 1 is in the other one
                egc = lds_eg(stn);
                qsc[0] = lds_qs(stn, 0), qsc[1] = lds_qs(stn, 1);  // this chunk's scales were applied before the barrier
            }
            if constexpr (op >= OP_BAR) fnext[op >= OP_BAR ? op - OP_BAR : 0] = lds_frag(stn, std::integral_constant<int, (op >= OP_BAR ? op - OP_BAR : 0)>{});
            // row scales and rows of v, a few ops ahead of the piece that uses them
            static_for<0, SCH::N_VS>([&](auto ic) {
                constexpr int i = decltype(ic)::value, x = i / 2, sub = i % 2;
                if constexpr (SCH::op_of(SCH::P_VS + i) - SCH::AHEAD == op)
                    ksr[i % 4] = *reinterpret_cast<const f32x4*>(st + KS_OFF + (16 * x + 8 * sub + 4 * lh) * 4);
            });
            static_for<0, SCH::N_XC>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                if constexpr (SCH::op_of(SCH::P_XC + i) - SCH::AHEAD == op) {
                    csr[i % 4] = *reinterpret_cast<const f32x4*>(st + CS_OFF + (8 * i + 4 * lh) * 4);
                    xvr[i % 4] = lds_read_tr4x16<true>(reinterpret_cast<const bf16_t*>(st + V_OFF), VLD / 2, 8 * i + 4 * lh, 32 * wave + 16 * g16, l16);
                }
            });

            // ---- side work ----
            static_for<0, SCH::NPIECES>([&](auto pcc) {
                if constexpr (SCH::op_of(decltype(pcc)::value) == op) run_piece(pcc);
            });

            // ---- the MFMA ----
            if constexpr (op < OP_Q) {  // K S0, fragment (tt, s): rows = tokens
                constexpr int s = op % KS16, tt = op / KS16;
                if constexpr (s == 0) {
                    f32x16 zero;
#pragma unroll
                    for (int r = 0; r < 16; r++) zero[r] = 0.f;
                    accv[tt] = mfma32_bf16(fr[op], sb[s], zero);
                } else {
                    accv[tt] = mfma32_bf16(fr[op], sb[s], accv[tt]);
                }
            } else if constexpr (op < OP_T) {  // O^T = (q S0)^T, scaled per token by a later piece
                constexpr int j = op - OP_Q, s = j % KS16, tt = j / KS16;
                if constexpr (s == 0) {
                    f32x16 zero;
#pragma unroll
                    for (int r = 0; r < 16; r++) zero[r] = 0.f;
                    acco[tt] = mfma32_bf16(sb[s], fr[op], zero);
                } else {
                    acco[tt] = mfma32_bf16(sb[s], fr[op], acco[tt]);
                }
            } else if constexpr (op < OP_K) {  // V~ = T' X: tile 0 from X tile 0, tile 1 from both
                constexpr int j = op - OP_T, tt = SCH::t_tile(j), s = SCH::t_slab(j);
                if constexpr (s == 0) {
                    f32x16 zero;
#pragma unroll
                    for (int r = 0; r < 16; r++) zero[r] = 0.f;
                    accv[tt] = mfma32_bf16(fr[op], xb[s], zero);
                } else {
                    accv[tt] = mfma32_bf16(fr[op], xb[s], accv[tt]);
                }
            } else if constexpr (op < OP_P) {  // S = e^{gamma_C} S + k^T (row-scaled V~), fragment (td, s)
                constexpr int s = SCH::k_slab(op - OP_K), td = SCH::k_tile(op - OP_K);
                S[td] = mfma32_bf16(fr[op], vbs[s], S[td]);
            } else {  // O^T += V~^T P^T; P[i < 32][j >= 32] = 0 is skipped
                constexpr int j = op - OP_P;
                constexpr int tt = j < 2 ? 0 : 1, s = j < 2 ? j : j - 2;
                acco[tt] = mfma32_bf16(vb[s], fr[op], acco[tt]);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (SAVE) {
            // V~ of this chunk: tile tt, register r holds token 32 tt + 8 (r/4) + 4 h + r%4 of this lane's column
            if (p.save_vnew != nullptr && c % p.save_every == 0 && c / p.save_every < p.save_nc) {
                const int entry = p.save_reverse ? save_last - c / p.save_every : c / p.save_every;
                char* base = reinterpret_cast<char*>(p.save_vnew + ((int64_t)chain * p.save_nc + entry) * C * p.V);
                const uint32_t lane_off = (uint32_t)((4 * lh) * p.V + 32 * tn + slice_col(l32)) * 4u;
                const uint32_t row_bytes = (uint32_t)p.V * 4u;
#pragma unroll
                for (int tt = 0; tt < 2; tt++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        *reinterpret_cast<float*>(base + (size_t)((32 * tt + 8 * (r / 4) + r % 4) * row_bytes) + lane_off) = accv[tt][r];
            }
        }
        valid_prev = valid;
        og += og_step;
    }

    // the output of the last chunk
#pragma unroll
    for (int tt = 0; tt < 2; tt++)
#pragma unroll
        for (int half = 0; half < 2; half++) {
            if (OS) {
                if (nchunks > 0)
                    *reinterpret_cast<bf16x8*>(ostage_at(wave, (nchunks - 1) & 1, 32 * tt + l32, 2 * half + lh)) =
                        pack8_16(acco[tt], half, 1.f);
            } else if (32 * tt + l32 < valid_prev) {
                *reinterpret_cast<bf16x8*>(og - og_step + (int64_t)(32 * tt) * p.o_stride_t + 16 * half) =
                    pack8_16(acco[tt], half, 1.f);
            }
        }
    if (OS) __syncthreads();

    if (p.ht != nullptr) {
#pragma unroll
        for (int td = 0; td < KD; td++)
#pragma unroll
            for (int r = 0; r < 16; r++) p.ht[st_off + (int64_t)st_row(td, r) * p.V] = S[td][r];
    }
}

// ------------------------------------------------------------------------------------------
// launch
// ------------------------------------------------------------------------------------------
int launch_chunk_fused(ChunkParams& p, int K, hipStream_t stream, int num_cus);  // gdn_chunk_fused.hip

// Which scan kernel a launch gets: compute waves (32-column slices) per workgroup, and whether a slice is split over
// two half-slice waves.
ScanPlan plan_scan(int K, int64_t chains, int V, bool packed, bool save, int records_given, int num_cus, const SaveRequest& req) {
    // Slices per scan workgroup: one while that gives no more workgroups than CUs, so that every slice has a CU's load
    // bandwidth to itself; otherwise 2 or 4 slices of a chain share the records through one workgroup's LDS (they must
    // divide the V / 32 tiles).
    const int vtiles = V / 32;
    int nw = 1;
    while (nw < 4 && vtiles % (2 * nw) == 0 && chains * (vtiles / nw) > (int64_t)num_cus) nw *= 2;
    // Packed batches are ragged as a rule, and their chains start longest first (chunk_offsets_kernel): the launch then
    // takes as long as the longest chain, which runs faster the fewer slices share its workgroup, while the workgroups
    // that do not fit at first fill in behind the short chains.  So up to two workgroups per CU are accepted there.
    // (Configuration 2, 11 sequences of 202 .. 6350 tokens, H = 16: 246 us with four slices per workgroup, 193 us with two.)
    if (packed && !save && nw > 1 && chains * (vtiles / (nw / 2)) <= 2 * (int64_t)num_cus) nw /= 2;
    if (save && nw == 2) nw = 1;  // the saving variant exists for 1 and 4 slices per workgroup
    // The saving scan of a packed batch (the backward's forward sweep): started longest first as well, its half-slice
    // variant, whose saves go through LDS (and may be bf16, which the chunk-local backward kernel reads at half the
    // traffic), finishes a ragged batch sooner than four slices per workgroup storing from their compute waves
    // (configuration 2, 2.75 workgroups per CU: 352 us against 575 us; the whole backward of 131072 ragged tokens, 7.5
    // workgroups per CU: 6.3 against 7.4 ms).
    if (save && packed && !records_given && K <= 128) nw = 1;
    if (K > 128) nw = 1;  // K = 256 has the half-slice scan only, also as the saving variant and on given records
    if (records_given == 2) nw = 1;  // records given in the half-slice scan's fragment order
    ScanPlan plan;
    plan.nw = nw;
    // a slice with a CU to itself is scanned by two waves of 16 columns each; the records are laid out for them
    plan.half = K > 128 || records_given == 2 || (nw == 1 && !records_given);
    // Saves go through LDS and the store wave in the half-slice scan: always at K <= 128; at K = 256 only in the scan
    // without output (no rows of q in LDS), with bf16 V~, and fp32 states at every second chunk at most (one buffer).
    plan.staged_saves = save && plan.half &&
                        (K <= 128 || (req.no_output && (!req.has_vnew || req.vnew_bf16) && (!req.has_state || req.state_bf16 || req.save_every >= 2)));
    plan.no_output = plan.staged_saves && req.no_output && K >= 128;
    return plan;
}

template <int K>
static int launch32(ChunkParams& p, hipStream_t stream, hipEvent_t* events, int num_cus) {
    const int64_t items = (int64_t)((p.TC + 7) / 8) * 8 * p.H;  // a multiple of 8, see the kernel
    const int64_t cap = (int64_t)(3 * num_cus + 7) / 8 * 8;      // three workgroups per CU (LDS and registers allow it)
    if (items >= ((int64_t)1 << 31)) return GDN_ERR_UNSUPPORTED;  // the kernel counts items in 32 bits
    const int grid_prep = (int)(items < cap ? items : cap);
    p.rec16 = 0;
    if (p.fused) {  // prepare and scan in one launch, when the shape qualifies
        if (events != nullptr) (void)hipEventRecord(events[2], stream);
        const int rc = launch_chunk_fused(p, K, stream, num_cus);
        if (rc != GDN_ERR_UNSUPPORTED) return rc;
    }
    const int64_t chains = (int64_t)p.N * p.H;
    const int64_t chains8 = (chains + 7) / 8 * 8;
    const int vtiles = p.V / 32;
    const bool save = p.save_state != nullptr || p.save_vnew != nullptr;
    SaveRequest req;
    req.no_output = p.no_output != 0, req.has_state = p.save_state != nullptr, req.has_vnew = p.save_vnew != nullptr;
    req.state_bf16 = p.save_state_bf16 != 0, req.vnew_bf16 = p.save_vnew_bf16 != 0, req.save_every = p.save_every;
    const ScanPlan plan = plan_scan(K, chains, p.V, p.cu_seqlens != nullptr, save, p.records_given, num_cus, req);
    const int nw = plan.nw;
    const bool half = plan.half;
    if ((p.save_state_bf16 || p.save_vnew_bf16) && !plan.staged_saves) return GDN_ERR_UNSUPPORTED;  // (the C entry asks plan_scan first)
    p.rec16 = half ? 1 : 0;
    if (!p.records_given) {
        hipLaunchKernelGGL((chunk_prepare32_kernel<K>), dim3(grid_prep), dim3(PREP_THREADS), 0, stream, p);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
    }
    if (events != nullptr) (void)hipEventRecord(events[2], stream);
    p.scan_groups = vtiles / nw;
    const dim3 grid((unsigned)(chains8 * p.scan_groups));
    if constexpr (K > 128) {
        if (save && plan.no_output) hipLaunchKernelGGL((chunk_scan32_kernel<K, 1, false, true, true, true>), grid, dim3(scan_waves(1, true) * WAVE), 0, stream, p);
        else if (save) hipLaunchKernelGGL((chunk_scan32_kernel<K, 1, false, true, true>), grid, dim3(scan_waves(1, true) * WAVE), 0, stream, p);
        else hipLaunchKernelGGL((chunk_scan32_kernel<K, 1, false, false, true>), grid, dim3(scan_waves(1, true) * WAVE), 0, stream, p);
        return (int)hipGetLastError();
    } else {
    if (save) {
        if (nw == 4) hipLaunchKernelGGL((chunk_scan32_kernel<K, 4, false, true>), grid, dim3(scan_waves(4) * WAVE), 0, stream, p);
        else if (half && plan.no_output && K == 128) hipLaunchKernelGGL((chunk_scan32_kernel<128, 1, false, true, true, true>), grid, dim3(scan_waves(1, true) * WAVE), 0, stream, p);
        else if (half) hipLaunchKernelGGL((chunk_scan32_kernel<K, 1, false, true, true>), grid, dim3(scan_waves(1, true) * WAVE), 0, stream, p);
        else hipLaunchKernelGGL((chunk_scan32_kernel<K, 1, false, true>), grid, dim3(scan_waves(1) * WAVE), 0, stream, p);
        return (int)hipGetLastError();
    }
    if (nw == 4 && p.scan_groups == 1) hipLaunchKernelGGL((chunk_scan32_kernel<K, 4, true>), grid, dim3(scan_waves(4) * WAVE), 0, stream, p);
    else if (nw == 4) hipLaunchKernelGGL((chunk_scan32_kernel<K, 4>), grid, dim3(scan_waves(4) * WAVE), 0, stream, p);
    else if (nw == 2) hipLaunchKernelGGL((chunk_scan32_kernel<K, 2>), grid, dim3(scan_waves(2) * WAVE), 0, stream, p);
    else if (half) hipLaunchKernelGGL((chunk_scan32_kernel<K, 1, false, false, true>), grid, dim3(scan_waves(1, true) * WAVE), 0, stream, p);
    else hipLaunchKernelGGL((chunk_scan32_kernel<K, 1>), grid, dim3(scan_waves(1) * WAVE), 0, stream, p);
    return (int)hipGetLastError();
    }
}

int launch_chunk32(ChunkParams& p, int K, hipStream_t stream, hipEvent_t* events, int num_cus) {
    if (K == 64) return launch32<64>(p, stream, events, num_cus);
    if (K == 128) return launch32<128>(p, stream, events, num_cus);
    if (K == 256) return launch32<256>(p, stream, events, num_cus);
    return GDN_ERR_UNSUPPORTED;
}

}  // namespace gdn

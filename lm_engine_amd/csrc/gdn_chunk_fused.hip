// The chunked forward as ONE launch (K <= 128, fixed-length batches whose scan fills about half of the CUs):
// producer workgroups run the prepare step and scan workgroups consume its records as they appear.
//
// Scan workgroups.  gdn_chunk32.hip's scan gives one wave a whole 32-column slice of the state, and a slice a CU.
// Here a workgroup holds two slices of a chain (64 columns: whole 128-byte lines of the output) and each slice is
// shared by a PAIR of compute waves on two SIMDs, so the scan of a batch needs half as many CUs and leaves the
// others to the producers.  Wave tt (0 or 1) of a pair owns
//   * token tile tt (tokens 32 tt .. 32 tt + 31 of the chunk) in every product whose rows are tokens:
//     K S0, X, V~ = T' X, and the output O = diag(qs) Q S0 + P V~;
//   * key half tt (state rows K/2 tt .. K/2 tt + K/2 - 1) of the state, as MFMA accumulators, in the update
//     S = e^{gamma_C} S + K^T diag(ks) V~.
// So each product is split by its OUTPUT rows: no partial sums are ever added across waves, every
// accumulator keeps the register layout of gdn_chunk32.hip (so an accumulator tile still turns into the
// next MFMA's operand without leaving registers), and what a wave lacks are operands only, all bf16:
//   1. the partner's half of S0 as B / A operand of K S0 and (Q S0)^T      (K/32 fragments each way)
//   2. X of token tile 0, which V~ of token tile 1 needs (T' is lower triangular: one way, 2 fragments)
//   3. the partner's tile of V~: row-scaled for the state update (2 fragments each way), plain for
//      P V~ of token tile 1 (2 fragments, one way)
// They go through three small LDS buffers per slice.  A wave publishes what it wrote by storing a running
// epoch number to an LDS word of its own; the partner polls that word.  (LDS operations of a wave execute
// in order, so whoever reads the new epoch reads the data written before it.)  Each wave starts on the
// half of a product that needs only its own operand and picks the partner's up when it gets there, which
// hides part of the hand-over.  Per chunk and wave (K = 128): 28 (tile 0) or 32 (tile 1) MFMAs.
// The exchange buffers overlap: a wave's tile of V~ is written over the partner's half of S0, which that
// wave alone reads and has finished with by then; the partner overwrites it with its next half of S0 only
// after it has read V~ from it.
// Loaders (4 waves) and the LDS double buffer are those of gdn_chunk32.hip; the loaders also write the output
// (a compute wave leaves its bf16 output tile in LDS at the start of the next chunk).  One workgroup barrier
// per chunk hands the stage halves over.  Waves of a scan workgroup with two slices: 0..3 compute (pairs 0-1,
// 2-3), 4..7 loaders.  (With one slice: 0 1 compute | 2 3 6 7 loaders | 4 output store | 5 exits at once.)
//
// What a wave pays, measured with one wave alone on a SIMD: 4.5 cycles per VALU instruction, 32 per MFMA (hidden
// behind up to ~7 independent VALU instructions), ~17 per ds_read_b128, ~29 per ds_write_b128, ~120 for an LDS write
// followed by a read of it.  The operand fragments (one ds_read_b128 per MFMA) and the bf16 conversions therefore
// cost a compute wave more than its MFMAs, in this scan as in the one-wave scan, and the hand-overs between the
// waves of a pair (~300 cycles each, three per chunk) eat what the second SIMD brings: a pair runs a slice in
// ~2750 cycles per chunk, the single wave in ~2850.

#include "gdn_chunk32_common.h"
#include "gdn_chunk_prepare32.h"
#include "gdn_launch.h"

namespace gdn {

constexpr int PAIR_THREADS = 8 * WAVE;
constexpr int PAIR_LOADERS = 4;

// Epochs: a wave stores 3 c + 1 once its half of the state chunk c starts from is in LDS, 3 c + 2 (wave 0
// only) after X of token tile 0, 3 c + 3 after its tile of V~ (pair_publish / pair_wait).

#define PIN() __builtin_amdgcn_sched_barrier(0)

// Fixes the place of the MFMA that produced `acc`: an empty asm statement is ordered with the PIN()s around it, the
// pure MFMA intrinsic is not and would be placed wherever its result is first needed.
__device__ __forceinline__ void pin_acc(f32x16& acc) { asm volatile("" : "+v"(acc)); }

// LDS bytes of a scan workgroup: two stage halves, exchange buffers and output staging per slice, the flags
template <int K, int NS>
constexpr int scan_pair_lds_bytes() {
    constexpr int STAGE = 12 * FRAG_BYTES + C * (64 * NS + 16) + 2 * C * (2 * K + 16) + 3 * C * 4 + 16;
    constexpr int XF = K / 32 > 4 ? K / 32 : 4;
    return 2 * STAGE + NS * ((2 * XF + 2) * FRAG_BYTES + 2 * C * 64) + 64;
}

// WAIT: the records are written by prepare workgroups of the same launch; a loader asks p.ready before it loads one.
// `id` numbers the scan workgroups.
template <int K, int NS, bool WAIT>
__device__ __forceinline__ void scan_pair_body(const ChunkParams& p, uint8_t* lds, const int id) {
    constexpr int NL = PAIR_LOADERS;
    constexpr int NB = 2;       // register buffers of a loader wave: chunks in flight
    constexpr int KD = K / 32;    // 32-row tiles of the state
    constexpr int KS16 = K / 16;  // 16-wide slabs over the key dim
    constexpr int KDH = KD / 2;   // state tiles per wave
    constexpr int SH = KS16 / 2;  // key slabs per wave
    static_assert(KD % 2 == 0, "the key dim splits into two halves of whole tiles");
    // One half of the stage, as in chunk_scan32_kernel: [T diag(beta) 6 | P 6] | the chunk's 64 rows of this
    // workgroup's columns of v | of q | of k | 64 row scales of q | of k for the state update | of k S0 | e^{gamma_C}
    constexpr int SHARED_FRAGS = 12;
    constexpr int SHARED_BYTES = SHARED_FRAGS * FRAG_BYTES;
    constexpr int VROW = 64 * NS;
    constexpr int VLD = VROW + 16;
    constexpr int V_UNITS = C * VROW / FRAG_BYTES;
    constexpr int QLD = 2 * K + 16;
    constexpr int Q_UNITS = C * 2 * K / FRAG_BYTES;
    constexpr int V_OFF = SHARED_BYTES;
    constexpr int Q_OFF = V_OFF + C * VLD;
    constexpr int K_OFF = Q_OFF + C * QLD;
    constexpr int QS_OFF = K_OFF + C * QLD;
    constexpr int KS_OFF = QS_OFF + C * 4;
    constexpr int CS_OFF = KS_OFF + C * 4;
    constexpr int EG_OFF = CS_OFF + C * 4;
    constexpr int STAGE_BYTES = EG_OFF + 16;
    constexpr int NF = SHARED_FRAGS / NL;
    constexpr int NV = V_UNITS / NL;
    constexpr int NQ = 2 * Q_UNITS / NL;
    constexpr int NLOAD = NF + NV + NQ;
    static_assert(SHARED_FRAGS % NL == 0 && V_UNITS % NL == 0 && (2 * Q_UNITS) % NL == 0, "the pieces must divide over the loader waves");
    // exchange buffers of a slice: [half 0 of S0 | half 1 of S0] (V~ of tile tt goes over half 1 - tt) | X of tile 0
    constexpr int XF = SH > 4 ? SH : 4;  // fragments per half: SH of the state, or 2 scaled + 2 plain of V~
    constexpr int XBYTES = (2 * XF + 2) * FRAG_BYTES;
    constexpr int OBYTES = 2 * C * 64;  // output staging of a slice: [chunk parity][64 tokens][64 bytes]
    static_assert(2 * STAGE_BYTES + NS * (XBYTES + OBYTES) + 64 <= 160 * 1024, "stage exceeds LDS");

    static_assert(2 * STAGE_BYTES + NS * (XBYTES + OBYTES) + 64 == scan_pair_lds_bytes<K, NS>(), "LDS layout and its size disagree");
    uint8_t (*const stage)[STAGE_BYTES] = reinterpret_cast<uint8_t (*)[STAGE_BYTES]>(lds);
    uint8_t (*const xbuf)[XBYTES] = reinterpret_cast<uint8_t (*)[XBYTES]>(lds + 2 * STAGE_BYTES);
    uint8_t (*const ostage)[OBYTES] = reinterpret_cast<uint8_t (*)[OBYTES]>(lds + 2 * STAGE_BYTES + NS * XBYTES);
    int (*const flags)[2] = reinterpret_cast<int (*)[2]>(lds + 2 * STAGE_BYTES + NS * (XBYTES + OBYTES));
    // set by a loader whose wait for a record ran out: from then on this workgroup writes no output
    volatile int* const wg_failed = reinterpret_cast<volatile int*>(lds + 2 * STAGE_BYTES + NS * (XBYTES + OBYTES) + 48);

    const int lane = threadIdx.x % WAVE;
    const int wave = threadIdx.x / WAVE;
    const int l32 = lane % 32, lh = lane / 32;

    // workgroup -> (sequence-head chain, column group); the groups of a chain stay on one XCD (id % 8)
    const int xcd = id % 8, rest = id / 8;
    const int vgroup = rest % p.scan_groups;
    const int per_xcd = (p.N * p.H + 7) / 8;
    const int chain = xcd * per_xcd + rest / p.scan_groups;
    if (rest / p.scan_groups >= per_xcd || chain >= p.N * p.H) return;  // whole workgroup
    const int n = chain / p.H, h = chain % p.H;

    int slot_begin, slot_end;
    int64_t b, seq_t0, seq_len;
    if (p.cu_seqlens == nullptr) {
        seq_len = p.pad_lens == nullptr ? p.T : min(max(p.pad_lens[n + 1] - p.pad_lens[n], 0), p.T);
        slot_begin = n * p.NT, slot_end = slot_begin + (int)((seq_len + C - 1) / C);
        b = n, seq_t0 = p.T - seq_len;
    } else {
        slot_begin = p.chunk_off[n], slot_end = p.chunk_off[n + 1];
        int t0, len;
        packed_bounds(p.cu_seqlens, n, p.T, t0, len);
        b = 0, seq_t0 = t0, seq_len = min(len, (slot_end - slot_begin) * C);
    }
    const int nchunks = slot_end - slot_begin;
    const uint8_t* rec = p.rec + ((int64_t)h * p.TC + slot_begin) * p.rec_bytes;

    if (threadIdx.x < NS * 2) flags[threadIdx.x / 2][threadIdx.x % 2] = 0;
    if (threadIdx.x == WAVE - 1) *wg_failed = 0;

    // output staging: the four 16-byte pieces of a row XOR-swizzled with (row / 4) % 4 (conflict-free on both sides)
    auto ostage_at = [&](int sl, int parity, int row, int piece) -> uint8_t* {
        return ostage[sl] + (parity * C + row) * 64 + ((piece ^ ((row >> 2) & 3)) << 4);
    };

    // With one slice a separate wave writes the output: a store in a loader wave sits in the same in-order
    // memory counter as its loads, and every wait for a load then also waits for the store's acknowledgement
    // (measured: the loaders alone 59 us for configuration 1 without the stores, 93 us with them).
    constexpr bool STORE_WAVE = NS == 1;
    const bool is_compute = wave < 2 * NS;
    const bool is_loader = NS == 2 ? (wave >= 4 && wave < 8) : (wave == 2 || wave == 3 || wave == 6 || wave == 7);
    const bool is_store = STORE_WAVE && wave == (NS == 2 ? 8 : 4);
    if (!is_compute && !is_loader && !is_store) return;
    __syncthreads();  // the flags are zero

    if (is_store) {
        // ------------------------------ output store ------------------------------
        const int row0 = lane / 4, piece = lane % 4;
        bf16_t* const og = p.o + b * p.o_stride_b + (seq_t0 + row0) * p.o_stride_t + (int64_t)h * p.o_stride_h +
                           32 * (vgroup * NS) + 8 * piece;
        auto flush = [&](int c) {
            if (WAIT && *wg_failed != 0) return;
            const int valid = (int)min((int64_t)C, seq_len - (int64_t)c * C);
#pragma unroll
            for (int sl = 0; sl < NS; sl++) {
                bf16x8 rows[4];
#pragma unroll
                for (int i = 0; i < 4; i++) rows[i] = *reinterpret_cast<const bf16x8*>(ostage_at(sl, c & 1, row0 + 16 * i, piece));
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (row0 + 16 * i < valid) {
                        __builtin_nontemporal_store(rows[i], reinterpret_cast<bf16x8*>(og + ((int64_t)c * C + 16 * i) * p.o_stride_t + 32 * sl));
                    }
            }
        };
        __syncthreads();  // stage[0] holds chunk 0
        for (int c = 0; c < nchunks; c++) {
            __syncthreads();  // barrier c: the output of chunk c - 1 is in the staging
            if (c > 0) flush(c - 1);
        }
        __syncthreads();
        if (nchunks > 0) flush(nchunks - 1);
        return;
    }

    if (is_loader) {
        // ------------------------------ loader ------------------------------
        const int lw = __builtin_amdgcn_readfirstlane(NS == 2 ? wave - 4 : (wave < 4 ? wave - 2 : wave - 4));
        const int rot_f = vgroup % NF;
        const int rot_q = vgroup % NQ;
        auto frag_of = [&](int i) { return lw * NF + (i + rot_f < NF ? i + rot_f : i + rot_f - NF); };
        auto vunit_of = [&](int i) { return lw * NV + i; };
        auto qunit_of = [&](int i) { return lw * NQ + (i + rot_q < NQ ? i + rot_q : i + rot_q - NQ); };
        constexpr int Q_ROWS = C / Q_UNITS, Q_PIECES = WAVE / Q_ROWS;
        constexpr int V_ROWS = C / V_UNITS, V_PIECES = WAVE / V_ROWS;
        const int q_row = lane / Q_PIECES, q_piece = lane % Q_PIECES;
        const int v_row = lane / V_PIECES, v_piece = lane % V_PIECES;
        const int hqk = qk_head_of(h, p.qk_div);
        const bf16_t* const qg = p.q + b * p.q_stride_b + seq_t0 * p.q_stride_t + (int64_t)hqk * p.q_stride_h + q_piece * 8;
        const bf16_t* const kg = p.k + b * p.k_stride_b + seq_t0 * p.k_stride_t + (int64_t)hqk * p.k_stride_h + q_piece * 8;
        const bf16_t* const vg = p.v + b * p.v_stride_b + seq_t0 * p.v_stride_t + (int64_t)h * p.v_stride_h + 32 * (vgroup * NS) + v_piece * 8;
        bf16x8 buf[NB][NLOAD];
        struct Scalars {
            float qs, ks, cs, eg;
        };
        Scalars sc[NB] = {};
        auto src_of = [&](int c, int i) -> const uint8_t* {
            if (i < NF) return rec + ((int64_t)c * p.rec_bytes + (int64_t)frag_of(i) * FRAG_BYTES) + lane * 16;
            if (i < NF + NV) {  // a row past the end of the sequence is read from the last token instead: never used
                const int tok = min(c * C + vunit_of(i - NF) * V_ROWS + v_row, (int)seq_len - 1);
                return reinterpret_cast<const uint8_t*>(vg + (int64_t)tok * p.v_stride_t);
            }
            const int u = qunit_of(i - NF - NV);
            const bool is_k = u >= Q_UNITS;
            const int tok = min(c * C + (is_k ? u - Q_UNITS : u) * Q_ROWS + q_row, (int)seq_len - 1);
            return reinterpret_cast<const uint8_t*>((is_k ? kg : qg) + (int64_t)tok * (is_k ? p.k_stride_t : p.q_stride_t));
        };
        auto dst_of = [&](uint8_t* st, int i) -> uint8_t* {
            if (i < NF) return st + frag_of(i) * FRAG_BYTES + lane * 16;
            if (i < NF + NV) return st + V_OFF + (vunit_of(i - NF) * V_ROWS + v_row) * VLD + v_piece * 16;
            return st + Q_OFF + (qunit_of(i - NF - NV) * Q_ROWS + q_row) * QLD + q_piece * 16;
        };
        auto load_scalars = [&](Scalars& sc, int c) {
            const uint8_t* r = rec + (int64_t)c * p.rec_bytes;
            sc.qs = reinterpret_cast<const float*>(r + p.off_qs)[lane];
            sc.ks = reinterpret_cast<const float*>(r + p.off_ks)[lane];
            sc.cs = reinterpret_cast<const float*>(r + p.off_cs)[lane];
            sc.eg = *reinterpret_cast<const float*>(r + p.off_eg);
        };
        auto fetch = [&](const uint8_t* src) -> bf16x8 { return *reinterpret_cast<const bf16x8*>(src); };
        auto load = [&](bf16x8(&buf)[NLOAD], Scalars& sc, int c) {
#pragma unroll
            for (int i = 0; i < NLOAD; i++) buf[i] = fetch(src_of(c, i));
            load_scalars(sc, c);
        };
        auto store_and_reload = [&](bf16x8(&buf)[NLOAD], Scalars& sc, int c, int c2, auto reload_tag) {
            constexpr bool reload = decltype(reload_tag)::value;
            uint8_t* dst = stage[c & 1];
            reinterpret_cast<float*>(dst + QS_OFF)[lane] = sc.qs;
            reinterpret_cast<float*>(dst + KS_OFF)[lane] = sc.ks;
            reinterpret_cast<float*>(dst + CS_OFF)[lane] = sc.cs;
            if (lane == 0) *reinterpret_cast<float*>(dst + EG_OFF) = sc.eg;
#pragma unroll
            for (int i = 0; i < NLOAD; i++) {
                *reinterpret_cast<bf16x8*>(dst_of(dst, i)) = buf[i];
                if constexpr (reload) buf[i] = fetch(src_of(c2, i));
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (reload) load_scalars(sc, c2);
        };
        bool failed = false;  // this wave's wait ran out (the four loaders poll the same flags, each for itself)
        // output of chunk c: this loader writes tokens 16 lw .. 16 lw + 15 of every slice, 64 bytes per row
        const int o_row = 16 * lw + lane / 4, o_piece = lane % 4;
        bf16_t* const og = p.o + b * p.o_stride_b + (seq_t0 + o_row) * p.o_stride_t + (int64_t)h * p.o_stride_h +
                           32 * (vgroup * NS) + 8 * o_piece;
        auto flush = [&](int c) {
            if constexpr (STORE_WAVE) return;
            if (WAIT && failed) return;
            const int valid = (int)min((int64_t)C, seq_len - (int64_t)c * C);
            bf16x8 rows[NS];
#pragma unroll
            for (int sl = 0; sl < NS; sl++) rows[sl] = *reinterpret_cast<const bf16x8*>(ostage_at(sl, c & 1, o_row, o_piece));
            if (o_row < valid) {
#pragma unroll
                for (int sl = 0; sl < NS; sl++) __builtin_nontemporal_store(rows[sl], reinterpret_cast<bf16x8*>(og + (int64_t)c * C * p.o_stride_t + 32 * sl));
            }
        };
        // Records written in this very launch: chunks below ready_upto are known to be complete.  One poll reads the
        // flags of the next 64 chunks, one per lane, with loads that bypass the caches; it also waits for every load
        // this wave has in flight (they return in order), so polls should be rare: prepare normally runs well ahead.
        int ready_upto = WAIT ? 0 : nchunks;
        auto ensure_ready = [&](int c) {
            if constexpr (WAIT) {
                if (c < ready_upto || c >= nchunks) return;
                const int32_t* flag = p.ready + (int64_t)h * p.TC + slot_begin + c;
                for (uint32_t spin = 0;; spin++) {
                    const int32_t got = c + lane < nchunks ? __hip_atomic_load(flag + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 1;
                    const uint64_t pending = __ballot(got == 0);
                    const int n = pending == 0 ? 64 : __builtin_ctzll(pending);
                    if (n > 0) {
                        ready_upto = c + n;
                        break;
                    }
                    if (spin >= p.spin_limit) {
                        // Bounded, so that a launch whose prepare half is missing or stuck still ends.  The record is NOT
                        // there: latch the error where the host finds it (gdn_chunk_fwd_status, gdn_args::error_word),
                        // stop this workgroup's output, and stop polling (the remaining chunks run on whatever the
                        // workspace holds; every address stays inside it).
                        if (lane == 0) {
                            __hip_atomic_store(p.err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            if (p.err_caller != nullptr) __hip_atomic_store(p.err_caller, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                            *wg_failed = 1;
                        }
                        failed = true;
                        ready_upto = nchunks;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(32);
                }
                asm volatile("" ::: "memory");
            }
        };
        constexpr std::true_type yes{};
        constexpr std::false_type no{};
        // Chunk c travels in register buffer c % NB: NB chunks are in flight or on their way into LDS at any time.
        ensure_ready(0);
        ensure_ready(NB - 1);
        static_for<0, NB>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            if (j < nchunks) load(buf[j], sc[j], j);
        });
        if (nchunks > 0) {
            ensure_ready(NB);
            if (nchunks > NB) store_and_reload(buf[0], sc[0], 0, NB, yes);
            else store_and_reload(buf[0], sc[0], 0, 0, no);
        }
        __syncthreads();  // stage[0] holds chunk 0
        // Barrier c: the compute waves are done with stage[c & 1], chunk c + 1 is in the other half, and the
        // output of chunk c - 1 is in the output staging.  Before it: write chunk c + 1 (its half was released by
        // barrier c - 1) and refill the freed registers with chunk c + 1 + NB.
        int c = 0;  // a multiple of NB at the top of both loops
        for (; c + 2 * NB < nchunks; c += NB) {  // steady state: straight-line code, every reload exists
            static_for<0, NB>([&](auto jc) {
                constexpr int j = decltype(jc)::value, bi = (j + 1) % NB;
                ensure_ready(c + j + 1 + NB);
                store_and_reload(buf[bi], sc[bi], c + j + 1, c + j + 1 + NB, yes);
                __syncthreads();
                if (c + j > 0) flush(c + j - 1);
            });
        }
        for (; c < nchunks; c += NB) {  // the last chunks
            static_for<0, NB>([&](auto jc) {
                constexpr int j = decltype(jc)::value, bi = (j + 1) % NB;
                const int cc = c + j;
                if (cc < nchunks) {
                    if (cc + 1 < nchunks) {
                        ensure_ready(cc + 1 + NB);
                        if (cc + 1 + NB < nchunks) store_and_reload(buf[bi], sc[bi], cc + 1, cc + 1 + NB, yes);
                        else store_and_reload(buf[bi], sc[bi], cc + 1, 0, no);
                    }
                    __syncthreads();
                    if (cc > 0) flush(cc - 1);
                }
            });
        }
        __syncthreads();  // the hand-over of the last output tile
        if (nchunks > 0) flush(nchunks - 1);
        if constexpr (WAIT) {
            // Leave the flags of this chain clear for the next launch on this workspace.  A producer set a flag to 1; every
            // scan workgroup of the chain (p.scan_groups of them) adds 1 once none of its waves polls any more (they all
            // passed the barrier above), and the one that finds 1 + (p.scan_groups - 1) there is the last: it stores 0.
            if (lw == 0) {
                int32_t* const flags_of_chain = p.ready + (int64_t)h * p.TC + slot_begin;
                for (int c0 = 0; c0 < nchunks; c0 += WAVE) {
                    if (c0 + lane < nchunks) {
                        int32_t* const flag = flags_of_chain + c0 + lane;
                        const int32_t before = __hip_atomic_fetch_add(flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (before == p.scan_groups) __hip_atomic_store(flag, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
        }
        return;
    }

    // ------------------------------ compute ------------------------------
    const int sl = wave >> 1;                // slice of this workgroup
    const int tn = vgroup * NS + sl;         // 32-column tile of V
    const int l16 = lane % 16, g16 = l32 / 16;
    uint8_t* const xb_slice = xbuf[sl];

    auto compute = [&](auto ttc) {
        constexpr int TT = decltype(ttc)::value;  // token tile and key half of this wave
        lds_flag_t* const my_flag = (lds_flag_t*)&flags[sl][TT];
        lds_flag_t* const other_flag = (lds_flag_t*)&flags[sl][1 - TT];
        bf16x8* const xs_mine = reinterpret_cast<bf16x8*>(xb_slice + TT * XF * FRAG_BYTES) + lane;         // my half of S0; the partner's V~ arrives here
        bf16x8* const xs_other = reinterpret_cast<bf16x8*>(xb_slice + (1 - TT) * XF * FRAG_BYTES) + lane;  // the partner's half of S0; my V~ goes here
        bf16x8* const xx = reinterpret_cast<bf16x8*>(xb_slice + 2 * XF * FRAG_BYTES) + lane;               // X of token tile 0

        // State tile t of this wave is tile KDH TT + t of the slice.  Register r: MFMA row i = 8 (r/4) + 4 h + r%4 holds
        // state row 32 td + slice_col(i) = 32 td + 16 (r/8) + 8 h + 4 ((r/4) % 2) + r%4, column 32 tn + slice_col(l32).
        f32x16 S[KDH];
        const int64_t st_off = ((int64_t)n * p.H + h) * K * p.V + (int64_t)(8 * lh) * p.V + 32 * tn + slice_col(l32);
        auto st_row = [](int td, int r) { return 32 * td + 16 * (r / 8) + 4 * ((r / 4) % 2) + r % 4; };
#pragma unroll
        for (int t = 0; t < KDH; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) S[t][r] = 0.f;
        if (p.h0 != nullptr) {
#pragma unroll
            for (int t = 0; t < KDH; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) S[t][r] = p.h0[st_off + (int64_t)st_row(KDH * TT + t, r) * p.V];
        }

        bf16x8 sbm[SH];  // my half of the state as MFMA operand
#pragma unroll
        for (int i = 0; i < SH; i++) {
            sbm[i] = pack8_16(S[i / 2], i % 2, 1.f);
            xs_mine[i * WAVE] = sbm[i];
        }
        pair_publish(my_flag, 1);

        f32x16 acco;
#pragma unroll
        for (int r = 0; r < 16; r++) acco[r] = 0.f;
        auto write_out = [&](int parity) {  // O^T tile: register r is token 32 TT + l32, column 16 (r/8) + 8 h + r%8 of the slice
#pragma unroll
            for (int half = 0; half < 2; half++)
                *reinterpret_cast<bf16x8*>(ostage_at(sl, parity, 32 * TT + l32, 2 * half + lh)) = pack8_16(acco, half, 1.f);
        };

        __syncthreads();  // stage[0] holds chunk 0
        bf16x8 kfn[SH];  // rows of k for the first products of the next chunk, read right after the barrier that releases them
#pragma unroll
        for (int i = 0; i < SH; i++)
            kfn[i] = *reinterpret_cast<const bf16x8*>(stage[0] + K_OFF + (32 * TT + l32) * QLD + (16 * (SH * TT + i) + 8 * lh) * 2);

        for (int c = 0; c < nchunks; c++) {
            const uint8_t* st = stage[c & 1];
            const bf16_t* km = reinterpret_cast<const bf16_t*>(st + K_OFF);
            auto k_frag = [&](int s) {  // rows of k, token tile TT, key slab s: A operand of K S0
                return *reinterpret_cast<const bf16x8*>(st + K_OFF + (32 * TT + l32) * QLD + (16 * s + 8 * lh) * 2);
            };
            auto q_frag = [&](int s) {  // rows of q: B operand of (Q S0)^T
                return *reinterpret_cast<const bf16x8*>(st + Q_OFF + (32 * TT + l32) * QLD + (16 * s + 8 * lh) * 2);
            };
            auto kT_frag = [&](int td, int s) {  // k^T, key tile td (rows in state order), token slab s
                const bf16x4 a = lds_read_tr4x16<true>(km, QLD / 2, 16 * s + 4 * lh, 32 * td + 16 * g16, l16);
                const bf16x4 bb = lds_read_tr4x16<true>(km, QLD / 2, 16 * s + 8 + 4 * lh, 32 * td + 16 * g16, l16);
                bf16x8 r;
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = a[e], r[4 + e] = bb[e];
                return r;
            };
            auto rec_frag = [&](int f) { return reinterpret_cast<const bf16x8*>(st)[f * WAVE + lane]; };  // T' 0..5 | P 6..11

            // The order below is the schedule: what stands between two PIN()s stays there.  A wave issues in order and
            // an MFMA holds the matrix pipe for 32 cycles, so every MFMA is followed by a handful of instructions that do
            // not depend on it ("slots").  What is on the chain from one state to the next (K S0 -> X -> V~ -> state
            // update -> bf16 copy of the state) comes as early as its inputs allow; the output products (Q S0)^T and
            // V~^T P^T, the decay and the hand-over of the previous output fill the slots around it.
            bf16x8 kf[KS16], qf[KS16], sbo[SH], tf[4], xb[2], vbs[2], vb[2], ktf[KDH][4];
            f32x4 csr[4], ksr[4];
            bf16x4 xvr[4];
            f32x16 accv, vt;
            auto g2 = [&](auto jc) {  // MFMA j of (Q S0)^T: slabs of my half first
                constexpr int j = decltype(jc)::value;
                if constexpr (j < SH) acco = mfma32_bf16(sbm[j], qf[j], acco);
                else acco = mfma32_bf16(sbo[j - SH], qf[j], acco);
                pin_acc(acco);
            };
            auto x_piece = [&](int q4) {  // X = V - diag(cs) K S0, tokens 32 TT + 8 q4 + 4 h + 0..3 of this lane's column
#pragma unroll
                for (int e = 0; e < 4; e++) accv[4 * q4 + e] = (float)xvr[q4][e] - csr[q4][e] * accv[4 * q4 + e];
            };
            auto v_piece = [&](int x, int sub) {  // half a fragment of V~ with its rows scaled for the state update
#pragma unroll
                for (int e = 0; e < 4; e++) vbs[x][4 * sub + e] = (bf16_t)(vt[8 * x + 4 * sub + e] * ksr[2 * x + sub][e]);
            };
#pragma unroll
            for (int i = 0; i < SH; i++) kf[i] = kfn[i];
            const float egc = *reinterpret_cast<const float*>(st + EG_OFF);
            const float qsc = reinterpret_cast<const float*>(st + QS_OFF)[32 * TT + l32];
#pragma unroll
            for (int r = 0; r < 16; r++) accv[r] = 0.f, vt[r] = 0.f;
            PIN();

            // ---- K S0, my half of the key dim | decay of the state (its bf16 copy for this chunk is in sbm), operand reads ----
            static_for<0, SH>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                accv = mfma32_bf16(kf[i], sbm[i], accv);
                pin_acc(accv);
                constexpr int per = (16 * KDH + SH - 1) / SH;
#pragma unroll
                for (int x = i * per; x < (i + 1) * per && x < 16 * KDH; x++) S[x / 16][x % 16] *= egc;
                kf[SH + i] = k_frag(SH * (1 - TT) + i);
                qf[i] = q_frag(SH * TT + i);
                PIN();
            });
            // ---- the previous chunk's output leaves the accumulators; first product of (Q S0)^T ----
            write_out((c - 1) & 1);  // (chunk 0 hands over zeros, which nobody writes out)
#pragma unroll
            for (int r = 0; r < 16; r++) acco[r] = 0.f;
            PIN();
            g2(std::integral_constant<int, 0>{});
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                csr[q4] = *reinterpret_cast<const f32x4*>(st + CS_OFF + (32 * TT + 8 * q4 + 4 * lh) * 4);
                xvr[q4] = lds_read_tr4x16<true>(reinterpret_cast<const bf16_t*>(st + V_OFF), VLD / 2, 32 * TT + 8 * q4 + 4 * lh, 32 * sl + 16 * g16, l16);
            }
            PIN();
            pair_wait(other_flag, 3 * c + 1);
#pragma unroll
            for (int i = 0; i < SH; i++) sbo[i] = xs_other[i * WAVE];
            PIN();
            // ---- K S0, the partner's half | operand reads ----
            static_for<0, SH>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                accv = mfma32_bf16(kf[SH + i], sbo[i], accv);
                pin_acc(accv);
                qf[SH + i] = q_frag(SH * (1 - TT) + i);
                if constexpr (i == 0) {
                    if constexpr (TT == 0) tf[0] = rec_frag(0), tf[1] = rec_frag(1);
                    else tf[0] = rec_frag(4), tf[1] = rec_frag(5), tf[2] = rec_frag(2), tf[3] = rec_frag(3);
                }
                if constexpr (i == 1) {
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) ksr[q4] = *reinterpret_cast<const f32x4*>(st + KS_OFF + (32 * TT + 8 * q4 + 4 * lh) * 4);
                }
                PIN();
            });
            // ---- X, with (Q S0)^T in the matrix pipe ----
            g2(std::integral_constant<int, 1>{});
            PIN();
            static_for<0, 2>([&](auto hc) {
                constexpr int hf = decltype(hc)::value;
                g2(std::integral_constant<int, 2 + hf>{});
                x_piece(2 * hf), x_piece(2 * hf + 1);
                xb[hf] = pack8_16(accv, hf, 1.f);
                if constexpr (TT == 0) xx[hf * WAVE] = xb[hf];
                PIN();
            });
            if constexpr (TT == 0) pair_publish(my_flag, 3 * c + 2);
            PIN();
            // ---- V~ = T' X (tile 1: its own X first, then tile 0's) ----
            vt = mfma32_bf16(tf[0], xb[0], vt);
            vt = mfma32_bf16(tf[1], xb[1], vt);
            pin_acc(vt);
#pragma unroll
            for (int t = 0; t < KDH; t++)
#pragma unroll
                for (int j = 0; j < 2; j++) ktf[t][j] = kT_frag(KDH * TT + t, 2 * TT + j);
            PIN();
            constexpr int G2_BEFORE_V = KS16 >= 8 ? 6 : 4;  // products of (Q S0)^T issued before V~ is packed
            if constexpr (TT == 1) {
                static_for<4, G2_BEFORE_V>([&](auto jc) { g2(jc); });
                PIN();
                pair_wait(other_flag, 3 * c + 2);
                const bf16x8 x0 = xx[0], x1 = xx[WAVE];
                vt = mfma32_bf16(tf[2], x0, vt);
                vt = mfma32_bf16(tf[3], x1, vt);
                pin_acc(vt);
                PIN();
            } else {
                static_for<4, G2_BEFORE_V>([&](auto jc) { g2(jc); });
                PIN();
            }
            const bf16x8 pm0 = rec_frag(TT == 0 ? 6 : 10), pm1 = rec_frag(TT == 0 ? 7 : 11);
            PIN();

            // ---- V~ as operands (rows scaled by ks for the state update, plain for P V~), the rest of (Q S0)^T between ----
            static_for<0, 2>([&](auto xc) {
                constexpr int x = decltype(xc)::value;
                if constexpr (G2_BEFORE_V + x < KS16) g2(std::integral_constant<int, (G2_BEFORE_V + x < KS16 ? G2_BEFORE_V + x : 0)>{});
                v_piece(x, 0), v_piece(x, 1);
                xs_other[x * WAVE] = vbs[x];
                PIN();
            });
            vb[0] = pack8_16(vt, 0, 1.f), vb[1] = pack8_16(vt, 1, 1.f);
            if constexpr (TT == 0) xs_other[2 * WAVE] = vb[0], xs_other[3 * WAVE] = vb[1];
            pair_publish(my_flag, 3 * c + 3);
            PIN();
            // ---- S += k^T V~', my token tile's slabs | q's row scale on (Q S0)^T, complete by now ----
            static_for<0, 2 * KDH>([&](auto uc) {
                constexpr int u = decltype(uc)::value, t = u / 2, j = u % 2;
                S[t] = mfma32_bf16(ktf[t][j], vbs[j], S[t]);
                pin_acc(S[t]);
                constexpr int per = (16 + 2 * KDH - 1) / (2 * KDH);
#pragma unroll
                for (int r = u * per; r < (u + 1) * per && r < 16; r++) acco[r] *= qsc;
                ktf[t][2 + j] = kT_frag(KDH * TT + t, 2 * (1 - TT) + j);
                PIN();
            });
            // ---- O^T += V~^T P^T, my slabs ----
            acco = mfma32_bf16(vb[0], pm0, acco);
            acco = mfma32_bf16(vb[1], pm1, acco);
            pin_acc(acco);
            bf16x8 po0 = {}, po1 = {};
            if constexpr (TT == 1) po0 = rec_frag(8), po1 = rec_frag(9);
            PIN();
            pair_wait(other_flag, 3 * c + 3);
            const bf16x8 vo0 = xs_mine[0], vo1 = xs_mine[WAVE];
            bf16x8 pv0 = {}, pv1 = {};
            if constexpr (TT == 1) pv0 = xs_mine[2 * WAVE], pv1 = xs_mine[3 * WAVE];
            PIN();
            // ---- S += k^T V~', the partner's slabs ----
#pragma unroll
            for (int t = 0; t < KDH; t++) {
                S[t] = mfma32_bf16(ktf[t][2], vo0, S[t]);
                S[t] = mfma32_bf16(ktf[t][3], vo1, S[t]);
            }
            PIN();
            __syncthreads();  // this wave has read all it needs of chunk c's half; chunk c + 1 is in the other one
            if constexpr (TT == 1) {
                acco = mfma32_bf16(pv0, po0, acco);
                acco = mfma32_bf16(pv1, po1, acco);
            }
            {   // the first operands of the next chunk
                const uint8_t* stn = stage[(c + 1) & 1];
#pragma unroll
                for (int i = 0; i < SH; i++)
                    kfn[i] = *reinterpret_cast<const bf16x8*>(stn + K_OFF + (32 * TT + l32) * QLD + (16 * (SH * TT + i) + 8 * lh) * 2);
            }
            PIN();

            // ---- the new state as operand of the next chunk ----
#pragma unroll
            for (int i = 0; i < SH; i++) {
                sbm[i] = pack8_16(S[i / 2], i % 2, 1.f);
                xs_mine[i * WAVE] = sbm[i];
            }
            pair_publish(my_flag, 3 * (c + 1) + 1);
        }

        if (nchunks > 0) write_out((nchunks - 1) & 1);
        __syncthreads();  // the loaders write the last output tile

        if (p.ht != nullptr && !(WAIT && *wg_failed != 0)) {
#pragma unroll
            for (int t = 0; t < KDH; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) p.ht[st_off + (int64_t)st_row(KDH * TT + t, r) * p.V] = S[t][r];
        }
    };
    if (wave & 1) compute(std::integral_constant<int, 1>{});
    else compute(std::integral_constant<int, 0>{});
}

// ------------------------------------------------------------------------------------------
// kernels
// ------------------------------------------------------------------------------------------
// Prepare and scan in one launch (fixed-length batches whose scan fills between 3/8 and 1/2 of the CUs).  Every workgroup
// takes a CU to itself (by its LDS size).  The first `prep_wgs` workgroups are producers: two groups of four waves
// each run the prepare step on items of the chains that are scanned on their XCD, earliest chunks first, and set a
// flag per finished record.  The others are scan workgroups whose loaders wait for those flags.  A producer never
// waits for anything and the producers have the lowest workgroup ids, which are dispatched first: the launch cannot
// block itself whatever part of it is resident.  What this buys: the prepare step runs beside the scan instead of
// before it, and the scan finds q, k and the records of a chain in the L2 of its XCD shortly after they were used.
constexpr int FUSED_GROUPS = 2;

template <int K, int NS>
__global__ __launch_bounds__(PAIR_THREADS) void chunk_fused_kernel(const ChunkParams p, const int prep_wgs) {
    constexpr int SCAN_LDS = scan_pair_lds_bytes<K, NS>(), PREP_LDS = FUSED_GROUPS * prepare32_lds_bytes<K>();
    __shared__ __attribute__((aligned(16))) uint8_t lds[SCAN_LDS > PREP_LDS ? SCAN_LDS : PREP_LDS];
    if ((int)blockIdx.x >= prep_wgs) {
        scan_pair_body<K, NS, true>(p, lds, (int)blockIdx.x - prep_wgs);  // prep_wgs is a multiple of 8: same XCD numbering
        return;
    }
    if (p.no_producers) return;  // GDN_FLAG_DEBUG_NO_PRODUCERS: the scan's waits run out
    // producer: items of XCD x are (chunk c, chain) for the chains x * per_xcd .. the scan puts on that XCD, chunk-major
    const int xcd = blockIdx.x % 8, rank = blockIdx.x / 8, per = prep_wgs / 8;
    const int chains = p.N * p.H, per_xcd = (chains + 7) / 8;
    const int first_chain = xcd * per_xcd;
    const int nch = max(0, min(per_xcd, chains - first_chain));
    const uint32_t items = (uint32_t)nch * (uint32_t)p.NT;
    const int H = p.H, NT = p.NT;
    auto item_of = [=](uint32_t i, int& h, int& slot) {
        const int c = (int)(i / (uint32_t)nch), chain = first_chain + (int)(i % (uint32_t)nch);
        h = chain % H;
        slot = (chain / H) * NT + c;
    };
    const uint32_t step = (uint32_t)(per * FUSED_GROUPS);
    const uint32_t rounds = (items + step - 1) / step;
    const uint32_t group = threadIdx.x / PREP_THREADS;
    if (group >= (uint32_t)FUSED_GROUPS) return;
    chunk_prepare32_body<K, FUSED_GROUPS, true>(p, lds, item_of, items, (uint32_t)rank * FUSED_GROUPS + group, step, rounds, p.ready, 1);
}

__global__ void fill_zero_kernel(int32_t* x, int64_t n) {
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) x[i] = 0;
}

// ------------------------------------------------------------------------------------------
// launch
// ------------------------------------------------------------------------------------------
// The fused launch: scan workgroups of two slices each beside the producers.  Returns GDN_ERR_UNSUPPORTED (before any
// launch) when the shape does not qualify; the caller then runs prepare and scan as two kernels.
template <int K>
static int launch_fused_k(ChunkParams& p, hipStream_t stream, int num_cus) {
    const int64_t chains8 = ((int64_t)p.N * p.H + 7) / 8 * 8;
    p.scan_groups = p.V / 64;
    const int64_t scan_wgs = chains8 * p.scan_groups;
    const int prep_wgs = (int)((num_cus - scan_wgs) / 8 * 8);
    if (!fused_launch_window((int64_t)p.N * p.H, p.V, num_cus)) return GDN_ERR_UNSUPPORTED;
    if (!p.ready_clear) {  // the scan waits for flags the producers set: they must start at zero (and end there: scan_pair_body)
        const int64_t nflags = (int64_t)p.H * p.TC + 1;  // with the error latch, the word in front of them
        hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((nflags + 255) / 256 < 64 ? (nflags + 255) / 256 : 64)), dim3(256), 0, stream, p.ready - 1, nflags);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL((chunk_fused_kernel<K, 2>), dim3((unsigned)(prep_wgs + scan_wgs)), dim3(PAIR_THREADS), 0, stream, p, prep_wgs);
    return (int)hipGetLastError();
}

bool chunk_fused_supported(const ChunkParams& p, int K) {
    return (K == 64 || K == 128) && p.V % 64 == 0 && p.cu_seqlens == nullptr && p.pad_lens == nullptr && p.ready != nullptr && p.err == p.ready - 1 &&
           !p.records_given && p.save_state == nullptr && p.save_vnew == nullptr;
}

int launch_chunk_fused(ChunkParams& p, int K, hipStream_t stream, int num_cus) {
    if (!chunk_fused_supported(p, K)) return GDN_ERR_UNSUPPORTED;
    if (K == 64) return launch_fused_k<64>(p, stream, num_cus);
    return launch_fused_k<128>(p, stream, num_cus);
}

}  // namespace gdn

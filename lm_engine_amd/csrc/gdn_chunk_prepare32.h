// The prepare step of the chunked forward on v_mfma_f32_32x32x16_bf16 (K = 64, 128, 256): everything about a chunk
// that does not depend on the state, written as one record per (head, chunk slot).  A device function, so that it can
// run as a kernel of its own (gdn_chunk32.hip) and as the producer half of the one-launch forward (gdn_chunk_fused.hip).
#pragma once

#include "gdn_chunk32_common.h"

namespace gdn {

// x of another lane as named by a DPP control word; lanes the move does not write (outside ROW_MASK, or shifted in
// from outside their row) get 0
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROW_MASK, 0xF, false));
}

// Stores into a record, `offset` bytes from its start.  DEVICE_SCOPE: written through to memory (scope bit sc1), so that
// a workgroup on another XCD, whose L2 is a different one, reads what was written once the flag of the record says so.
// (The alternative, a release fence at device scope, writes back every dirty line of the XCD's L2: 13 us per record.
// And the stores are buffer stores through the compiler's builtin, not inline asm: the compiler has to count them, or
// its waits for the prefetched loads of the next item come out wrong.)
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
template <bool DEVICE_SCOPE>
__device__ __forceinline__ void record_store(uint8_t* rec, uint32_t bytes, uint32_t offset, bf16x8 v) {
    if constexpr (DEVICE_SCOPE)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), __builtin_amdgcn_make_buffer_rsrc(rec, 0, bytes, 0x00020000), offset, 0, 16);
    else *reinterpret_cast<bf16x8*>(rec + offset) = v;
}
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
template <bool DEVICE_SCOPE>
__device__ __forceinline__ void record_store(uint8_t* rec, uint32_t bytes, uint32_t offset, bf16x4 v) {
    if constexpr (DEVICE_SCOPE)
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), __builtin_amdgcn_make_buffer_rsrc(rec, 0, bytes, 0x00020000), offset, 0, 16);
    else *reinterpret_cast<bf16x4*>(rec + offset) = v;
}
template <bool DEVICE_SCOPE>
__device__ __forceinline__ void record_store(uint8_t* rec, uint32_t bytes, uint32_t offset, float v) {
    if constexpr (DEVICE_SCOPE)
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), __builtin_amdgcn_make_buffer_rsrc(rec, 0, bytes, 0x00020000), offset, 0, 16);
    else *reinterpret_cast<float*>(rec + offset) = v;
}

// ------------------------------------------------------------------------------------------
// prepare
// ------------------------------------------------------------------------------------------
// LDS bytes one group of four waves needs
template <int K>
constexpr int prepare32_lds_bytes() {
    constexpr int LDK = K + 8, LDA = C + 4, LDT = 36, LDM = 20;
    constexpr int SCRATCH_FLOATS = 32 * LDT + 2 * 16 * LDM + 32 * LDT;
    constexpr int KM_BYTES = (C * LDK * 2 > SCRATCH_FLOATS * 4) ? C * LDK * 2 : SCRATCH_FLOATS * 4;
    return KM_BYTES + C * LDK * 2 + C * LDA * 4 + 6 * C * 4;
}

// Work of one prepare item (one chunk of one head) by a group of four waves; a workgroup holds GROUPS such groups,
// each with its own LDS region and its own items, which pass the eight barriers of an item together.
//   items            number of items;  item_of(i, h, slot) names item i (head, chunk slot)
//   first, step      this group works on items first, first + step, ...; `rounds` iterations for every group
//                    of the workgroup (a group whose item index runs past `items` only keeps the barriers company)
//   FLAGS, ready     ready[h * TC + slot] is set to `epoch` once the record is complete and visible to the whole
//                    device (the scan of the same launch waits for it)
template <int K, int GROUPS, bool FLAGS, typename ItemOf>
__device__ __forceinline__ void chunk_prepare32_body(const ChunkParams& p, uint8_t* lds_base, ItemOf item_of, uint32_t items,
                                                     uint32_t first, uint32_t step, uint32_t rounds, int32_t* ready, int32_t epoch) {
    constexpr int LDK = K + 8;  // bf16 elements per LDS row of K / Q
    constexpr int LDA = C + 4;  // fp32 elements per LDS row of A / T
    constexpr int LDT = 36;     // fp32 elements per row of the 32 x 32 transposed blocks
    constexpr int LDM = 20;     // fp32 elements per row of a 16 x 16 scratch block
    constexpr int KS16 = K / 16;
    constexpr int KD = K / 32;  // 32-row tiles of the key dim
    constexpr int CPR = K / 8;  // 16 B pieces per row of K / Q
    constexpr int RPP = PREP_THREADS / CPR;  // rows per pass of the K / Q copy
    constexpr int NPASS = C / RPP;
    // K is dead once A and P are formed; the scratch blocks of the block merges take its place.  T is built in
    // place of A, block by block.
    constexpr int SCRATCH_FLOATS = 32 * LDT + 2 * 16 * LDM + 32 * LDT;
    constexpr int KM_BYTES = (C * LDK * 2 > SCRATCH_FLOATS * 4) ? C * LDK * 2 : SCRATCH_FLOATS * 4;
    static_assert(KM_BYTES + C * LDK * 2 + C * LDA * 4 + 6 * C * 4 == prepare32_lds_bytes<K>(), "LDS layout and its size disagree");
    const int group = GROUPS == 1 ? 0 : (int)(threadIdx.x / PREP_THREADS);
    uint8_t* const lds = lds_base + group * prepare32_lds_bytes<K>();
    uint8_t* const sKM = lds;
    bf16_t* const sQ = reinterpret_cast<bf16_t*>(lds + KM_BYTES);
    float* const sA = reinterpret_cast<float*>(lds + KM_BYTES + C * LDK * 2);
    float* const s_gam = sA + C * LDA;
    float* const s_beta = s_gam + C, * const s_ssk = s_beta + C, * const s_ssq = s_ssk + C, * const s_rk = s_ssq + C, * const s_rq = s_rk + C;
    float* const s_bri = s_ssk, * const s_g2 = s_ssq;  // from barrier #2 on: beta / |k| and gamma log2(e) per token
    float* const sT = sA;
    bf16_t* const sK = reinterpret_cast<bf16_t*>(sKM);
    float* const sTtA = reinterpret_cast<float*>(sKM);  // transpose of the top-left 32 x 32 of T
    float* const sMt = sTtA + 32 * LDT;                 // transposed products
    float* const sMtB = sMt + 2 * 16 * LDM;

    const int tid = threadIdx.x % PREP_THREADS;
    // role of this wave in its group; the hardware puts wave w of a workgroup on SIMD w % 4, so with several groups the
    // roles are rotated from group to group: the one-wave steps of the inverse then run on different SIMDs
    const int wave = (tid / WAVE + group) % 4;
    // ---- register prefetch of one item's inputs ----
    bf16x8 kx[NPASS], qx[NPASS];
    float gx = 0.f;
    uint32_t bx_raw = 0;  // beta of the prefetched item, raw bits: any arithmetic on it here would wait for every load in flight
    ChunkCoord ncc;  // coordinates of the prefetched item
    int nh = 0, nslot = 0;
    auto locate = [&](uint32_t w) {  // wave-uniform 32-bit arithmetic
        if (w < items) {
            item_of(w, nh, nslot);
            ncc = locate_chunk(p, nslot);
        } else {
            nh = 0, nslot = 0, ncc.n = 0, ncc.b = 0, ncc.t0 = 0, ncc.len = 0;
        }
    };
    // Loads are written as (workgroup-uniform base pointer) + (32-bit per-lane element offset) so that the
    // compiler keeps one offset register per stream instead of a 64-bit address per load.
    const uint32_t kq_piece = tid % CPR, kq_row0 = tid / CPR;
    const uint32_t k_lane_off = kq_row0 * (uint32_t)p.k_stride_t + kq_piece * 8;
    const uint32_t q_lane_off = kq_row0 * (uint32_t)p.q_stride_t + kq_piece * 8;
    const int lane0 = tid % WAVE;
    auto prefetch_kq = [&]() {
        const int nhqk = qk_head_of(nh, p.qk_div);
        const bf16_t* kg = p.k + ncc.b * p.k_stride_b + ncc.t0 * p.k_stride_t + (int64_t)nhqk * p.k_stride_h;
        const bf16_t* qg = p.q + ncc.b * p.q_stride_b + ncc.t0 * p.q_stride_t + (int64_t)nhqk * p.q_stride_h;
#pragma unroll
        for (int it = 0; it < NPASS; it++) {
            const int row = kq_row0 + it * RPP;
            kx[it] = bf16x8{};
            qx[it] = bf16x8{};
            if (row < ncc.len) {
                kx[it] = *reinterpret_cast<const bf16x8*>(kg + (int64_t)(it * RPP) * p.k_stride_t + k_lane_off);
                qx[it] = *reinterpret_cast<const bf16x8*>(qg + (int64_t)(it * RPP) * p.q_stride_t + q_lane_off);
            }
        }
        if (wave == 0) {
            gx = 0.f, bx_raw = 0u;
            if (lane0 < ncc.len) {
                const int64_t sbase = (ncc.b * p.T + ncc.t0) * p.H + nh;
                const uint32_t soff = (uint32_t)lane0 * (uint32_t)p.H;
                if (p.g != nullptr) gx = (p.g + sbase)[soff];
                if (p.beta == nullptr) bx_raw = 0x3f800000u;  // 1.0f
                else if (p.beta_dtype == GDN_BF16) bx_raw = (reinterpret_cast<const uint16_t*>(p.beta) + sbase)[soff];  // shifted at use
                else bx_raw = (reinterpret_cast<const uint32_t*>(p.beta) + sbase)[soff];
            }
        }
    };
    uint32_t w = first;
    locate(w);
    prefetch_kq();

    for (uint32_t round = 0; round < rounds; round++, w += step) {
        // Lane coordinates are re-derived in every iteration from a value the optimiser cannot see
        // through: hoisted out of this loop, the many lane-dependent addresses and masks below would
        // stay live across all phases and spill.
        int lane = tid % WAVE;
        asm volatile("" : "+v"(lane));
        const int l16 = lane % 16, lq = lane / 16;  // 16 x 16 MFMA coordinates
        const int l32 = lane % 32, lh = lane / 32;  // 32 x 32 MFMA coordinates
        const int g16 = l32 / 16;                   // which 16-lane group of the 32-row operand
        const ChunkCoord cc = ncc;
        const int h = nh;
        const int len = cc.len;  // <= 0 for an unused slot (packed batch, rounded-up grid): nothing to do
        uint8_t* const rec = p.rec + ((int64_t)h * p.TC + nslot) * p.rec_bytes;
        const bool has_next = round + 1 < rounds;
        const int slot = nslot;

        // ---- registers -> LDS (K, Q), row sums of squares, gamma = cumsum(g), beta ----
        if (len > 0) {
            const int piece = tid % CPR;
#pragma unroll
            for (int it = 0; it < NPASS; it++) {
                const int row = tid / CPR + it * RPP;
                *reinterpret_cast<bf16x8*>(&sK[row * LDK + piece * 8]) = kx[it];
                *reinterpret_cast<bf16x8*>(&sQ[row * LDK + piece * 8]) = qx[it];
                if (p.l2norm) {  // row sums of squares (uniform branch)
                    float a = 0.f, b = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        a += (float)kx[it][e] * (float)kx[it][e];
                        b += (float)qx[it][e] * (float)qx[it][e];
                    }
#pragma unroll
                    for (int off = 1; off < CPR; off <<= 1) {
                        a += __shfl_xor(a, off, WAVE);
                        b += __shfl_xor(b, off, WAVE);
                    }
                    if (piece == 0) s_ssk[row] = a, s_ssq[row] = b;
                }
            }
            if (wave == 0) {
                // inclusive prefix sum over the 64 lanes in data-parallel-primitive moves (shifts inside a row of 16
                // lanes with zero fill, then the last lane of a row broadcast to the rows above): six dependent adds
                // instead of six round trips through the LDS crossbar
                float gv = gx;
                gv += dpp_move<0x111, 0xF>(gv);  // row_shr:1
                gv += dpp_move<0x112, 0xF>(gv);  // row_shr:2
                gv += dpp_move<0x114, 0xF>(gv);  // row_shr:4
                gv += dpp_move<0x118, 0xF>(gv);  // row_shr:8
                gv += dpp_move<0x142, 0xA>(gv);  // row_bcast:15 into rows 1 and 3
                gv += dpp_move<0x143, 0xC>(gv);  // row_bcast:31 into rows 2 and 3
                s_gam[lane] = gv;
                s_beta[lane] = __builtin_bit_cast(float, (p.beta != nullptr && p.beta_dtype == GDN_BF16) ? bx_raw << 16 : bx_raw);
            }
        }
        // the q, k registers are free: start on the next item
        if (has_next) {
            locate(w + step);
            prefetch_kq();
        }
        if (len <= 0) {  // uniform over the group: nothing to do
            if constexpr (GROUPS > 1) {  // the other groups of the workgroup still meet at their barriers
#pragma unroll
                for (int i = 0; i < 8; i++) __syncthreads();
            }
            continue;
        }
        __syncthreads();  // #1

        if (tid < C) {
            const float gam = s_gam[tid], gl = s_gam[C - 1];
            const float rk = p.l2norm ? rsqrtf(s_ssk[tid] + L2NORM_EPS) : 1.f;
            const float rq = p.l2norm ? rsqrtf(s_ssq[tid] + L2NORM_EPS) : 1.f;
            s_rk[tid] = rk;
            s_rq[tid] = rq;
            // what the tile epilogues below multiply with, once per token instead of once per matrix entry (the sums of
            // squares are not needed any more): beta_i / |k_i| and gamma_i in units of log 2
            s_ssk[tid] = s_beta[tid] * rk;
            s_ssq[tid] = gam * 1.44269504088896341f;
            // row scales the scan applies: to q S0, to the rows of V~ in the state update, to k S0 (none for
            // the rows past the end of a short chunk: the scan reads some other token's k and v there)
            const bool valid = tid < len;
            record_store<FLAGS>(rec, p.rec_bytes, p.off_qs + 4 * tid, __expf(gam) * p.scale * rq);
            record_store<FLAGS>(rec, p.rec_bytes, p.off_ks + 4 * tid, valid ? __expf(gl - gam) * rk : 0.f);
            record_store<FLAGS>(rec, p.rec_bytes, p.off_cs + 4 * tid, valid ? __expf(gam) * rk : 0.f);
            if (tid == 0) record_store<FLAGS>(rec, p.rec_bytes, p.off_eg, __expf(gl));
        }
        __syncthreads();  // #2

        // ---- A = strict-lower(beta_i e^{gamma_i - gamma_j} k^_i . k^_j) -> sA;  P -> record ----
        {
            // 32 x 32 tile jobs: G(Ti, Tj) = K_Ti K_Tj^T (rows i, column j), Pt(Tj, Ti) = K_Tj Q_Ti^T (rows j, column i)
            auto tile_job = [&](bool is_p, int trow, int tcol) {
                f32x16 acc;
#pragma unroll
                for (int r = 0; r < 16; r++) acc[r] = 0.f;
                const bf16_t* bsrc = is_p ? sQ : sK;
#pragma unroll
                for (int s = 0; s < KS16; s++) {
                    const bf16x8 a = *reinterpret_cast<const bf16x8*>(&sK[(32 * trow + l32) * LDK + 16 * s + 8 * lh]);
                    const bf16x8 b = *reinterpret_cast<const bf16x8*>(&bsrc[(32 * tcol + l32) * LDK + 16 * s + 8 * lh]);
                    acc = mfma32_bf16(a, b, acc);
                    if (s % 2 == 1) __builtin_amdgcn_sched_barrier(0);  // keeps the operand reads from piling up in registers
                }
                // register quad q of the tile holds rows 32 trow + 8 q + 4 h + 0..3: their per-token values in one read
                if (!is_p) {
                    const int j = 32 * tcol + l32;
                    const float gj = s_g2[j], rkj = s_rk[j];
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int i0 = 32 * trow + 8 * q + 4 * lh;
                        const f32x4 bi = *reinterpret_cast<const f32x4*>(&s_bri[i0]);
                        const f32x4 gi = *reinterpret_cast<const f32x4*>(&s_g2[i0]);
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float val = bi[e] * __builtin_amdgcn_exp2f(gi[e] - gj) * (rkj * acc[4 * q + e]);
                            sA[(i0 + e) * LDA + j] = (trow > tcol || i0 + e > j) ? val : 0.f;
                        }
                    }
                } else {
                    const int i = 32 * tcol + l32;
                    const float gi = s_g2[i], qi = p.scale * s_rq[i];
                    f32x16 pv;
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int j0 = 32 * trow + 8 * q + 4 * lh;
                        const f32x4 rj = *reinterpret_cast<const f32x4*>(&s_rk[j0]);
                        const f32x4 gj = *reinterpret_cast<const f32x4*>(&s_g2[j0]);
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float val = rj[e] * __builtin_amdgcn_exp2f(gi - gj[e]) * (qi * acc[4 * q + e]);
                            pv[4 * q + e] = (tcol > trow || i >= j0 + e) ? val : 0.f;
                        }
                    }
                    if (p.rec16) {
                        // 16x16x32 fragments (it, s): 16 output tokens 16 it .. of P, 32 reduction tokens 32 s ..; lane
                        // (i, g) of a fragment holds P[16 it + i][32 s + 4 g + 0..3] and P[16 it + i][32 s + 16 + 4 g + 0..3].
                        // This lane has token i = 32 tcol + l32 and, in register quad q, tokens j = 32 trow + 8 q + 4 h + 0..3:
                        // a half of lane (l32 % 16, 2 (q % 2) + h) of fragment (2 tcol + l32 / 16, trow).
                        const int it = 2 * tcol + l32 / 16;
                        const int frag = it < 2 ? it : 2 * it - 2 + trow;  // (0,0) (1,0) (2,0) (2,1) (3,0) (3,1)
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            bf16x4 piece;
#pragma unroll
                            for (int e = 0; e < 4; e++) piece[e] = (bf16_t)pv[4 * q + e];
                            const int g = 2 * (q % 2) + lh;
                            record_store<FLAGS>(rec, p.rec_bytes, p.off_p + (frag * WAVE + 16 * g + l32 % 16) * 16 + 8 * (q / 2), piece);
                        }
                    } else {
                        // fragments (tcol, 2 trow + s); the all-zero pair (tcol 0, trow 1) has no place in the record
                        const int first = tcol == 0 ? 0 : 2 + 2 * trow;
                        record_store<FLAGS>(rec, p.rec_bytes, p.off_p + ((first + 0) * WAVE + lane) * 16, pack8_16(pv, 0, 1.f));
                        record_store<FLAGS>(rec, p.rec_bytes, p.off_p + ((first + 1) * WAVE + lane) * 16, pack8_16(pv, 1, 1.f));
                    }
                }
            };
            // first the two diagonal tiles of A, which the inverse starts from, and two of the three tiles of P
            if (wave == 0) tile_job(false, 0, 0);
            else if (wave == 1) tile_job(true, 0, 0);
            else if (wave == 2) tile_job(false, 1, 1);
            else tile_job(true, 1, 1);  // P[i < 32][j >= 32] = 0 is not stored
            __syncthreads();  // #3: the diagonal tiles of A are complete
            // then wave 0 inverts the diagonal blocks (a long dependent chain on one wave) while two others
            // finish the tiles: K and Q stay in place until barrier #4
            if (wave == 1) tile_job(false, 1, 0);
            else if (wave == 2) tile_job(true, 0, 1);
        }

        // ---- wave 0: inverses of the four 16 x 16 diagonal blocks, written over the blocks of A ----
        float x[16];  // column l16 of the inverse of block lq (wave 0)
        if (wave == 0) {
            const int blk = lq, j = l16;  // lane owns column j of block `blk`
            const float* a = &sA[(16 * blk) * LDA + 16 * blk];
#pragma unroll
            for (int i = 0; i < 16; i++) {
                f32x4 row[4];
#pragma unroll
                for (int c4 = 0; c4 < (i + 3) / 4; c4++) row[c4] = *reinterpret_cast<const f32x4*>(&a[i * LDA + 4 * c4]);
                float part[4] = {(i == j) ? 1.f : 0.f, 0.f, 0.f, 0.f};  // four independent partial sums
#pragma unroll
                for (int kk = 0; kk < i; kk++) part[kk % 4] -= row[kk / 4][kk % 4] * x[kk];
                x[i] = (part[0] + part[1]) + (part[2] + part[3]);
            }
            // every lane of the wave has read its block of A by now (one wave, program order)
#pragma unroll
            for (int i = 0; i < 16; i++) sT[(16 * blk + i) * LDA + 16 * blk + j] = x[i];
        }
        __syncthreads();  // #4: diagonal blocks of T, all of A and P; K and Q are dead

        // 16 x 16 output tile of a product X Y on the fp32 MFMA (16x16x4: no operand is rounded).  Lane (l16, lq) supplies
        // reduction entries k = 4 n lq + e, e < 4 n, of row l16 of X and of column l16 of Y (a row of Y^T); MFMA e takes
        // entry e of every lane, i.e. the four k = 4 n lq' + e, and the 4 n MFMAs together cover all 16 n.
        auto mm16 = [&](const float* xrow, const float* ytrow) -> f32x4 {  // 16 reduction entries, k = 4 lq + e
            const f32x4 x = *reinterpret_cast<const f32x4*>(xrow), y = *reinterpret_cast<const f32x4*>(ytrow);
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < 4; e++) acc = mfma_f32(x[e], y[e], acc);
            return acc;
        };
        auto mm16x32 = [&](const float* xrow, const float* ytrow) -> f32x4 {  // 32 reduction entries, k = 8 lq + e
            const f32x4 x0 = *reinterpret_cast<const f32x4*>(xrow), x1 = *reinterpret_cast<const f32x4*>(xrow + 4);
            const f32x4 y0 = *reinterpret_cast<const f32x4*>(ytrow), y1 = *reinterpret_cast<const f32x4*>(ytrow + 4);
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < 4; e++) acc = mfma_f32(x0[e], y0[e], acc);
#pragma unroll
            for (int e = 0; e < 4; e++) acc = mfma_f32(x1[e], y1[e], acc);
            return acc;
        };

        // ---- level A: T_10 = -T_11 (A_10 T_00) on wave 0, T_32 = -T_33 (A_32 T_22) on wave 1 ----
        if (wave < 2) {
            const int bi = 2 * wave + 1, bj = 2 * wave;
            const int kk = 4 * lq;
            float* const mt = &sMt[wave * 16 * LDM];
            // column l16 of T_bj,bj, entries kk .. kk + 3 (a row of its transpose)
            f32x4 y0;
#pragma unroll
            for (int e = 0; e < 4; e++) y0[e] = sT[(16 * bj + kk + e) * LDA + 16 * bj + l16];
            f32x4 m = {0.f, 0.f, 0.f, 0.f};
            {
                const f32x4 xa = *reinterpret_cast<const f32x4*>(&sA[(16 * bi + l16) * LDA + 16 * bj + kk]);
#pragma unroll
                for (int e = 0; e < 4; e++) m = mfma_f32(xa[e], y0[e], m);
            }
            if (wave == 0 && lq < 2) {
                // K's region is free now: the transposes of T_00 and T_11 for level B, from the registers of the inverse,
                // and the zero block (T_01)^T
#pragma unroll
                for (int c4 = 0; c4 < 4; c4++)
                    *reinterpret_cast<f32x4*>(&sTtA[(16 * lq + l16) * LDT + 16 * lq + 4 * c4]) =
                        f32x4{x[4 * c4], x[4 * c4 + 1], x[4 * c4 + 2], x[4 * c4 + 3]};
                if (lq == 1) {
#pragma unroll
                    for (int c4 = 0; c4 < 4; c4++)
                        *reinterpret_cast<f32x4*>(&sTtA[(16 + l16) * LDT + 4 * c4]) = f32x4{0.f, 0.f, 0.f, 0.f};
                }
            }
            *reinterpret_cast<f32x4*>(&mt[l16 * LDM + 4 * lq]) = m;  // M^T[n][4 lq + e]
            const f32x4 t = mm16(&sT[(16 * bi + l16) * LDA + 16 * bi + kk], &mt[l16 * LDM + kk]);
#pragma unroll
            for (int e = 0; e < 4; e++) sT[(16 * bi + 4 * lq + e) * LDA + 16 * bj + l16] = -t[e];  // over A_bi,bj, read above
            if (wave == 0) *reinterpret_cast<f32x4*>(&sTtA[l16 * LDT + 16 + 4 * lq]) = -t;  // (T_10)^T
        }
        __syncthreads();  // #5

        // ---- level B: T_BA = -T_BB (A_BA T_AA) with 32 x 32 blocks; one 16 x 16 output tile per wave ----
        {
            const int ta = wave / 2, tb = wave % 2;
            const f32x4 m = mm16x32(&sA[(32 + 16 * ta + l16) * LDA + 8 * lq], &sTtA[(16 * tb + l16) * LDT + 8 * lq]);
            *reinterpret_cast<f32x4*>(&sMtB[(16 * tb + l16) * LDT + 16 * ta + 4 * lq]) = m;
            __syncthreads();  // #6
            const f32x4 t = mm16x32(&sT[(32 + 16 * ta + l16) * LDA + 32 + 8 * lq], &sMtB[(16 * tb + l16) * LDT + 8 * lq]);
#pragma unroll
            for (int e = 0; e < 4; e++) sT[(32 + 16 * ta + 4 * lq + e) * LDA + 16 * tb + l16] = -t[e];
        }
        __syncthreads();  // #7: T complete

        // ---- T diag(beta) as A operands of V~ = T' X: tiles (0, 0), (1, 0), (1, 1), two 16-token slabs each ----
        // The reduction index (token j of X) runs in the order in which an accumulator tile of the scan hands its
        // rows over as a B operand: lane half h supplies tokens 16 s + 4 h + 0..3 and 16 s + 8 + 4 h + 0..3.
        // (16x16x32 layout: fragments (tt, s) = (0,0) (1,0) (2,0) (2,1) (3,0) (3,1), 16 rows 16 tt .., lane (i, g) holds
        // columns 32 s + 4 g + 0..3 and 32 s + 16 + 4 g + 0..3: the order in which two 16 x 16 accumulator tiles hand
        // their rows over)
        for (int f = wave; f < 6; f += 4) {
            const int ti = f < 2 ? 0 : 1, tj = f < 4 ? 0 : 1, sl = f % 2;
            const int tt16 = f < 2 ? f : 2 + (f - 2) / 2, s16 = f < 2 ? 0 : f % 2;
            const int i = p.rec16 ? 16 * tt16 + l16 : 32 * ti + l32;
            const int j0 = p.rec16 ? 32 * s16 + 4 * lq : 32 * tj + 16 * sl + 4 * lh;
            const int j1 = p.rec16 ? j0 + 16 : j0 + 8;
            const f32x4 t0 = *reinterpret_cast<const f32x4*>(&sT[i * LDA + j0]);
            const f32x4 t1 = *reinterpret_cast<const f32x4*>(&sT[i * LDA + j1]);
            const f32x4 c0 = *reinterpret_cast<const f32x4*>(&s_beta[j0]);
            const f32x4 c1 = *reinterpret_cast<const f32x4*>(&s_beta[j1]);
            bf16x8 r;
#pragma unroll
            for (int e = 0; e < 4; e++) {  // sT holds the whole of T here: unit diagonal, zeros above it
                r[e] = (bf16_t)(t0[e] * c0[e]);
                r[4 + e] = (bf16_t)(t1[e] * c1[e]);
            }
            record_store<FLAGS>(rec, p.rec_bytes, (f * WAVE + lane) * 16, r);
        }
        if constexpr (FLAGS) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the record has reached memory
        __syncthreads();  // #8: LDS is reused by the next item
        if (FLAGS && tid == 0)
            __hip_atomic_store(&ready[(int64_t)h * p.TC + slot], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace gdn

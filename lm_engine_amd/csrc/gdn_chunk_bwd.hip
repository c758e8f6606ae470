// Chunk-local gradients of the gated delta rule: one workgroup per (sequence, head, chunk).
//
// What the reference's training step gets from fla's backward of chunk_gated_delta_rule
// (lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:194-209), once the two sweeps
// over the chunks have delivered, per chunk, the state it starts from (S0), the gradient of the state it ends
// with (dS1), V~ and Y = T^T dV~.  With C = 64 tokens, gamma the prefix sum of g inside the chunk,
// e = exp(gamma), tail = exp(gamma_C - gamma), E_ij = exp(gamma_i - gamma_j) (j <= i), Q already normalised and
// scaled, K normalised:
//
//     QK = Q K^T        KK = K K^T        DP = dO V~^T        DA = Y V~^T                (64 x 64)
//     P  = tril(E . QK)                   A  = stril(beta_i E . KK)
//     dP = tril(DP)     G = dP . E        dA = -stril(DA)     Hm = dA . beta_i E
//     dQe = dO S0^T     Z  = Y S0^T       dKd = V~ dS1^T                                 (64 x K)
//     dQ  = G K + diag(e) dQe
//     dK  = G^T Q + diag(tail) dKd - diag(beta e) Z + (Hm + Hm^T) K
//     dbeta_i  = -e_i <Z_i, K_i> + <Y_i, V_i> + sum_j (dA . E . KK)_ij
//     dgamma_i = rowsum(dP . P + dA . A)_i - colsum(dP . P + dA . A)_i
//                + e_i <dQe_i, Q_i> - tail_i <dKd_i, K_i> - beta_i e_i <Z_i, K_i>
//     dgamma_C += exp(gamma_C) <dS1, S0> + sum_i tail_i <dKd_i, K_i>
//
// Every matrix product is an "A B^T" of two row-major bf16 matrices staged in LDS, on 32x32x16 MFMA with fp32
// accumulation.  The 64 x K results are kept transposed ([key dim][token]) so that a lane owns one token: the
// per-token scales are per-lane scalars and the sums over the key dim stay inside a lane.
//
// Three phases share one LDS buffer of 64.5 KiB at most, so that two workgroups fit a CU and one's loads run beside
// the other's products (K <= 128; K = 256 holds its 64 x K results for both key halves in registers and takes a CU
// to itself by its register count):
//   1. over the value dim in slabs of 64 columns: dO, Y, V~ and the slab of S0, then of dS1, staged; the products
//      with the states and the two 64 x 64 products that contract over the value dim accumulate;
//   2. the rows of q and k (128 keys at a time) for Q K^T and K K^T, then the 64 x 64 stage: G, G^T and Hm + Hm^T
//      are left in LDS;
//   3. per 128 keys: the transposes of q and k (K <= 128: staged from the rows phase 2 left in LDS; K = 256: read out
//      of those rows with the transposing LDS load), the per-token sums over the key dim, dQ^T and dK^T.
// K = 256 on the sliced saves of the staging scans has one wave per SIMD and so 512 registers per lane: it asks for the
// rows of the next slab, and of the next half of q and k, while the products of the current one run, and keeps them
// in registers until their turn (PIPE below).
// K = 64, 128, 256; V a multiple of 64.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gdn_chunk32_common.h"
#include "gdn_launch.h"

namespace gdn {

namespace {

constexpr int BWD_THREADS = 256;
constexpr int LDS64 = 72;  // bf16 per LDS row of a [.][64] matrix: 16 bytes of padding

struct ChunkLocalParams {
#ifdef GDN_CYCLE_BUDGET
    uint64_t* cycle_out;  // measurement build only: where sampled workgroups report their cycles
#endif
    const void* vnew;   // V~ [chunk][64][V], fp32 or bf16 (saves_bf16)
    const void* s0;     // S0 [chunk][K][V], fp32 or bf16 (saves_bf16)
    const void* ds1;    // dS1 [chunk][K][V], fp32 or bf16 (the kernel's DS1H)
    int saves_bf16;
    const float* gam;
    const float* beta;
    const float* rq;  // 1 / |q|, 1 / |k| per token when q and k were normalised, else NULL
    const float* rk;
    float scale;
    // chunk = (n H + h) NC + c.  Y is read from the output of the scan over the mirror problem; q, k, v, dO are the
    // caller's tensors (bf16, element strides); the gradients go out in the caller's layout, [N, NC 64, H, .] bf16
    // for q, k, v and fp32 [N, NC 64, H] for g (reverse prefix sum of dgamma done here) and beta
    const bf16_t* y_mirror;  // [N][2 NC 64][H][V], or NULL and
    const bf16_t* y_chunks;  // [chunk][64][V]: Y of the chunk, tokens reversed
    const bf16_t* q_raw;
    const bf16_t* k_raw;
    const bf16_t* v_raw;
    const bf16_t* d_raw;
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    int64_t d_stride_b, d_stride_t, d_stride_h;
    bf16_t* dq_out;
    bf16_t* dk_out;
    bf16_t* dv_out;
    float* dg_out;
    float* dbeta_out;
    int H, NC, V;
    // sequences that are not whole rows of whole chunks (packed or left-padded batches): first token (flat index
    // over the rows of the caller's tensors) and length of every sequence; NULL = sequence n is row n
    const int32_t* seq_start;
    const int32_t* seq_len;
    int T_rows;  // tokens per row of the caller's tensors
};

// acc[r] += sum_k A[8 (r/4) + 4 h + r%4][k] B[l32][k] over k < kd: A, B point at the first of 32 rows
__device__ __forceinline__ f32x16 mma_nt(const bf16_t* A, int lda, const bf16_t* B, int ldb, int kd, f32x16 acc, int l32, int lh) {
    for (int kk = 0; kk < kd; kk += 16) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(A + l32 * lda + kk + 8 * lh);
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(B + l32 * ldb + kk + 8 * lh);
        acc = mfma32_bf16(a, b, acc);
    }
    return acc;
}

// acc[r] += sum_t M[t][col0 + 8 (r/4) + 4 h + r%4] B[l32][t] over t < kd: the A operand is the transpose of 32 columns of
// the row-major matrix M, read through the transposing LDS load (4 tokens x 16 columns per instruction)
__device__ __forceinline__ f32x16 mma_tn(const bf16_t* M, int ldm, int col0, const bf16_t* B, int ldb, int kd, f32x16 acc, int l32, int lh) {
    const int l16 = l32 % 16, g16 = l32 / 16;
    for (int kk = 0; kk < kd; kk += 16) {
        const bf16x4 lo = lds_read_tr4x16<false>(M, ldm, kk + 8 * lh, col0 + 16 * g16, l16);
        const bf16x4 hi = lds_read_tr4x16<false>(M, ldm, kk + 8 * lh + 4, col0 + 16 * g16, l16);
        bf16x8 a;
#pragma unroll
        for (int e = 0; e < 4; e++) a[e] = lo[e], a[4 + e] = hi[e];
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(B + l32 * ldb + kk + 8 * lh);
        acc = mfma32_bf16(a, b, acc);
    }
    return acc;
}

// acc[r] += sum_t A[8 (r/4) + 4 h + r%4][t] M[t][col0 + l32] over t < kd: the B operand is the transpose of 32 columns of the
// row-major matrix M (same transposing loads as mma_tn, on the other operand)
__device__ __forceinline__ f32x16 mma_nn(const bf16_t* A, int lda, const bf16_t* M, int ldm, int col0, int kd, f32x16 acc, int l32, int lh) {
    const int l16 = l32 % 16, g16 = l32 / 16;
    for (int kk = 0; kk < kd; kk += 16) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(A + l32 * lda + kk + 8 * lh);
        const bf16x4 lo = lds_read_tr4x16<false>(M, ldm, kk + 8 * lh, col0 + 16 * g16, l16);
        const bf16x4 hi = lds_read_tr4x16<false>(M, ldm, kk + 8 * lh + 4, col0 + 16 * g16, l16);
        bf16x8 b;
#pragma unroll
        for (int e = 0; e < 4; e++) b[e] = lo[e], b[4 + e] = hi[e];
        acc = mfma32_bf16(a, b, acc);
    }
    return acc;
}

// Sixteen sums over the 32 lanes of a wave half at once: on return every lane holds the sum of x[l32 / 2].  Each
// exchange halves the number of values a lane carries (16 shuffles instead of 80).
__device__ __forceinline__ float half_sums16(const float (&x)[16], int l32) {
    float y[8], z[4], w[2];
    const bool b4 = l32 & 16, b3 = l32 & 8, b2 = l32 & 4, b1 = l32 & 2;
#pragma unroll
    for (int e = 0; e < 8; e++) y[e] = (b4 ? x[8 + e] : x[e]) + __shfl_xor(b4 ? x[e] : x[8 + e], 16, WAVE);
#pragma unroll
    for (int e = 0; e < 4; e++) z[e] = (b3 ? y[4 + e] : y[e]) + __shfl_xor(b3 ? y[e] : y[4 + e], 8, WAVE);
#pragma unroll
    for (int e = 0; e < 2; e++) w[e] = (b2 ? z[2 + e] : z[e]) + __shfl_xor(b2 ? z[e] : z[2 + e], 4, WAVE);
    float u = (b1 ? w[1] : w[0]) + __shfl_xor(b1 ? w[0] : w[1], 2, WAVE);
    return u + __shfl_xor(u, 1, WAVE);
}

__device__ __forceinline__ void put4(bf16_t* dst, f32x4 x) {
    bf16x4 r;
    r.x = (bf16_t)x.x, r.y = (bf16_t)x.y, r.z = (bf16_t)x.z, r.w = (bf16_t)x.w;
    *reinterpret_cast<bf16x4*>(dst) = r;
}

constexpr int cmax(int a, int b) { return a > b ? a : b; }

// element (row, column c) of a [rows][V] array laid out by groups of 8 rows and, within a group, by 32-column slice
__device__ __forceinline__ int sliced_at(int row, int c, int rows) { return (c / 32) * rows * 32 + row * 32 + c % 32; }

// DS1H: dS1 comes as bf16 (fp32 otherwise); SL: V~, S0, dS1 and Y lie in the sliced layout of the staging scans (all bf16)
template <int K, bool DS1H, bool SL>
__global__ __launch_bounds__(BWD_THREADS, (K <= 128 ? 2 : 1)) void chunk_local_grads_kernel(const ChunkLocalParams p) {
    const int V = p.V;
    constexpr int VW = 64;                     // columns of the value dim staged at a time
    constexpr int KW = K < 128 ? K : 128;      // keys staged at a time in phases 2 and 3
    constexpr int KH = K / KW;                 // key halves: 1 or 2
    constexpr int LDK = KW + 8;                // bf16 per LDS row of a [.][KW] matrix
    constexpr int NKT = KW / 32;               // key tiles per half: 2 or 4
    // wave -> 32-key tile of every half and token tiles: with four key tiles a wave has one of them and both token
    // tiles, with two (K = 64) a quarter each
    constexpr int NTW = NKT == 4 ? 2 : 1;
    static_assert(K == 64 || K == 128 || K == 256, "head dims");
    constexpr int SLAB = C * LDS64 * 2;        // bytes of a staged [64][64] matrix
    constexpr int PHASE1 = 3 * SLAB + K * LDS64 * 2;        // dO | Y | V~ | states
    constexpr int PHASE2 = 3 * SLAB + 2 * C * LDK * 2;      // G | G^T | Hm + Hm^T | q | k
    // Phase 3 needs q^T and k^T as MFMA operands.  K = 256 (a CU to itself) reads them out of the row-major copies with
    // the transposing LDS load; with two workgroups per CU (K <= 128) that variant ran slower (more registers, spills)
    // than staging the transposes once more, 2 bytes at a time.
    constexpr bool TR = K > 128;
    constexpr int PHASE3 = TR ? PHASE2 : 3 * SLAB + 2 * KW * LDS64 * 2;  // G | G^T | Hm + Hm^T | q^T | k^T
    constexpr int LDS_BYTES = cmax(PHASE1, cmax(PHASE2, PHASE3));
    __shared__ __attribute__((aligned(16))) uint8_t lds[LDS_BYTES];
    __shared__ float s_gam[C], s_beta[C], s_e[C], s_tail[C], s_dgam[C], s_dbeta[C], s_dotq[C], s_dotk[C], s_fq[C], s_fk[C], s_red[4];
    bf16_t* const sDO = reinterpret_cast<bf16_t*>(lds);
    bf16_t* const sY = sDO + C * LDS64;
    bf16_t* const sVN = sY + C * LDS64;
    bf16_t* const sST = sVN + C * LDS64;  // [K][LDS64]: S0, then dS1
    bf16_t* const sG = reinterpret_cast<bf16_t*>(lds);
    bf16_t* const sGT = sG + C * LDS64;
    bf16_t* const sH = sGT + C * LDS64;
    bf16_t* const sQ = sH + C * LDS64;    // phase 2 (and 3 with TR): [64][LDK]
    bf16_t* const sK = sQ + C * LDK;
    bf16_t* const sQT = sH + C * LDS64;   // phase 3 without TR: [KW][LDS64]
    bf16_t* const sKT = sQT + KW * LDS64;

    const int t = threadIdx.x;
    const int lane = t % WAVE, wave = t / WAVE;
    const int l32 = lane % 32, lh = lane / 32;
    const int ktl = NKT == 4 ? wave : wave % 2;              // this wave's key tile within a half
    auto tt_of = [&](int m) { return NTW == 2 ? m : wave / 2; };  // its token tiles
    const int64_t chunk = blockIdx.x;
    const int ci = (int)(chunk % p.NC);
    const int chain = (int)(chunk / p.NC);
    const int n = chain / p.H, h = chain % p.H;
    // first token of the chunk as a flat index over the rows of the caller's tensors, and its number of tokens
    int valid = C;
    int64_t tok0;
    if (p.seq_start != nullptr) {
        valid = min(max(p.seq_len[n] - ci * C, 0), C);
        tok0 = (int64_t)p.seq_start[n] + (int64_t)ci * C;
    } else {
        tok0 = (int64_t)n * p.T_rows + (int64_t)ci * C;
    }
    if (valid == 0) return;  // a chunk past the end of its sequence (whole workgroup)
    const int64_t mirA = ((int64_t)n * p.NC + (p.NC - 1 - ci)) * 2 * C;  // first token of mirror chunk A
    // row `row` of the chunk in one of the caller's tensors (a chunk lies within one row of the batch); rows past the
    // end of the sequence read its last token and are zeroed
    const int64_t row_b = tok0 / p.T_rows, row_t = tok0 % p.T_rows;
    auto row_of = [&](const bf16_t* base, int64_t sb, int64_t st, int64_t sh, int row) -> const bf16_t* {
        return base + row_b * sb + (row_t + min(row, valid - 1)) * st + (int64_t)h * sh;
    };
    bf16x8 zero8;
#pragma unroll
    for (int e = 0; e < 8; e++) zero8[e] = (bf16_t)0.f;
    f32x16 zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.f;

    if (t < C) {
        const float g = p.gam[chunk * C + t];
        s_gam[t] = g;
        s_beta[t] = p.beta[chunk * C + t];
        s_e[t] = __expf(g);
        s_tail[t] = __expf(p.gam[chunk * C + C - 1] - g);
        s_dgam[t] = 0.f;
        s_dbeta[t] = 0.f;
        s_dotq[t] = 0.f;
        s_dotk[t] = 0.f;
        s_fq[t] = (p.rq != nullptr ? p.rq[chunk * C + t] : 1.f) * p.scale;  // q and k rows are scaled on their way into LDS
        s_fk[t] = p.rk != nullptr ? p.rk[chunk * C + t] : 1.f;
    }
    if (t < 4) s_red[t] = 0.f;
#ifdef GDN_CYCLE_BUDGET
    // Measurement build (python -m lm_engine_amd.build --cycle-budget): wave 0 reads the shader clock between the steps
    // of the kernel and adds the cycles of each up; sampled workgroups report at the end (the steps are named in bench.py's LOCAL_GROUPS).
    uint64_t cyc[16] = {};
    uint64_t cyc_t0 = __builtin_readcyclecounter();
    auto ltick = [&](int g) {
        const uint64_t t1 = __builtin_readcyclecounter();
        cyc[g] += t1 - cyc_t0;
        cyc_t0 = t1;
        __builtin_amdgcn_sched_barrier(0);
    };
#define LTICK(g) ltick(g)
#else
#define LTICK(g)
#endif

    // ---------------- phase 1: everything that contracts over the value dim, 64 columns at a time ----------------
    // products with the states, transposed: rows = keys 32 (ktl + NKT kh) .., columns = tokens 32 tt + l32; and the
    // 64 x 64 products dO V~^T and Y V~^T (wave -> tile (wave / 2, wave % 2))
    f32x16 dQeT[KH][NTW], ZT[KH][NTW], dKdT[KH][NTW], DP = zero, DA = zero;
#pragma unroll
    for (int kh = 0; kh < KH; kh++)
#pragma unroll
        for (int m = 0; m < NTW; m++) dQeT[kh][m] = zero, ZT[kh][m] = zero, dKdT[kh][m] = zero;
    const char* const s0b = static_cast<const char*>(p.s0) + chunk * K * (int64_t)V * (p.saves_bf16 ? 2 : 4);
    const char* const vnb = static_cast<const char*>(p.vnew) + chunk * C * (int64_t)V * (p.saves_bf16 ? 2 : 4);
    const float* const ds1 = static_cast<const float*>(p.ds1) + chunk * K * (int64_t)V;         // when fp32
    const bf16_t* const ds1h = static_cast<const bf16_t*>(p.ds1) + chunk * K * (int64_t)V;    // when bf16
    constexpr int SROWS = K / 16;  // 16-byte fp32 pieces of a state slab per thread: K rows x 16 pieces
    float dot = 0.f;
    // K = 256 on the sliced bf16 saves (a CU to itself: one wave per SIMD, 512 registers each): the rows of the next
    // slab are asked for while the products of this one run and wait in registers, so that no trip through memory
    // stands between a slab's barriers.
    constexpr bool PIPE = SL && K > 128;
    bf16x8 nx_v[PIPE ? 2 : 1], nx_d[PIPE ? 2 : 1], nx_y[PIPE ? 2 : 1], nx_vn[PIPE ? 2 : 1], nx_s0[TR ? K / 32 : 1];  // nx_s0: also q and k on their way into LDS
    auto ask_slab = [&](int v0) {
        const int p8 = t % 8;
        const bf16_t* vnew = reinterpret_cast<const bf16_t*>(vnb);
        const bf16_t* s0 = reinterpret_cast<const bf16_t*>(s0b);
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int row = t / 8 + 32 * it;
            nx_v[it] = *reinterpret_cast<const bf16x8*>(row_of(p.v_raw, p.v_stride_b, p.v_stride_t, p.v_stride_h, row) + v0 + 8 * p8);
            nx_d[it] = *reinterpret_cast<const bf16x8*>(row_of(p.d_raw, p.d_stride_b, p.d_stride_t, p.d_stride_h, row) + v0 + 8 * p8);
            nx_y[it] = *reinterpret_cast<const bf16x8*>(p.y_chunks + chunk * C * V + sliced_at(C - 1 - row, v0 + 8 * p8, C));
            nx_vn[it] = *reinterpret_cast<const bf16x8*>(vnew + sliced_at(row, v0 + 8 * p8, C));
        }
#pragma unroll
        for (int i = 0; i < K / 32; i++) nx_s0[i] = *reinterpret_cast<const bf16x8*>(s0 + sliced_at(t / 8 + 32 * i, v0 + 8 * p8, K));
    };
    // rows of q and k (keys KW kh ..) into registers, and from there, scaled, row-major into sQ and sK (TR only)
    auto ask_qk = [&](int kh) {
        constexpr int CPR = KW / 8, RPP = BWD_THREADS / CPR;  // 16-byte pieces per staged row, rows per pass
        int tl = t;
        asm volatile("" : "+v"(tl));  // the row addresses are formed here, not ahead of phase 1 (where they would be spilled)
        const int p8 = tl % CPR;
#pragma unroll
        for (int it = 0; it < C / RPP; it++) {
            const int row = tl / CPR + RPP * it;
            nx_s0[2 * it] = *reinterpret_cast<const bf16x8*>(row_of(p.q_raw, p.q_stride_b, p.q_stride_t, p.q_stride_h, row) + KW * kh + 8 * p8);
            nx_s0[2 * it + 1] = *reinterpret_cast<const bf16x8*>(row_of(p.k_raw, p.k_stride_b, p.k_stride_t, p.k_stride_h, row) + KW * kh + 8 * p8);
        }
    };
    auto put_qk = [&]() {
        constexpr int CPR = KW / 8, RPP = BWD_THREADS / CPR;
        const int p8 = t % CPR;
#pragma unroll
        for (int it = 0; it < C / RPP; it++) {
            const int row = t / CPR + RPP * it;
            const bool live = row < valid;
            const float fq = live ? s_fq[row] : 0.f, fk = live ? s_fk[row] : 0.f;
            bf16x8 qb, kb;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                qb[e] = (bf16_t)((float)nx_s0[2 * it][e] * fq);
                kb[e] = (bf16_t)((float)nx_s0[2 * it + 1][e] * fk);
            }
            *reinterpret_cast<bf16x8*>(sQ + row * LDK + 8 * p8) = qb;
            *reinterpret_cast<bf16x8*>(sK + row * LDK + 8 * p8) = kb;
        }
    };
    if constexpr (PIPE) ask_slab(0);
#pragma unroll 1
    for (int hv = 0; hv < V / VW; hv++) {
        const int v0 = VW * hv;
        float yv[2];  // <Y_i, V_i> pieces, reduced after the barrier (s_dbeta is cleared before the first one)
        if constexpr (PIPE) {
            const int p8 = t % 8;
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const int row = t / 8 + 32 * it;
                const bool live = row < valid;
                const bf16x8 vr = live ? nx_v[it] : zero8, dr = live ? nx_d[it] : zero8, yr = nx_y[it];
                const float b = p.beta[chunk * C + row];
                bf16x8 dv;
                float acc = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    dv[e] = (bf16_t)((float)yr[e] * b);
                    acc += (float)yr[e] * (float)vr[e];
                }
                *reinterpret_cast<bf16x8*>(sDO + row * LDS64 + 8 * p8) = dr;
                *reinterpret_cast<bf16x8*>(sY + row * LDS64 + 8 * p8) = yr;
                *reinterpret_cast<bf16x8*>(sVN + row * LDS64 + 8 * p8) = live ? nx_vn[it] : zero8;
                if (live) *reinterpret_cast<bf16x8*>(p.dv_out + ((tok0 + row) * p.H + h) * V + v0 + 8 * p8) = dv;
                yv[it] = acc;
            }
#pragma unroll
            for (int i = 0; i < K / 32; i++) *reinterpret_cast<bf16x8*>(sST + (t / 8 + 32 * i) * LDS64 + 8 * p8) = nx_s0[i];
        } else {
            // v, dO and Y (token `row` is token 63 - row of mirror chunk A); dV = beta Y goes out right away
            const int p8 = t % 8;
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const int row = t / 8 + 32 * it;
                const bool live = row < valid;
                bf16x8 vr = *reinterpret_cast<const bf16x8*>(row_of(p.v_raw, p.v_stride_b, p.v_stride_t, p.v_stride_h, row) + v0 + 8 * p8);
                bf16x8 dr = *reinterpret_cast<const bf16x8*>(row_of(p.d_raw, p.d_stride_b, p.d_stride_t, p.d_stride_h, row) + v0 + 8 * p8);
                if (!live) vr = zero8, dr = zero8;
                const bf16_t* yrow;
                if constexpr (SL) yrow = p.y_chunks + chunk * C * V + sliced_at(C - 1 - row, v0 + 8 * p8, C);
                else yrow = p.y_mirror != nullptr ? p.y_mirror + ((mirA + (C - 1 - row)) * p.H + h) * V + v0 + 8 * p8
                                                  : p.y_chunks + (chunk * C + (C - 1 - row)) * V + v0 + 8 * p8;
                const bf16x8 yr = *reinterpret_cast<const bf16x8*>(yrow);
                const float b = p.beta[chunk * C + row];
                bf16x8 dv;
                float acc = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    dv[e] = (bf16_t)((float)yr[e] * b);
                    acc += (float)yr[e] * (float)vr[e];
                }
                *reinterpret_cast<bf16x8*>(sDO + row * LDS64 + 8 * p8) = dr;
                *reinterpret_cast<bf16x8*>(sY + row * LDS64 + 8 * p8) = yr;
                if (live) *reinterpret_cast<bf16x8*>(p.dv_out + ((tok0 + row) * p.H + h) * V + v0 + 8 * p8) = dv;
                yv[it] = acc;
            }
            if (p.saves_bf16) {
                const bf16_t* vnew = reinterpret_cast<const bf16_t*>(vnb);
#pragma unroll
                for (int it = 0; it < 2; it++) {  // rows of V~ past the end of the sequence hold whatever the scan left
                    const int row = t / 8 + 32 * it;
                    const bf16x8 x = *reinterpret_cast<const bf16x8*>(SL ? vnew + sliced_at(row, v0 + 8 * p8, C)
                                                                                : vnew + row * V + v0 + 8 * p8);
                    *reinterpret_cast<bf16x8*>(sVN + row * LDS64 + 8 * p8) = row < valid ? x : zero8;
                }
                const bf16_t* s0 = reinterpret_cast<const bf16_t*>(s0b);
#pragma unroll
                for (int i = 0; i < K / 32; i++) {  // S0[:, v0 .. v0 + 63]: row = 32 i + t / 8
                    const int row = t / 8 + 32 * i;
                    *reinterpret_cast<bf16x8*>(sST + row * LDS64 + 8 * p8) =
                        *reinterpret_cast<const bf16x8*>(SL ? s0 + sliced_at(row, v0 + 8 * p8, K) : s0 + row * V + v0 + 8 * p8);
                }
            } else {
                const float* vnew = reinterpret_cast<const float*>(vnb);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int idx = t + BWD_THREADS * i, row = idx / 16, c4 = idx % 16;
                    const f32x4 x = *reinterpret_cast<const f32x4*>(vnew + row * V + v0 + 4 * c4);
                    put4(sVN + row * LDS64 + 4 * c4, row < valid ? x : f32x4{0.f, 0.f, 0.f, 0.f});
                }
                const float* s0 = reinterpret_cast<const float*>(s0b);
#pragma unroll
                for (int i = 0; i < SROWS; i++) {  // S0[:, v0 .. v0 + 63] fp32: row = 16 i + t / 16
                    const int idx = t + BWD_THREADS * i, row = idx / 16, c4 = idx % 16;
                    put4(sST + row * LDS64 + 4 * c4, *reinterpret_cast<const f32x4*>(s0 + row * V + v0 + 4 * c4));
                }
            }
        }
        LTICK(0);
        __syncthreads();
        LTICK(1);
#pragma unroll
        for (int it = 0; it < 2; it++) {  // 8 lanes hold one row
            float x = yv[it];
#pragma unroll
            for (int off = 4; off >= 1; off >>= 1) x += __shfl_xor(x, off, WAVE);
            if (t % 8 == 0) atomicAdd(&s_dbeta[t / 8 + 32 * it], x);
        }

        // K = 256 (a CU to itself, registers to spare): dS1 of this slab is asked for now and stays in registers while the
        // products with S0 run, so that its trip through memory is behind them instead of in front of the barrier below.
        // With two workgroups per CU the other one's products fill that wait, and the registers are needed.
        constexpr bool PREFETCH = K > 128;
        f32x4 ds1_rows[DS1H ? 1 : SROWS];     // fp32 dS1: 16 pieces of 16 bytes per row of the slab
        bf16x8 ds1_half[DS1H ? K / 32 : 1];   // bf16 dS1: 8 pieces per row, as for S0
        auto ask_ds1 = [&]() {
            if constexpr (DS1H) {
#pragma unroll
                for (int i = 0; i < K / 32; i++) {
                    const int row = t / 8 + 32 * i, c8 = 8 * (t % 8);
                    ds1_half[i] = *reinterpret_cast<const bf16x8*>(SL ? ds1h + sliced_at(row, v0 + c8, K) : ds1h + row * V + v0 + c8);
                }
            } else {
#pragma unroll
                for (int i = 0; i < SROWS; i++) {
                    const int idx = t + BWD_THREADS * i, row = idx / 16, c4 = idx % 16;
                    ds1_rows[i] = *reinterpret_cast<const f32x4*>(ds1 + row * V + v0 + 4 * c4);
                }
            }
        };
        LTICK(2);
        if constexpr (PREFETCH) {
            ask_ds1();  // first: it is waited for first
            LTICK(3);
            if constexpr (PIPE) {
                if (hv + 1 < V / VW) ask_slab(v0 + VW);
                else ask_qk(0);
            }
            __builtin_amdgcn_sched_barrier(0);
            LTICK(4);
        }
#pragma unroll
        for (int kh = 0; kh < KH; kh++)
#pragma unroll
            for (int m = 0; m < NTW; m++) {
                const bf16_t* srows = sST + 32 * (ktl + NKT * kh) * LDS64;
                dQeT[kh][m] = mma_nt(srows, LDS64, sDO + 32 * tt_of(m) * LDS64, LDS64, VW, dQeT[kh][m], l32, lh);
                ZT[kh][m] = mma_nt(srows, LDS64, sY + 32 * tt_of(m) * LDS64, LDS64, VW, ZT[kh][m], l32, lh);
            }
        DP = mma_nt(sDO + 32 * (wave / 2) * LDS64, LDS64, sVN + 32 * (wave % 2) * LDS64, LDS64, VW, DP, l32, lh);
        DA = mma_nt(sY + 32 * (wave / 2) * LDS64, LDS64, sVN + 32 * (wave % 2) * LDS64, LDS64, VW, DA, l32, lh);
        if constexpr (!PREFETCH) ask_ds1();
        LTICK(5);
        __syncthreads();  // S0 has been read by every wave
        LTICK(6);

        // dS1 takes the place of S0; <dS1, S0> on the way (S0 as the bf16 the products used)
        if constexpr (DS1H) {
#pragma unroll
            for (int i = 0; i < K / 32; i++) {
                bf16_t* const at = sST + (t / 8 + 32 * i) * LDS64 + 8 * (t % 8);
                const bf16x8 sv = *reinterpret_cast<const bf16x8*>(at);
#pragma unroll
                for (int e = 0; e < 8; e++) dot += (float)ds1_half[i][e] * (float)sv[e];
                *reinterpret_cast<bf16x8*>(at) = ds1_half[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < SROWS; i++) {
                const int idx = t + BWD_THREADS * i, row = idx / 16, c4 = idx % 16;
                const f32x4 x = ds1_rows[i];
                const bf16x4 sv = *reinterpret_cast<const bf16x4*>(sST + row * LDS64 + 4 * c4);
                dot += x.x * (float)sv.x + x.y * (float)sv.y + x.z * (float)sv.z + x.w * (float)sv.w;
                put4(sST + row * LDS64 + 4 * c4, x);
            }
        }
        LTICK(7);
        __syncthreads();
        LTICK(8);
#pragma unroll
        for (int kh = 0; kh < KH; kh++)
#pragma unroll
            for (int m = 0; m < NTW; m++)
                dKdT[kh][m] = mma_nt(sST + 32 * (ktl + NKT * kh) * LDS64, LDS64, sVN + 32 * tt_of(m) * LDS64, LDS64, VW, dKdT[kh][m], l32, lh);
        LTICK(9);
        __syncthreads();  // the staged slab is free
        LTICK(10);
    }
    dot = wave_sum(dot);
    if (lane == 0) atomicAdd(&s_red[0], dot);

    LTICK(11);
    // ---------------- phase 2: Q K^T, K K^T and the 64 x 64 stage ----------------
    // wave -> tile (ti, tj); rows i = 32 ti + 8 (r/4) + 4 h + r%4, column j = 32 tj + l32
    {
        const int ti = wave / 2, tj = wave % 2;
        f32x16 QK = zero, KK = zero;
#pragma unroll
        for (int kh = 0; kh < KH; kh++) {
            if (kh > 0) __syncthreads();  // the products of the previous half have read q and k
            if constexpr (TR) {
                if constexpr (!PIPE) {
                    if (kh == 0) ask_qk(0);
                }
                put_qk();
            } else {
                constexpr int CPR = KW / 8, RPP = BWD_THREADS / CPR;
                const int p8 = t % CPR;
#pragma unroll
                for (int it = 0; it < C / RPP; it++) {
                    const int row = t / CPR + RPP * it;
                    bf16x8 qr = *reinterpret_cast<const bf16x8*>(row_of(p.q_raw, p.q_stride_b, p.q_stride_t, p.q_stride_h, row) + KW * kh + 8 * p8);
                    bf16x8 kr = *reinterpret_cast<const bf16x8*>(row_of(p.k_raw, p.k_stride_b, p.k_stride_t, p.k_stride_h, row) + KW * kh + 8 * p8);
                    if (row >= valid) qr = zero8, kr = zero8;
                    const float fq = s_fq[row], fk = s_fk[row];
                    bf16x8 qb, kb;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        qb[e] = (bf16_t)((float)qr[e] * fq);
                        kb[e] = (bf16_t)((float)kr[e] * fk);
                    }
                    *reinterpret_cast<bf16x8*>(sQ + row * LDK + 8 * p8) = qb;
                    *reinterpret_cast<bf16x8*>(sK + row * LDK + 8 * p8) = kb;
                }
            }
            __syncthreads();
            if constexpr (TR) {  // the rows staged next travel while these products run: the other half, then half 0 again for phase 3
                ask_qk(kh + 1 < KH ? kh + 1 : 0);
                __builtin_amdgcn_sched_barrier(0);
            }
            QK = mma_nt(sQ + 32 * ti * LDK, LDK, sK + 32 * tj * LDK, LDK, KW, QK, l32, lh);
            KK = mma_nt(sK + 32 * ti * LDK, LDK, sK + 32 * tj * LDK, LDK, KW, KK, l32, lh);
        }
        const int j = 32 * tj + l32;
        const float gj = s_gam[j];
        float colsum = 0.f;
        float rowm[16], rowb[16];  // this lane's terms of the row sums for dgamma and dbeta
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int i = 32 * ti + 8 * (r / 4) + 4 * lh + r % 4;
            const float bi = s_beta[i];
            const float E = i >= j ? __expf(s_gam[i] - gj) : 0.f;
            const float dP = i >= j ? DP[r] : 0.f;
            const float dA = i > j ? -DA[r] : 0.f;
            const float Pm = E * QK[r];
            const float Am = i > j ? bi * E * KK[r] : 0.f;
            const float G = dP * E;
            const float Hm = dA * bi * E;
            const float m = dP * Pm + dA * Am;
            colsum += m;
            rowm[r] = m;
            rowb[r] = dA * E * KK[r];
            sG[i * LDS64 + j] = (bf16_t)G;
            sGT[j * LDS64 + i] = (bf16_t)G;
            if (i > j) {
                sH[i * LDS64 + j] = (bf16_t)Hm;
                sH[j * LDS64 + i] = (bf16_t)Hm;
            } else if (i == j) {
                sH[i * LDS64 + i] = (bf16_t)0.f;
            }
        }
        {
            const float sm = half_sums16(rowm, l32), sb = half_sums16(rowb, l32);
            const int r = l32 / 2;
            const int i = 32 * ti + 8 * (r / 4) + 4 * lh + r % 4;
            if (l32 % 2 == 0) {
                atomicAdd(&s_dgam[i], sm);
                atomicAdd(&s_dbeta[i], sb);
            }
        }
        atomicAdd(&s_dgam[j], -colsum);
    }
    LTICK(12);
    // K <= 128: the transposes of phase 3 take the place of the rows of q and k in LDS; every thread picks its pieces of
    // the rows up here, before the barrier that ends their use
    bf16x8 tq[TR ? 1 : KW / 32], tk[TR ? 1 : KW / 32];
    if constexpr (!TR) {
        static_assert(TR || KH == 1, "one staging of q and k");
#pragma unroll
        for (int it = 0; it < KW / 32; it++) {
            const int row = t % C, p8 = t / C + 4 * it;
            tq[it] = *reinterpret_cast<const bf16x8*>(sQ + row * LDK + 8 * p8);
            tk[it] = *reinterpret_cast<const bf16x8*>(sK + row * LDK + 8 * p8);
        }
    }
    // ---------------- phase 3: per-token sums over the key dim, dQ^T and dK^T, 128 keys at a time ----------------
    // (dQ^T and dK^T are built in the registers of dQe^T and dKd^T)
    float nkd = 0.f;
    auto& accq = dQeT;
    auto& acck = dKdT;
    bf16x8 qv[KH][NTW][2], kv[KH][NTW][2];  // this lane's entries of q and k, kept for the backward of the normalisation
#pragma unroll
    for (int kx = 0; kx < KH; kx++) {
        const int kh = TR ? KH - 1 - kx : kx;  // TR: the half that phase 2 staged last is still there
        __syncthreads();  // G, G^T, Hm + Hm^T are complete (or: the previous half's reads are over)
        if constexpr (TR) {
            if (kx > 0) {
                put_qk();
                __syncthreads();
            }
        } else {
            // a wave takes 16 bytes of all 64 rows at a time: its 2-byte writes of one key then cover 64 consecutive
            // tokens of a transposed row (no bank conflicts; the rows themselves come out of the cache)
            // (the values are the scaled rows that phase 2 staged, taken out of LDS before the barrier above)
            constexpr int CPR = KW / 8;
            const int row = t % C;
#pragma unroll
            for (int it = 0; it < CPR / 4; it++) {
                const int p8 = t / C + 4 * it;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    sQT[(8 * p8 + e) * LDS64 + row] = tq[it][e];
                    sKT[(8 * p8 + e) * LDS64 + row] = tk[it][e];
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int m = 0; m < NTW; m++) {
            const int tt = tt_of(m);
            const int i = 32 * tt + l32;
            const float ei = s_e[i], tl = s_tail[i], bi = s_beta[i];
            float s_qe = 0.f, s_kd = 0.f, s_zk = 0.f;
            if constexpr (TR) {
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {  // keys 32 ktl + 8 r4 + 4 h + 0..3 of token i
                    const bf16x4 q4 = *reinterpret_cast<const bf16x4*>(sQ + i * LDK + 32 * ktl + 8 * r4 + 4 * lh);
                    const bf16x4 k4 = *reinterpret_cast<const bf16x4*>(sK + i * LDK + 32 * ktl + 8 * r4 + 4 * lh);
#pragma unroll
                    for (int e = 0; e < 4; e++) qv[kh][m][r4 / 2][4 * (r4 % 2) + e] = q4[e], kv[kh][m][r4 / 2][4 * (r4 % 2) + e] = k4[e];
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int d = 32 * ktl + 8 * (r / 4) + 4 * lh + r % 4;
                    qv[kh][m][r / 8][r % 8] = sQT[d * LDS64 + i], kv[kh][m][r / 8][r % 8] = sKT[d * LDS64 + i];
                }
            }
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const bf16_t qe = qv[kh][m][r / 8][r % 8], ke = kv[kh][m][r / 8][r % 8];
                s_qe += dQeT[kh][m][r] * (float)qe;
                s_kd += dKdT[kh][m][r] * (float)ke;
                s_zk += ZT[kh][m][r] * (float)ke;
            }
            atomicAdd(&s_dgam[i], ei * s_qe - tl * s_kd - bi * ei * s_zk);
            atomicAdd(&s_dbeta[i], -ei * s_zk);
            nkd += tl * s_kd;

#pragma unroll
            for (int r = 0; r < 16; r++) {
                accq[kh][m][r] *= ei;
                acck[kh][m][r] = acck[kh][m][r] * tl - ZT[kh][m][r] * (bi * ei);
            }
            if constexpr (TR) {
                accq[kh][m] = mma_tn(sK, LDK, 32 * ktl, sG + 32 * tt * LDS64, LDS64, C, accq[kh][m], l32, lh);
                acck[kh][m] = mma_tn(sQ, LDK, 32 * ktl, sGT + 32 * tt * LDS64, LDS64, C, acck[kh][m], l32, lh);
                acck[kh][m] = mma_tn(sK, LDK, 32 * ktl, sH + 32 * tt * LDS64, LDS64, C, acck[kh][m], l32, lh);
            } else {
                accq[kh][m] = mma_nt(sKT + 32 * ktl * LDS64, LDS64, sG + 32 * tt * LDS64, LDS64, C, accq[kh][m], l32, lh);
                acck[kh][m] = mma_nt(sQT + 32 * ktl * LDS64, LDS64, sGT + 32 * tt * LDS64, LDS64, C, acck[kh][m], l32, lh);
                acck[kh][m] = mma_nt(sKT + 32 * ktl * LDS64, LDS64, sH + 32 * tt * LDS64, LDS64, C, acck[kh][m], l32, lh);
            }
            if (p.rq != nullptr) {  // <dQs_i, Qs_i> and <dK_i, K_i> for the backward of the normalisation
                float dq_q = 0.f, dk_k = 0.f;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    dq_q += accq[kh][m][r] * (float)qv[kh][m][r / 8][r % 8];
                    dk_k += acck[kh][m][r] * (float)kv[kh][m][r / 8][r % 8];
                }
                atomicAdd(&s_dotq[i], dq_q);
                atomicAdd(&s_dotk[i], dk_k);
            }
        }
    }
    LTICK(13);
    nkd = wave_sum(nkd);
    if (lane == 0) atomicAdd(&s_red[1], nkd);
    __syncthreads();

    // With x = y / r the normalised row (y: input, r = |y|^-1 incl. epsilon): dy = r (dx - x <x, dx>); the scale of
    // q moves through: Qs = scale Qn, so dQn = scale dQs and Qn <Qn, dQn> = Qs <Qs, dQs> / scale.
#pragma unroll
    for (int kh = 0; kh < KH; kh++)
#pragma unroll
        for (int m = 0; m < NTW; m++) {
            const int i = 32 * tt_of(m) + l32;
            const int64_t at = ((tok0 + i) * p.H + h) * K + KW * kh + 32 * ktl + 4 * lh;
            const bool norm = p.rq != nullptr;
            const float rq = norm ? p.rq[chunk * C + i] : 1.f, rk = norm ? p.rk[chunk * C + i] : 1.f;
            const float cq = norm ? s_dotq[i] / p.scale : 0.f, ck = norm ? s_dotk[i] : 0.f;
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                f32x4 oq, ok;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int r = 4 * r4 + e;
                    oq[e] = rq * (accq[kh][m][r] * p.scale - cq * (float)qv[kh][m][r / 8][r % 8]);
                    ok[e] = rk * (acck[kh][m][r] - ck * (float)kv[kh][m][r / 8][r % 8]);
                }
                if (i < valid) {
                    store4<bf16_t>(p.dq_out + at + 8 * r4, oq);
                    store4<bf16_t>(p.dk_out + at + 8 * r4, ok);
                }
            }
        }

    if (t < C) {  // wave 0
        float dg = s_dgam[t];
        if (t == C - 1) dg += s_e[C - 1] * s_red[0] + s_red[1];
        // dg_t = sum of dgamma over the tokens t .. 63 of the chunk
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
            const float y = __shfl_down(dg, off, WAVE);
            if (t + off < C) dg += y;
        }
        if (t < valid) {
            p.dg_out[(tok0 + t) * p.H + h] = dg;
            p.dbeta_out[(tok0 + t) * p.H + h] = s_dbeta[t];
        }
    }
#ifdef GDN_CYCLE_BUDGET
    LTICK(14);
    // 32 workgroups spread over the grid report: [slot][15 groups | slabs]
    const int stride = max((int)gridDim.x / GDN_LOCAL_CYCLE_SLOTS, 1);
    if (p.cycle_out != nullptr && t == 0 && blockIdx.x % stride == 0 && blockIdx.x / stride < GDN_LOCAL_CYCLE_SLOTS) {
        uint64_t* out = p.cycle_out + (blockIdx.x / stride) * 16;
#pragma unroll
        for (int i = 0; i < 15; i++) out[i] = cyc[i];
        out[15] = (uint64_t)(V / VW);
    }
#endif
#undef LTICK
}


// ------------------------------------------------------------------------------------------
// Everything the backward needs per chunk before its two sweeps, one workgroup per (sequence, head, chunk),
// for batches of whole chunks (one sequence per row, T a multiple of 64):
//   * gamma, beta (fp32) and the inverse norms of the rows of q and k, packed per chunk, for
//     chunk_local_grads_kernel;
//   * the "mirror" problem that turns the reverse sweep into a forward scan (tokens in reverse order; chunk c
//     becomes chunks A, B = 2 r, 2 r + 1 with r = NC - 1 - c):
//         A:  v := P^T dO, k := k, T' := T^T mirrored, P := I, row scales of k: -tail / |k| before T',
//             -beta e / |k| for the state update, e^{gamma_C} decay
//         B:  v := dO, k := q, T' := I, P := 0, row scale e scale / |q| for the state update, no decay
//     i.e. the rows of k_m and v_m and both records, in the layout chunk_prepare32_kernel writes.
// K = 64, 128, 256; V a multiple of 64 up to 512.  The rows of q and k are only needed for K K^T and Q K^T; slabs of
// dO^T and the scratch of the inverse then take their place in LDS (K <= 128: two workgroups per CU).
// ------------------------------------------------------------------------------------------
constexpr int LDA = 68;  // floats per LDS row of A / T

struct BwdPrepareParams {
    const bf16_t* q;
    const bf16_t* k;
    const bf16_t* dout;
    const float* g;  // [N][T][H], NULL = 0
    const void* beta;  // [N][T][H], NULL = 1
    int beta_dtype;
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t d_stride_b, d_stride_t, d_stride_h;
    int N, H, NC, V;
    int l2norm;
    int rec16;  // fragments of the records in the lane order of the 16x16x32 MFMA (GDN_FLAG_RECORDS_16X16)
    int skip_empty;  // chunk slots past the end of a sequence get nothing (GDN_FLAG_SKIP_EMPTY_CHUNKS)
    float scale;
    float* gam;
    float* bc;
    float* rq;
    float* rk;
    const int32_t* seq_start;  // as in ChunkLocalParams
    const int32_t* seq_len;
    int T_rows;
    bf16_t* k_m;
    bf16_t* v_m;
    uint8_t* rec;
    uint8_t* rec_fwd;  // the forward sweep's own records, [H][N NC] (whole-chunk batches), or NULL
    uint32_t rec_bytes, off_p, off_qs, off_ks, off_cs, off_eg;
};

// T = (I + A)^-1 for a strictly lower-triangular 64 x 64 matrix A (fp32 in LDS, rows LDA floats apart, zeros on and
// above the diagonal), in place, by the four waves of the workgroup together; `scratch` holds INVERSE_SCRATCH_FLOATS.
// The same blocked scheme as the forward's prepare step (gdn_chunk_prepare32.h, which interleaves it with its tile
// products): wave 0 inverts the four 16 x 16 diagonal blocks by substitution (a lane owns a column: 120 dependent
// multiply-adds instead of the 2016 of a substitution over all 64 rows), then the blocks below the diagonal follow
// from T_BA = -T_BB (A_BA T_AA), first with 16 x 16 blocks on two waves, then with 32 x 32 blocks, one 16 x 16
// output tile per wave, as products on the fp32 MFMA (16x16x4: no operand is rounded).  Ends with a barrier.
constexpr int INV_LDT = 36, INV_LDM = 20;  // floats per row of the transposed 32 x 32 and 16 x 16 scratch blocks
constexpr int INVERSE_SCRATCH_FLOATS = 32 * INV_LDT + 2 * 16 * INV_LDM + 32 * INV_LDT;
template <int LDA_>
__device__ __forceinline__ void invert_unit_lower_64(float* sA, float* scratch, const int wave, const int lane) {
    constexpr int LDT = INV_LDT, LDM = INV_LDM;
    float* const sT = sA;
    float* const sTtA = scratch;           // transpose of the top-left 32 x 32 of T
    float* const sMt = sTtA + 32 * LDT;    // transposed products of the first merge
    float* const sMtB = sMt + 2 * 16 * LDM;  // transposed product of the second merge
    const int l16 = lane % 16, lq = lane / 16;
    __syncthreads();  // A is complete and the scratch is free
    float x[16];  // column l16 of the inverse of diagonal block lq (wave 0)
    if (wave == 0) {
        const float* a = &sA[(16 * lq) * LDA_ + 16 * lq];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            f32x4 row[4];
#pragma unroll
            for (int c4 = 0; c4 < (i + 3) / 4; c4++) row[c4] = *reinterpret_cast<const f32x4*>(&a[i * LDA_ + 4 * c4]);
            float part[4] = {(i == l16) ? 1.f : 0.f, 0.f, 0.f, 0.f};  // four independent partial sums
#pragma unroll
            for (int kk = 0; kk < i; kk++) part[kk % 4] -= row[kk / 4][kk % 4] * x[kk];
            x[i] = (part[0] + part[1]) + (part[2] + part[3]);
        }
        // every lane of the wave has read its block of A by now (one wave, program order)
#pragma unroll
        for (int i = 0; i < 16; i++) sT[(16 * lq + i) * LDA_ + 16 * lq + l16] = x[i];
    }
    __syncthreads();
    // 16 x 16 output tile of a product X Y: lane (l16, lq) supplies reduction entries k = 4 n lq + e, e < 4 n, of row l16
    // of X and of column l16 of Y (a row of Y^T); MFMA e takes entry e of every lane.
    auto mm16 = [&](const float* xrow, const float* ytrow) -> f32x4 {
        const f32x4 xv = *reinterpret_cast<const f32x4*>(xrow), yv = *reinterpret_cast<const f32x4*>(ytrow);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; e++) acc = mfma_f32(xv[e], yv[e], acc);
        return acc;
    };
    auto mm16x32 = [&](const float* xrow, const float* ytrow) -> f32x4 {
        const f32x4 x0 = *reinterpret_cast<const f32x4*>(xrow), x1 = *reinterpret_cast<const f32x4*>(xrow + 4);
        const f32x4 y0 = *reinterpret_cast<const f32x4*>(ytrow), y1 = *reinterpret_cast<const f32x4*>(ytrow + 4);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; e++) acc = mfma_f32(x0[e], y0[e], acc);
#pragma unroll
        for (int e = 0; e < 4; e++) acc = mfma_f32(x1[e], y1[e], acc);
        return acc;
    };
    // first merge: T_10 = -T_11 (A_10 T_00) on wave 0, T_32 = -T_33 (A_32 T_22) on wave 1
    if (wave < 2) {
        const int bi = 2 * wave + 1, bj = 2 * wave;
        const int kk = 4 * lq;
        float* const mt = &sMt[wave * 16 * LDM];
        f32x4 y0;  // column l16 of T_bj,bj, entries kk .. kk + 3 (a row of its transpose)
#pragma unroll
        for (int e = 0; e < 4; e++) y0[e] = sT[(16 * bj + kk + e) * LDA_ + 16 * bj + l16];
        f32x4 m = {0.f, 0.f, 0.f, 0.f};
        {
            const f32x4 xa = *reinterpret_cast<const f32x4*>(&sA[(16 * bi + l16) * LDA_ + 16 * bj + kk]);
#pragma unroll
            for (int e = 0; e < 4; e++) m = mfma_f32(xa[e], y0[e], m);
        }
        if (wave == 0 && lq < 2) {
            // the transposes of T_00 and T_11 for the second merge, from the registers of the inverse, and the zero block (T_01)^T
#pragma unroll
            for (int c4 = 0; c4 < 4; c4++)
                *reinterpret_cast<f32x4*>(&sTtA[(16 * lq + l16) * LDT + 16 * lq + 4 * c4]) = f32x4{x[4 * c4], x[4 * c4 + 1], x[4 * c4 + 2], x[4 * c4 + 3]};
            if (lq == 1) {
#pragma unroll
                for (int c4 = 0; c4 < 4; c4++) *reinterpret_cast<f32x4*>(&sTtA[(16 + l16) * LDT + 4 * c4]) = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
        *reinterpret_cast<f32x4*>(&mt[l16 * LDM + 4 * lq]) = m;  // M^T[n][4 lq + e]
        const f32x4 t = mm16(&sT[(16 * bi + l16) * LDA_ + 16 * bi + kk], &mt[l16 * LDM + kk]);
#pragma unroll
        for (int e = 0; e < 4; e++) sT[(16 * bi + 4 * lq + e) * LDA_ + 16 * bj + l16] = -t[e];  // over A_bi,bj, read above
        if (wave == 0) *reinterpret_cast<f32x4*>(&sTtA[l16 * LDT + 16 + 4 * lq]) = -t;  // (T_10)^T
    }
    __syncthreads();
    // second merge: T_BA = -T_BB (A_BA T_AA) with 32 x 32 blocks; one 16 x 16 output tile per wave
    {
        const int ta = wave / 2, tb = wave % 2;
        const f32x4 m = mm16x32(&sA[(32 + 16 * ta + l16) * LDA_ + 8 * lq], &sTtA[(16 * tb + l16) * LDT + 8 * lq]);
        *reinterpret_cast<f32x4*>(&sMtB[(16 * tb + l16) * LDT + 16 * ta + 4 * lq]) = m;
        __syncthreads();
        const f32x4 t = mm16x32(&sT[(32 + 16 * ta + l16) * LDA_ + 32 + 8 * lq], &sMtB[(16 * tb + l16) * LDT + 8 * lq]);
#pragma unroll
        for (int e = 0; e < 4; e++) sT[(32 + 16 * ta + 4 * lq + e) * LDA_ + 16 * tb + l16] = -t[e];
    }
    __syncthreads();  // T is complete
}

template <int K>
__global__ __launch_bounds__(BWD_THREADS, (K <= 64 ? 3 : 2)) void chunk_bwd_prepare_kernel(const BwdPrepareParams p) {
    const int V = p.V;
    constexpr int LDK = K + 8;                 // bf16 per LDS row of q / k
    constexpr int CPR = K / 8;                 // 16-byte pieces per row of q / k
    constexpr int RPP = BWD_THREADS / CPR;     // rows per pass of their copy
    // dO is staged as it lies (rows of tokens), 128 (or a last 64) columns at a time, over the rows of q and k once they
    // are dead; P^T dO takes it as the B operand through the transposing LDS load (staging it transposed took 32 2-byte
    // writes per thread and slab with 16-way bank conflicts: a third of the kernel's cycles at V = 512)
    // K = 256: the rows of q are staged one half of the key dim at a time (Q K^T adds up over the halves, the second
    // half waits in registers), which brings the workgroup from 96 KB of LDS to 79 KB: two per CU instead of one.
    constexpr bool QH = K > 128;
    constexpr int LDQ = QH ? K / 2 + 8 : LDK;  // bf16 per LDS row of (the staged half of) q
    constexpr int QK_ELEMS = C * LDQ + C * LDK;
    static_assert((128 + 8) * C <= QK_ELEMS, "a slab of dO fits the rows of q and k");
    __shared__ __attribute__((aligned(16))) bf16_t sQK[QK_ELEMS];   // rows of q, of k; then slabs of dO; then the scratch of the inverse
    __shared__ __attribute__((aligned(16))) bf16_t sPT[C * LDS64];     // P^T
    __shared__ __attribute__((aligned(16))) float sA[C * LDA];         // A, then T in its place
    __shared__ float s_gam[C], s_beta[C], s_e[C], s_tail[C], s_rq[C], s_rk[C];
    bf16_t* const sQ = sQK;
    bf16_t* const sK = sQK + C * LDQ;
    bf16_t* const sDO = sQK;  // [64][VS + 8]

    const int t = threadIdx.x;
    const int lane = t % WAVE, wave = t / WAVE;
    const int l32 = lane % 32, lh = lane / 32;
    const int64_t chunk = blockIdx.x;
    const int ci = (int)(chunk % p.NC);
    const int chain = (int)(chunk / p.NC);
    const int n = chain / p.H, h = chain % p.H;
    const int64_t TM = (int64_t)p.NC * 2 * C;  // tokens per sequence of the mirror problem
    // first token of the chunk as a flat index over the rows of the caller's tensors, and its number of tokens;
    // a chunk past the end of its sequence (valid = 0) still gets its (neutral) records and zero rows, unless the caller
    // scans without them (skip_empty below)
    int valid = C;
    int64_t tok0 = (int64_t)n * p.T_rows + (int64_t)ci * C;
    if (p.seq_start != nullptr) {
        valid = min(max(p.seq_len[n] - ci * C, 0), C);
        tok0 = (int64_t)p.seq_start[n] + (int64_t)ci * C;
    }
    // (GDN_FLAG_SKIP_EMPTY_CHUNKS: the mirror scan walks every row over its own chunks and never comes here; an empty
    // sequence keeps its first slot, which that scan does walk)
    if (valid == 0 && p.skip_empty && ci > 0) return;  // whole workgroup
    // (a chunk lies within one row of the batch; rows past the end of the sequence read its last token and are zeroed)
    const int64_t row_b = tok0 / p.T_rows, row_t = tok0 % p.T_rows;
    auto row_of = [&](const bf16_t* base, int64_t sb, int64_t st, int64_t sh, int row) -> const bf16_t* {
        return base + row_b * sb + (row_t + max(min(row, valid - 1), 0)) * st + (int64_t)h * sh;
    };
    bf16x8 zero8;
#pragma unroll
    for (int e = 0; e < 8; e++) zero8[e] = (bf16_t)0.f;
    const int64_t mir0 = (int64_t)(p.NC - 1 - ci) * 2 * C;  // first token of chunk A in the mirror problem
    // token `row` of this chunk is token 63 - row of the mirror chunks A and B
    auto tok_a = [&](int row) -> int64_t { return ((int64_t)n * TM + mir0 + (C - 1 - row)) * p.H + h; };
    // without reversed copies (k_m NULL) P^T dO goes out in the caller's token order, [N, NC 64, H, V], and nothing else
    const bool copies = p.k_m != nullptr;
    auto tok_u = [&](int row) -> int64_t { return copies ? tok_a(row) : (((int64_t)n * p.NC + ci) * C + row) * p.H + h; };

    // Everything the chunk reads first is asked for at once - the rows of q and k, the first slab of dO, g and beta - so
    // that wave 0's prefix sum below runs while the rows are on their way, not in front of them.
    bf16x8 qn[C / RPP], kn[C / RPP], dpre[4];
    if (valid > 0) {
        const int p8 = t % CPR;
#pragma unroll
        for (int it = 0; it < C / RPP; it++) {
            const int row = t / CPR + RPP * it;
            qn[it] = *reinterpret_cast<const bf16x8*>(row_of(p.q, p.q_stride_b, p.q_stride_t, p.q_stride_h, row) + 8 * p8);
            kn[it] = *reinterpret_cast<const bf16x8*>(row_of(p.k, p.k_stride_b, p.k_stride_t, p.k_stride_h, row) + 8 * p8);
        }
        const int vpr = V >= 128 ? 16 : 8, vrpp = BWD_THREADS / vpr;
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int row = t / vpr + vrpp * it;
            dpre[it] = zero8;
            if (row < C) dpre[it] = *reinterpret_cast<const bf16x8*>(row_of(p.dout, p.d_stride_b, p.d_stride_t, p.d_stride_h, row) + 8 * (t % vpr));
        }
    }

    // ---- gamma (prefix sum of g inside the chunk) and beta: wave 0 ----
    if (wave == 0) {
        const int64_t at = (lane < valid ? tok0 + lane : 0) * p.H + h;
        float x = (p.g == nullptr || lane >= valid) ? 0.f : p.g[at];
        const float b = lane < valid ? load_beta(p.beta, p.beta_dtype, at) : 0.f;
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
            const float y = __shfl_up(x, off, WAVE);
            if (lane >= off) x += y;
        }
        const float gl = __shfl(x, WAVE - 1, WAVE);
        s_gam[lane] = x, s_beta[lane] = b, s_e[lane] = __expf(x), s_tail[lane] = __expf(gl - x);
        p.gam[chunk * C + lane] = x;
        p.bc[chunk * C + lane] = b;
    }

    if (valid == 0) {
        // A chunk slot past the end of its sequence (batches laid out with the chunk count of their longest sequence):
        // what the code below would arrive at from rows of zeros - zero rows of the mirror problem, T = I, the constant
        // inverse norms - written directly; only the records are then formed as for any other chunk.
        const float r0 = p.l2norm ? rsqrtf(L2NORM_EPS) : 1.f;
        if (t < C) {
            s_rq[t] = r0, s_rk[t] = r0;
            p.rq[chunk * C + t] = r0, p.rk[chunk * C + t] = r0;
        }
        for (int i = t; i < C * (K / 8); i += BWD_THREADS) {
            const int row = i / (K / 8), p8 = i % (K / 8);
            *reinterpret_cast<bf16x8*>(p.k_m + tok_a(row) * K + 8 * p8) = zero8;
            *reinterpret_cast<bf16x8*>(p.k_m + (tok_a(row) + (int64_t)C * p.H) * K + 8 * p8) = zero8;
        }
        for (int i = t; i < C * (V / 8); i += BWD_THREADS) {
            const int row = i / (V / 8), p8 = i % (V / 8);
            *reinterpret_cast<bf16x8*>(p.v_m + tok_a(row) * V + 8 * p8) = zero8;
            *reinterpret_cast<bf16x8*>(p.v_m + (tok_a(row) + (int64_t)C * p.H) * V + 8 * p8) = zero8;
        }
        for (int i = t; i < C * C; i += BWD_THREADS) sA[(i / C) * LDA + i % C] = (i / C == i % C) ? 1.f : 0.f;
        __syncthreads();
    } else {
        // ---- rows of q and k: 16-byte pieces, CPR lanes per row ----
        {
            const int p8 = t % CPR;
#pragma unroll
            for (int it = 0; it < C / RPP; it++) {
                const int row = t / CPR + RPP * it;
                const bool live = row < valid;
                bf16x8 qr = qn[it], kr = kn[it];
                if (!live) qr = zero8, kr = zero8;
                float ssq = 0.f, ssk = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) ssq += (float)qr[e] * (float)qr[e], ssk += (float)kr[e] * (float)kr[e];
#pragma unroll
                for (int off = CPR / 2; off >= 1; off >>= 1) ssq += __shfl_xor(ssq, off, WAVE), ssk += __shfl_xor(ssk, off, WAVE);
                const float rq = p.l2norm ? rsqrtf(ssq + L2NORM_EPS) : 1.f, rk = p.l2norm ? rsqrtf(ssk + L2NORM_EPS) : 1.f;
                if (p8 == 0) {
                    s_rq[row] = rq, s_rk[row] = rk;
                    p.rq[chunk * C + row] = rq, p.rk[chunk * C + row] = rk;
                }
                bf16x8 qb, kb;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    qb[e] = (bf16_t)((float)qr[e] * rq * p.scale);
                    kb[e] = (bf16_t)((float)kr[e] * rk);
                }
                if constexpr (QH) {
                    qn[it] = qb;  // scaled; the pieces of the second half are written after the first half's products
                    if (p8 < CPR / 2) *reinterpret_cast<bf16x8*>(sQ + row * LDQ + 8 * p8) = qb;
                } else {
                    *reinterpret_cast<bf16x8*>(sQ + row * LDQ + 8 * p8) = qb;
                }
                *reinterpret_cast<bf16x8*>(sK + row * LDK + 8 * p8) = kb;
                // mirror rows: k of chunk A is k, k of chunk B is q
                if (copies) {
                    const int64_t tokA = tok_a(row), tokB = tokA + (int64_t)C * p.H;
                    *reinterpret_cast<bf16x8*>(p.k_m + tokA * K + 8 * p8) = kr;
                    *reinterpret_cast<bf16x8*>(p.k_m + tokB * K + 8 * p8) = qr;
                }
            }
        }
        __syncthreads();

        f32x16 zero;
#pragma unroll
        for (int r = 0; r < 16; r++) zero[r] = 0.f;

        // ---- A = stril(beta_i E . K K^T) and P^T = tril(E . Q K^T)^T: wave -> tile (ti, tj) ----
        {
            const int ti = wave / 2, tj = wave % 2;
            const f32x16 KK = mma_nt(sK + 32 * ti * LDK, LDK, sK + 32 * tj * LDK, LDK, K, zero, l32, lh);
            f32x16 QK = mma_nt(sQ + 32 * ti * LDQ, LDQ, sK + 32 * tj * LDK, LDK, QH ? K / 2 : K, zero, l32, lh);
            if constexpr (QH) {
                __syncthreads();  // the first half of q has been read
                const int p8 = t % CPR;
                if (p8 >= CPR / 2) {
#pragma unroll
                    for (int it = 0; it < C / RPP; it++) *reinterpret_cast<bf16x8*>(sQ + (t / CPR + RPP * it) * LDQ + 8 * (p8 - CPR / 2)) = qn[it];
                }
                __syncthreads();
                QK = mma_nt(sQ + 32 * ti * LDQ, LDQ, sK + 32 * tj * LDK + K / 2, LDK, K / 2, QK, l32, lh);
            }
            const int j = 32 * tj + l32;
            const float gj = s_gam[j];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int i = 32 * ti + 8 * (r / 4) + 4 * lh + r % 4;
                const float E = i >= j ? __expf(s_gam[i] - gj) : 0.f;
                sA[i * LDA + j] = i > j ? s_beta[i] * E * KK[r] : 0.f;
                sPT[j * LDS64 + i] = (bf16_t)(E * QK[r]);
            }
        }
        __syncthreads();  // the rows of q and k are dead

        // ---- P^T dO -> rows of v_m for chunk A, a slab of columns at a time; dO itself -> rows of v_m for chunk B ----
        auto slab = [&](int v0, auto vsc) {
            constexpr int VS = decltype(vsc)::value;
            constexpr int VPR = VS / 8, VRPP = BWD_THREADS / VPR;  // pieces per row of the slab, rows per pass
            const int p8 = t % VPR;
#pragma unroll
            for (int it = 0; it < C / VRPP; it++) {
                const int row = t / VPR + VRPP * it;
                bf16x8 dr;
                if (v0 == 0) dr = dpre[it];  // (uniform)
                else dr = *reinterpret_cast<const bf16x8*>(row_of(p.dout, p.d_stride_b, p.d_stride_t, p.d_stride_h, row) + v0 + 8 * p8);
                if (row >= valid) dr = zero8;
                *reinterpret_cast<bf16x8*>(sDO + row * (VS + 8) + 8 * p8) = dr;
                if (copies) *reinterpret_cast<bf16x8*>(p.v_m + (tok_a(row) + (int64_t)C * p.H) * V + v0 + 8 * p8) = dr;
            }
            __syncthreads();
            // rows j = 32 tj + .., columns v = v0 + 32 tv + l32, tv = wave, wave + 4, ..
            // K >= 128: the rows of q and k leave room behind the slab for the 64 x VS result, which then goes out as whole
            // rows (16 bytes per lane) instead of 2-byte pieces that fill half a line per store
            constexpr bool STAGED = QK_ELEMS >= 128 * LDS64 + C * 128;
            bf16_t* const sU = sQK + 128 * LDS64;  // [64][VS]
#pragma unroll
            for (int tv = wave; tv < VS / 32; tv += BWD_THREADS / WAVE)
#pragma unroll
                for (int tj = 0; tj < 2; tj++) {
                    const f32x16 u = mma_nn(sPT + 32 * tj * LDS64, LDS64, sDO, VS + 8, 32 * tv, C, zero, l32, lh);
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int j = 32 * tj + 8 * (r / 4) + 4 * lh + r % 4;
                        if constexpr (STAGED) sU[j * VS + 32 * tv + l32] = (bf16_t)u[r];
                        else p.v_m[tok_u(j) * V + v0 + 32 * tv + l32] = (bf16_t)u[r];
                    }
                }
            if constexpr (STAGED) {
                __syncthreads();
#pragma unroll
                for (int it = 0; it < C / VRPP; it++) {
                    const int j = t / VPR + VRPP * it;
                    *reinterpret_cast<bf16x8*>(p.v_m + tok_u(j) * V + v0 + 8 * p8) = *reinterpret_cast<const bf16x8*>(sU + j * VS + 8 * p8);
                }
            }
            __syncthreads();  // the slab is free (also for the scratch of the inverse)
        };
        int v0 = 0;
#pragma unroll 1
        for (; v0 + 128 <= V; v0 += 128) slab(v0, std::integral_constant<int, 128>{});
        if (v0 < V) slab(v0, std::integral_constant<int, 64>{});

        // ---- T = (I + A)^-1 in place of A (its scratch over the dead rows of q) ----
        static_assert(INVERSE_SCRATCH_FLOATS * 4 <= QK_ELEMS * 2, "the scratch of the inverse fits the rows of q and k");
        invert_unit_lower_64<LDA>(sA, reinterpret_cast<float*>(sQK), wave, lane);
    }

    // ---- the two records ----
    uint8_t* recA = p.rec + ((int64_t)h * ((int64_t)p.N * 2 * p.NC) + (int64_t)n * 2 * p.NC + 2 * (p.NC - 1 - ci)) * p.rec_bytes;
    uint8_t* recB = recA + p.rec_bytes;
    for (int fl = t; fl < 6 * WAVE; fl += BWD_THREADS) {
        const int f = fl / WAVE, L = fl % WAVE;
        // fragment f, lane L, element e -> entry (row, col) of the lower-triangular 64 x 64 matrix.  32x32x16 order:
        // fragments (row tile, 16-column slab) = (0,0) (0,1) (1,0) (1,1) (1,2) (1,3); a lane holds columns 4 h + 0..3 and
        // 8 + 4 h + 0..3 of the slab.  16x16x32 order: (16-row tile, 32-column slab) = (0,0) (1,0) (2,0) (2,1) (3,0) (3,1);
        // a lane holds columns 4 g + 0..3 and 16 + 4 g + 0..3 of the slab.
        const int row = p.rec16 ? 16 * (f < 2 ? f : 2 + (f - 2) / 2) + L % 16 : 32 * (f < 2 ? 0 : 1) + L % 32;
        const int col0 = p.rec16 ? 32 * (f < 2 ? 0 : f % 2) + 4 * (L / 16) : 16 * (f < 2 ? f : f - 2) + 4 * (L / 32);
        const int second = p.rec16 ? 12 : 4;  // elements 4..7 lie this many columns past e
        bf16x8 tm, id, zz;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int col = col0 + (e < 4 ? e : e + second);
            // mirrored transpose: entry (row, col) is T[63 - col][63 - row], zero above the diagonal
            tm[e] = (bf16_t)(row >= col ? sA[(C - 1 - col) * LDA + (C - 1 - row)] : 0.f);
            id[e] = (bf16_t)(row == col ? 1.f : 0.f);
            zz[e] = (bf16_t)0.f;
        }
        reinterpret_cast<bf16x8*>(recA)[fl] = tm;
        reinterpret_cast<bf16x8*>(recA + p.off_p)[fl] = id;
        // (the fragments of a B chunk are the same for every chunk: a scan with mirror reads takes them from chunk 1 of the
        // chain, which is this sequence's last chunk, and only the row scales from the chunk's own record)
        if (copies || ci == p.NC - 1) {
            reinterpret_cast<bf16x8*>(recB)[fl] = id;
            reinterpret_cast<bf16x8*>(recB + p.off_p)[fl] = zz;
        }
    }
    if (p.rec_fwd != nullptr) {
        // The record the forward's prepare step would write for this chunk (T diag(beta), P, the three row scales,
        // e^{gamma_C}), so that the forward sweep of the backward pass needs no prepare launch of its own.
        uint8_t* const recF = p.rec_fwd + ((int64_t)h * ((int64_t)p.N * p.NC) + (int64_t)n * p.NC + ci) * p.rec_bytes;
        for (int fl = t; fl < 6 * WAVE; fl += BWD_THREADS) {
            const int f = fl / WAVE, L = fl % WAVE;
            const int row = p.rec16 ? 16 * (f < 2 ? f : 2 + (f - 2) / 2) + L % 16 : 32 * (f < 2 ? 0 : 1) + L % 32;
            const int col0 = p.rec16 ? 32 * (f < 2 ? 0 : f % 2) + 4 * (L / 16) : 16 * (f < 2 ? f : f - 2) + 4 * (L / 32);
            const int second = p.rec16 ? 12 : 4;
            bf16x8 tb, pm;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int col = col0 + (e < 4 ? e : e + second);
                tb[e] = (bf16_t)(row >= col ? sA[row * LDA + col] * s_beta[col] : 0.f);
                pm[e] = (valid > 0 && row >= col) ? sPT[col * LDS64 + row] : (bf16_t)0.f;
            }
            reinterpret_cast<bf16x8*>(recF)[fl] = tb;
            reinterpret_cast<bf16x8*>(recF + p.off_p)[fl] = pm;
        }
        if (t < C) {
            const bool live = t < valid;
            reinterpret_cast<float*>(recF + p.off_qs)[t] = s_e[t] * s_rq[t] * p.scale;
            reinterpret_cast<float*>(recF + p.off_ks)[t] = live ? s_tail[t] * s_rk[t] : 0.f;
            reinterpret_cast<float*>(recF + p.off_cs)[t] = live ? s_e[t] * s_rk[t] : 0.f;
            if (t == 0) *reinterpret_cast<float*>(recF + p.off_eg) = s_e[C - 1];
        }
    }
    if (t < C) {
        const int src = C - 1 - t;
        reinterpret_cast<float*>(recA + p.off_qs)[t] = 0.f;
        reinterpret_cast<float*>(recA + p.off_ks)[t] = -(s_beta[src] * s_e[src] * s_rk[src]);
        reinterpret_cast<float*>(recA + p.off_cs)[t] = -(s_tail[src] * s_rk[src]);
        reinterpret_cast<float*>(recB + p.off_qs)[t] = 0.f;
        reinterpret_cast<float*>(recB + p.off_ks)[t] = s_e[src] * s_rq[src] * p.scale;
        reinterpret_cast<float*>(recB + p.off_cs)[t] = 0.f;
        if (t == 0) {
            *reinterpret_cast<float*>(recA + p.off_eg) = s_e[C - 1];
            *reinterpret_cast<float*>(recB + p.off_eg) = 1.f;
        }
    }
}

}  // namespace

static bool bwd_shape_built(int K, int V) { return (K == 64 || K == 128 || K == 256) && V > 0 && V % 64 == 0; }

int launch_chunk_bwd_local(const gdn_chunk_local_args& a, hipStream_t stream) {
    ChunkLocalParams p;
#ifdef GDN_CYCLE_BUDGET
    p.cycle_out = cycle_buffer();
    if (p.cycle_out != nullptr) (void)hipMemsetAsync(p.cycle_out, 0, GDN_LOCAL_CYCLE_SLOTS * 16 * sizeof(uint64_t), stream);
#endif
    p.vnew = a.v_new, p.s0 = a.states, p.ds1 = a.dstates, p.saves_bf16 = a.saves_dtype == GDN_BF16 ? 1 : 0;
    const bool h = a.dstates_dtype == GDN_BF16;
    const bool sl = a.saves_sliced != 0;
    p.gam = a.gamma, p.beta = a.beta;
    p.rq = a.rq, p.rk = a.rk, p.scale = a.scale;
    p.y_mirror = static_cast<const bf16_t*>(a.y_mirror), p.y_chunks = static_cast<const bf16_t*>(a.y_chunks);
    p.dq_out = static_cast<bf16_t*>(a.dq_out), p.dk_out = static_cast<bf16_t*>(a.dk_out), p.dv_out = static_cast<bf16_t*>(a.dv_out);
    p.dg_out = a.dg_out, p.dbeta_out = a.dbeta_out;
    p.H = a.H, p.NC = a.NC, p.V = a.V;
    p.q_raw = static_cast<const bf16_t*>(a.q_raw), p.k_raw = static_cast<const bf16_t*>(a.k_raw);
    p.v_raw = static_cast<const bf16_t*>(a.v_raw), p.d_raw = static_cast<const bf16_t*>(a.dout_raw);
    p.q_stride_b = a.q_stride_b, p.q_stride_t = a.q_stride_t, p.q_stride_h = a.q_stride_h;
    p.k_stride_b = a.k_stride_b, p.k_stride_t = a.k_stride_t, p.k_stride_h = a.k_stride_h;
    p.v_stride_b = a.v_stride_b, p.v_stride_t = a.v_stride_t, p.v_stride_h = a.v_stride_h;
    p.d_stride_b = a.dout_stride_b, p.d_stride_t = a.dout_stride_t, p.d_stride_h = a.dout_stride_h;
    p.seq_start = a.seq_start, p.seq_len = a.seq_len, p.T_rows = a.seq_start != nullptr ? a.T_rows : a.NC * C;
    const dim3 grid((unsigned)a.chunks), block(BWD_THREADS);
    auto launch = [&](auto kc) {
        constexpr int KK = decltype(kc)::value;
        if (sl) hipLaunchKernelGGL((chunk_local_grads_kernel<KK, true, true>), grid, block, 0, stream, p);
        else if (h) hipLaunchKernelGGL((chunk_local_grads_kernel<KK, true, false>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((chunk_local_grads_kernel<KK, false, false>), grid, block, 0, stream, p);
    };
    if (a.K == 64) launch(std::integral_constant<int, 64>{});
    else if (a.K == 128) launch(std::integral_constant<int, 128>{});
    else launch(std::integral_constant<int, 256>{});
    return (int)hipGetLastError();
}

bool chunk_bwd_local_supported(const gdn_chunk_local_args& a) { return bwd_shape_built(a.K, a.V); }

bool chunk_bwd_prepare_supported(const gdn_chunk_bwd_prepare_args& a) {
    if (!bwd_shape_built(a.K, a.V) || a.T <= 0) return false;
    return a.seq_start != nullptr ? (a.seq_len != nullptr && a.NC > 0) : a.T % C == 0;
}

uint64_t chunk_bwd_record_bytes(const gdn_chunk_bwd_prepare_args& a) {
    const uint64_t nc = a.seq_start != nullptr ? a.NC : a.T / C;
    return (uint64_t)a.H * a.N * 2 * nc * record_layout(a.K, a.V).bytes;
}

int launch_chunk_bwd_prepare(const gdn_chunk_bwd_prepare_args& a, hipStream_t stream) {
    const RecordLayout r = record_layout(a.K, a.V);
    BwdPrepareParams p;
    p.q = static_cast<const bf16_t*>(a.q), p.k = static_cast<const bf16_t*>(a.k);
    p.dout = static_cast<const bf16_t*>(a.dout);
    p.g = a.g, p.beta = a.beta, p.beta_dtype = a.beta_dtype;
    p.q_stride_b = a.q_stride_b, p.q_stride_t = a.q_stride_t, p.q_stride_h = a.q_stride_h;
    p.k_stride_b = a.k_stride_b, p.k_stride_t = a.k_stride_t, p.k_stride_h = a.k_stride_h;
    p.d_stride_b = a.dout_stride_b, p.d_stride_t = a.dout_stride_t, p.d_stride_h = a.dout_stride_h;
    p.N = a.N, p.H = a.H, p.V = a.V, p.NC = a.seq_start != nullptr ? a.NC : a.T / C;
    p.seq_start = a.seq_start, p.seq_len = a.seq_len, p.T_rows = a.T;
    p.l2norm = (a.flags & GDN_FLAG_L2NORM) ? 1 : 0;
    p.rec16 = (a.flags & GDN_FLAG_RECORDS_16X16) ? 1 : 0;
    p.skip_empty = (a.flags & GDN_FLAG_SKIP_EMPTY_CHUNKS) ? 1 : 0;
    p.scale = a.scale;
    p.gam = a.gamma, p.bc = a.beta_packed;
    p.rq = a.rq, p.rk = a.rk;
    p.k_m = static_cast<bf16_t*>(a.k_mirror), p.v_m = static_cast<bf16_t*>(a.v_mirror);
    p.rec = static_cast<uint8_t*>(a.records);
    p.rec_fwd = a.seq_start == nullptr ? static_cast<uint8_t*>(a.records_fwd) : nullptr;
    p.rec_bytes = r.bytes, p.off_p = r.off_p, p.off_qs = r.off_qs, p.off_ks = r.off_ks, p.off_cs = r.off_cs, p.off_eg = r.off_eg;
    const int64_t chunks = (int64_t)a.N * a.H * p.NC;
    const dim3 grid((unsigned)chunks), block(BWD_THREADS);
    if (a.K == 64) hipLaunchKernelGGL(chunk_bwd_prepare_kernel<64>, grid, block, 0, stream, p);
    else if (a.K == 128) hipLaunchKernelGGL(chunk_bwd_prepare_kernel<128>, grid, block, 0, stream, p);
    else hipLaunchKernelGGL(chunk_bwd_prepare_kernel<256>, grid, block, 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace gdn

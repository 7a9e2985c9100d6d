// C[M, N] = alpha * A[M, K] * W[N, K]^T for few rows M (decoding, the output
// head): bfloat16 operands on the matrix cores, float32 accumulation, float32
// or bfloat16 result.  The weight matrix is streamed once per 64 rows of A.
//
// Grid (ceil(N/(16*NT)), ceil(M/(16*MT))), WPB waves.  Every wave owns the same
// NT tiles of 16 weight rows and a share of K (k-steps of 32, dealt in turn; WPB is 4, 8
// or 16 so that narrow matrices still fill the chip); lane
// (r = l%16, kq = l/16) loads 16 bytes W[n0+r][k0+8kq..+7] and the matching
// 16 bytes of each A row tile, and feeds them to one v_mfma_f32_16x16x32_bf16
// as A and B operands.  Both operands use the same lane->k mapping, so the
// order of k inside a step does not matter.  The waves' partial sums meet in LDS.
// Two variants of the walk over K: OWN_K gives each wave one contiguous run of
// k-steps (long rows), and AG > 1 lets one load of the token operand serve AG
// k-steps when at most 16 / AG rows are in use (the spare lanes carry the other
// steps' data and a row rotation hands it over).
//
// With 32,768 weight rows or more and up to 16 rows of A (the output head) a second kernel runs, in which
// waves own whole weight tiles (gemm_wide_kernel below).
//
// 16x16x32 layout (lane l): A[i = l%16][k = 8(l/16)..+7], B[k = 8(l/16)..+7][j = l%16],
// D[i = 4(l/16) + e][j = l%16], e = 0..3.
#include "common.h"
#include "infinicore_infer_variants.h"
#include <utility>

typedef short v4s __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));


// 8 consecutive bf16 from p (valid: how many of them exist), zero-filled.
template <bool ALIGNED>
__device__ __forceinline__ void load8(const uint16_t* __restrict__ p, int valid, v4s& lo, v4s& hi) {
    if (ALIGNED && valid >= 8) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        lo[0] = (short)(v.x & 0xffff); lo[1] = (short)(v.x >> 16);
        lo[2] = (short)(v.y & 0xffff); lo[3] = (short)(v.y >> 16);
        hi[0] = (short)(v.z & 0xffff); hi[1] = (short)(v.z >> 16);
        hi[2] = (short)(v.w & 0xffff); hi[3] = (short)(v.w >> 16);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo[e] = (e < valid) ? (short)p[e] : (short)0;
            hi[e] = (e + 4 < valid) ? (short)p[e + 4] : (short)0;
        }
    }
}

// What the fused projection + rotary + cache-write epilogue needs beside the product.
struct RopeEpilogue {
    const int* positions;      // [M]
    const int* slots;          // [M] token slot in the cache (page * page_size + offset), < 0: no write
    const float* cos_t;        // [max_pos, dh/2]
    const float* sin_t;
    void* kcache;              // [pages, nkvh, page_size, dh]
    void* vcache;
    int nh, nkvh, dh, page_size;
    int rr;                    // weight rows per tile that are used: 16, 8 or 4 (few heads: smaller tiles make more blocks)
};

// A norm split over two products (M <= 16).  The product BEFORE the norm (EPI == 3) owns the
// residual add: h = x + rscale * (its result), written back to x; it stores y = h * g (g: the
// norm's weight) instead of its result, and per column block the sums of h^2 of every row.  The
// product AFTER the norm takes y as its operand and multiplies row m of its result by
// rsqrt(sum over the column blocks / width + eps): the norm's row factor commutes with the product.
constexpr int kMaxSumParts = 256;
constexpr int kOwnKFrom = 8192;          // from this K on the waves of the few-row product own contiguous runs of k-steps
struct NormFuse {
    const float* ss_in;        // [n_parts_in, 16] sums of squares per column block and row; nullptr: rows are normed already
    int n_parts_in;            // <= kMaxSumParts
    float inv_width, eps;
    float* x;                  // EPI == 3: float32 residual stream [M, N], row stride ldx, updated in place
    int ldx;
    const float* g;            // [N]
    float rscale;
    float* ss_out;             // [gridDim.x, 16]
};

// lane i of a row of 16 lanes takes the value of lane (i + S) % 16 (a DPP row rotation, no LDS)
template <int S> __device__ __forceinline__ v4s row_from_above(v4s v) {
    if constexpr (S % 16 == 0) return v;
    else {
        typedef int v2i __attribute__((ext_vector_type(2)));
        const v2i a = __builtin_bit_cast(v2i, v);
        v2i b;
        b[0] = __builtin_amdgcn_update_dpp(0, a[0], 0x120 + (16 - S % 16), 0xf, 0xf, false);
        b[1] = __builtin_amdgcn_update_dpp(0, a[1], 0x120 + (16 - S % 16), 0xf, 0xf, false);
        return __builtin_bit_cast(v4s, b);
    }
}
// step u of an iteration takes its token operand out of the register that was loaded for its group of AG steps
template <int AG, int MP, int... Us>
__device__ __forceinline__ void spread_token_operand(const v4s* glo, const v4s* ghi, v4s (*alo)[1], v4s (*ahi)[1],
                                                     std::integer_sequence<int, Us...>) {
    ((alo[Us][0] = row_from_above<(Us % AG) * MP>(glo[Us / AG]), ahi[Us][0] = row_from_above<(Us % AG) * MP>(ghi[Us / AG])), ...);
}

// LINES (K a multiple of 64, aligned operands): the weights come in whole cache lines, a wave's load covering 8 rows x
// 128 bytes (two k-steps), with the non-temporal hint: a kernel that only streams a weight matrix so takes 9.4 us for
// the 2B shape's 53 MB gate/up matrix where loads in operand layout (16 rows x 64 bytes) take 15.6.  What a load
// brings is not in operand layout, so each wave passes it through LDS of its own on its way to the matrix cores.  In the
// kernel below the loads write it there themselves (global_load_lds_dwordx4: lane l puts 16 bytes at the tile's half +
// 16 l, no registers and no LDS store instructions, which take 13 cycles per KB and unit where reads take 6): rows of
// 128 bytes without padding, chunk c of row r at position c ^ (r / 2 % 8), which each lane arranges by what it fetches, so
// that the 16-byte operand reads of 16 rows cover the 64 banks once; a tile of 2 KB per pair of k-steps in flight and
// 16-row tile.  2B shape, recorded steps, against registers + ds_write: batch 1 1.90 -> 1.88 ms, batch 8 2.92 -> 2.89.
// The kernel for very many weight rows further down still stores from registers, into rows 144 bytes apart.
constexpr int kLineRowBytes = 144;
template <typename TC, int NT, int MT, int WPB, int UNROLL, bool ALIGNED, int EPI, bool OWN_K = false, int AG = 1, bool LINES = false>
__global__ void __launch_bounds__(WPB * 64)
gemm_nt_bf16_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W, TC* __restrict__ C,
                    int M, int N, int K, int lda, int ldw, int ldc, float alpha, RopeEpilogue rope, NormFuse nf) {
    constexpr bool CSWIGLU = (EPI == 1);
    constexpr bool CROPE = (EPI == 2);
    constexpr bool CRESID = (EPI == 3);
    constexpr int PV = kMaxSumParts / (WPB * 4);             // column-block sums a thread fetches
    static_assert(!LINES || (ALIGNED && UNROLL % 2 == 0), "whole-line weight loads take k-steps in pairs");
    // the waves' partial sums after the loop; while the loop runs the same memory passes the weights on (LINES)
    constexpr int kWaveLineBytes = (UNROLL / 2 > 0 ? UNROLL / 2 : 1) * NT * 2048;      // a wave's tiles of an iteration: 16 rows x 128 bytes each
    constexpr int kRedBytes = (WPB - 1) * NT * MT * 64 * 4 * 4, kLineBytes = LINES ? WPB * kWaveLineBytes : 0;
    __shared__ __attribute__((aligned(16))) unsigned char red_mem[kRedBytes > kLineBytes ? kRedBytes : kLineBytes];
    float (*red)[NT * MT][64][4] = reinterpret_cast<float (*)[NT * MT][64][4]>(red_mem);
    __shared__ float ssum[WPB * 4][16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, kq = lane >> 4;
    // CSWIGLU: W = [gate rows (N/2); up rows (N/2)]; a block owns R = ceil((N/2) / blocks) <= 16 G
    // gate rows (G = NT / 2 tiles of 16) and the matching up rows and writes C[m][n] = up * silu(gate)
    // for its R columns of the N/2 wide output.  R need not be a multiple of 16: the launcher picks
    // the number of blocks so that they fill the chip in one round where 16-row tiles would need
    // a second, part-filled one.
    // CROPE: W = [q heads; k heads; v heads] (rows of dh).  A block owns rr (16, 8 or 4) rows j.. of one q
    // or k head and the rr rows j + dh/2.. that rotate with them, or 2 rr consecutive rows of a v head; with
    // rr < 16 the other rows of its two tiles repeat the last one and are dropped.
    constexpr int G = CSWIGLU ? NT / 2 : 1;
    const int NO = CSWIGLU ? N / 2 : N;                      // output columns
    const int sw_cols = CSWIGLU ? (NO + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    int n0 = CSWIGLU ? blockIdx.x * sw_cols : blockIdx.x * (16 * NT);
    const int sw_end = (n0 + sw_cols < NO) ? n0 + sw_cols : NO;   // CSWIGLU: one past the block's last column
    // CRESID: a block owns ceil(N / blocks) <= 16 columns, so that few columns still make a block per compute unit
    const int rs_cols = CRESID ? (N + (int)gridDim.x - 1) / (int)gridDim.x : 0;
    if (CRESID) n0 = blockIdx.x * rs_cols;
    const int rs_end = (n0 + rs_cols < N) ? n0 + rs_cols : N;
    const int m0 = blockIdx.y * (16 * MT);
    int rope_head = 0, rope_j = 0;                           // CROPE: head and first index in the head
    bool rope_is_v = false;
    if (CROPE) {
        const int half = rope.dh >> 1, pt = half / rope.rr, n_rot = (rope.nh + rope.nkvh) * pt;
        const int p = blockIdx.x;
        if (p < n_rot) { rope_head = p / pt; rope_j = rope.rr * (p - rope_head * pt); }
        else {
            const int vt = rope.dh / (2 * rope.rr), pv = p - n_rot;
            rope_is_v = true;
            rope_head = rope.nh + rope.nkvh + pv / vt;
            rope_j = 2 * rope.rr * (pv % vt);
        }
        n0 = rope_head * rope.dh + rope_j;
    }

    const uint16_t* wp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int base = CSWIGLU ? n0 + 16 * (nt % G) + (nt / G) * NO : n0 + 16 * nt;
        if (CROPE) base = n0 + nt * (rope_is_v ? rope.rr : (rope.dh >> 1));
        const int lim = CSWIGLU ? (nt / G) * NO + sw_end : (CRESID ? rs_end : (CROPE ? base + rope.rr : N));
        const int nrow = (base + r < lim) ? base + r : lim - 1;
        wp[nt] = W + (size_t)nrow * ldw + 8 * kq;
    }
    // LINES: lane l loads 16 bytes of row 8 h + l / 8 of the tile (h = 0, 1) at byte 16 (l % 8) of a 128-byte line
    const uint16_t* wp8[NT][2];
    if (LINES) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            int base = CSWIGLU ? n0 + 16 * (nt % G) + (nt / G) * NO : n0 + 16 * nt;
            if (CROPE) base = n0 + nt * (rope_is_v ? rope.rr : (rope.dh >> 1));
            const int lim = CSWIGLU ? (nt / G) * NO + sw_end : (CRESID ? rs_end : (CROPE ? base + rope.rr : N));
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int row = base + 8 * h + (lane >> 3);
                wp8[nt][h] = W + (size_t)(row < lim ? row : lim - 1) * ldw + 8 * ((lane & 7) ^ (((8 * h + (lane >> 3)) >> 1) & 7));
            }
        }
    }
    unsigned char* const line_buf = red_mem + (LINES ? wave * kWaveLineBytes : 0);
    const uint16_t* ap[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int mrow = (m0 + 16 * mt + r < M) ? m0 + 16 * mt + r : M - 1;
        ap[mt] = A + (size_t)mrow * lda + 8 * kq;
    }
    v4f acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = v4f{0.f, 0.f, 0.f, 0.f};

    // the row factors' partial sums are fetched first and used last: their latency hides behind the loop
    float pv[PV];
    if (nf.ss_in) {
#pragma unroll
        for (int i = 0; i < PV; ++i) {
            const int b = (tid >> 4) + i * (WPB * 4);
            pv[i] = (b < nf.n_parts_in) ? nf.ss_in[b * 16 + (tid & 15)] : 0.f;
        }
    }

    // the residual epilogue's operands are fetched first as well
    float xres[4] = {0.f, 0.f, 0.f, 0.f}, gres[4] = {0.f, 0.f, 0.f, 0.f};
    if (CRESID && wave == 0 && m0 + r < M) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = n0 + 4 * kq + e;
            if (n < rs_end) { xres[e] = nf.x[(size_t)(m0 + r) * nf.ldx + n]; gres[e] = nf.g[n]; }
        }
    }

    // k-steps of 32 are dealt to the waves in turn; UNROLL steps are loaded before any is used.
    // OWN_K (for long rows): a wave owns a contiguous run of steps instead, so that it walks
    // UNROLL * 64 bytes of every row at a time and one stretch of each row overall.
    const int nsteps = (K + 31) >> 5;
    const int spw = ((nsteps + WPB - 1) / WPB + UNROLL - 1) / UNROLL * UNROLL;      // OWN_K: steps per wave
    const int s_begin = OWN_K ? wave * spw : wave;
    const int s_end = OWN_K ? ((wave + 1) * spw < nsteps ? (wave + 1) * spw : nsteps) : nsteps;
    constexpr int s_stride = OWN_K ? 1 : WPB;                // between the UNROLL steps of one iteration
    // LINES without OWN_K: the waves are dealt PAIRS of k-steps in turn (a 128-byte line holds two), and s0 counts pairs
    constexpr bool PAIR_DEAL = LINES && !OWN_K;
    auto step_at = [&](int s0, int u) { return PAIR_DEAL ? 2 * (s0 + (u >> 1) * WPB) + (u & 1) : s0 + u * s_stride; };
    const int it_end = PAIR_DEAL ? (nsteps >> 1) : s_end;    // (K is a multiple of 64 with LINES: the steps come in whole pairs)
    constexpr int it_stride = PAIR_DEAL ? WPB * (UNROLL / 2) : s_stride * UNROLL;
    for (int s0 = s_begin; s0 < it_end; s0 += it_stride) {
        v4s wlo[LINES ? 1 : UNROLL][NT], whi[LINES ? 1 : UNROLL][NT], alo[UNROLL][MT], ahi[UNROLL][MT];
        if constexpr (LINES) {
            // straight into this wave's LDS (lane l writes 16 bytes at the tile's half + 16 l: rows of 128 bytes without
            // padding, their chunks swizzled by the choice of what each lane fetches), with the non-temporal hint
            typedef const void __attribute__((address_space(1)))* gptr_t;
            typedef void __attribute__((address_space(3)))* lptr_t;
#pragma unroll
            for (int j = 0; j < UNROLL / 2; ++j) {
                const int st = step_at(s0, 2 * j);
                // a pair beyond the end loads the first one again and is multiplied with zeros: the loads stay without a
                // condition (measured: skipping them, with the wait that a branch then needs written out, was 1 % slower at
                // batch 8; and the compiler's own wait for loads into LDS does not survive a branch)
                const int stc = st < s_end ? st : 0;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        __builtin_amdgcn_global_load_lds((gptr_t)(wp8[nt][h] + 32 * stc), (lptr_t)(line_buf + (j * NT + nt) * 2048 + 1024 * h), 16, 0, 2);
            }
        } else {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int kk = 32 * step_at(s0, u);
            const int valid = (step_at(s0, u) < s_end) ? K - kk - 8 * kq : 0;          // <= 0 beyond the end
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (valid > 0) load8<ALIGNED>(wp[nt] + kk, valid, wlo[u][nt], whi[u][nt]);
                else { wlo[u][nt] = v4s{0, 0, 0, 0}; whi[u][nt] = wlo[u][nt]; }
            }
        }
        }
        if constexpr (AG == 1) {
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int kk = 32 * step_at(s0, u);
                const int valid = (step_at(s0, u) < s_end) ? K - kk - 8 * kq : 0;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    if (valid > 0) load8<ALIGNED>(ap[mt] + kk, valid, alo[u][mt], ahi[u][mt]);
                    else { alo[u][mt] = v4s{0, 0, 0, 0}; ahi[u][mt] = alo[u][mt]; }
                }
            }
        } else {
            // Up to 16 / AG rows (MT == 1): one load serves AG steps.  Lane r of a row of 16 loads token row
            // r % MP of step r / MP; step t's operand is then that register rotated down by t * MP lanes
            // (the columns from MP on hold other steps' rows and are never stored).  The cost of the token
            // operand is the number of its load instructions, not its bytes.
            static_assert(AG == 1 || (MT == 1 && UNROLL % AG == 0 && 16 % AG == 0), "grouped token loads");
            constexpr int MP = 16 / AG;
            v4s glo[UNROLL / AG], ghi[UNROLL / AG];
            const int gt = r / MP, gm = r % MP;
            const uint16_t* gp = A + (size_t)((m0 + gm < M) ? m0 + gm : M - 1) * lda + 8 * kq;
#pragma unroll
            for (int g = 0; g < UNROLL / AG; ++g) {
                const int st = step_at(s0, g * AG + gt);
                const int kk = 32 * st;
                const int valid = (st < s_end && m0 + gm < M) ? K - kk - 8 * kq : 0;
                if (valid > 0) load8<ALIGNED>(gp + kk, valid, glo[g], ghi[g]);
                else { glo[g] = v4s{0, 0, 0, 0}; ghi[g] = glo[g]; }
            }
            spread_token_operand<AG, MP>(glo, ghi, alo, ahi, std::make_integer_sequence<int, UNROLL>{});
        }
        typedef short v8s __attribute__((ext_vector_type(8)));
        typedef __bf16 v8b __attribute__((ext_vector_type(8)));
        if constexpr (LINES) {
#pragma unroll
            for (int j = 0; j < UNROLL / 2; ++j) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    // through this wave's LDS: in as rows of 128 bytes, out as the operands of the pair's two k-steps
                    // (row r, bytes 16 kq .. of the first half and of the second).  LDS serves a wave's requests in order.
                    uint4 w2[2];
#pragma unroll
                    for (int e = 0; e < 2; ++e)
                        w2[e] = *reinterpret_cast<const uint4*>(line_buf + (j * NT + nt) * 2048 + r * 128 + 16 * ((4 * e + kq) ^ ((r >> 1) & 7)));
#pragma unroll
                    for (int e = 0; e < 2; ++e)
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) {
                            const v8s a8 = __builtin_shufflevector(alo[2 * j + e][mt], ahi[2 * j + e][mt], 0, 1, 2, 3, 4, 5, 6, 7);
                            acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, w2[e]), __builtin_bit_cast(v8b, a8),
                                                                                  acc[nt][mt], 0, 0, 0);
                        }
                }
            }
        } else {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    // one 16x16x32 product per k-step: a lane's 8 elements of W and of A are k = 8 kq .. 8 kq + 7 of the step
                    const v8s w8 = __builtin_shufflevector(wlo[u][nt], whi[u][nt], 0, 1, 2, 3, 4, 5, 6, 7);
                    const v8s a8 = __builtin_shufflevector(alo[u][mt], ahi[u][mt], 0, 1, 2, 3, 4, 5, 6, 7);
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, w8), __builtin_bit_cast(v8b, a8),
                                                                          acc[nt][mt], 0, 0, 0);
                }
        }
    }
    if (LINES) __syncthreads();                              // every wave is done passing weights through what now holds the sums
    if (wave > 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int e = 0; e < 4; ++e) red[wave - 1][nt * MT + mt][lane][e] = acc[nt][mt][e];
    }
    if (nf.ss_in) {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < PV; ++i) t += pv[i];
        ssum[tid >> 4][tid & 15] = t;
    }
    __syncthreads();
    if (wave > 0) return;
    float rowf = 1.0f;                                       // norm factor of row r (lanes of one column of D)
    if (nf.ss_in) {
        float t = 0.f;
#pragma unroll
        for (int j = 0; j < WPB; ++j) t += ssum[4 * j + kq][r];
        t += __shfl_xor(t, 16, kWave);
        t += __shfl_xor(t, 32, kWave);
        rowf = rsqrtf(t * nf.inv_width + nf.eps);
    }
    alpha *= rowf;
    if (CSWIGLU) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m0 + 16 * mt + r;
#pragma unroll
            for (int gi = 0; gi < G; ++gi)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float g = acc[gi][mt][e], u = acc[G + gi][mt][e];
#pragma unroll
                    for (int w = 0; w < WPB - 1; ++w) { g += red[w][gi * MT + mt][lane][e]; u += red[w][(G + gi) * MT + mt][lane][e]; }
                    // both projections are rounded to the output type first, as when they are stored
                    g = to_f32(from_f32<TC>(alpha * g));
                    u = to_f32(from_f32<TC>(alpha * u));
                    const int n = n0 + 16 * gi + 4 * kq + e;
                    if (m < M && n < sw_end) C[(size_t)m * ldc + n] = from_f32<TC>(silu_mul_fast(g, u));
                }
        }
        return;
    }
    if (CROPE) {
        if (4 * kq >= rope.rr) return;                  // rows of the tiles that repeat the last one
        const int half = rope.dh >> 1;
        const int jj = rope_j + 4 * kq;                 // first of this lane's four indices in the head
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m0 + 16 * mt + r;
            if (m >= M) continue;
            float v0[4], v1[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float a0 = acc[0][mt][e], a1 = acc[NT - 1][mt][e];
#pragma unroll
                for (int w = 0; w < WPB - 1; ++w) { a0 += red[w][mt][lane][e]; a1 += red[w][(NT - 1) * MT + mt][lane][e]; }
                v0[e] = to_f32(from_f32<TC>(alpha * a0));   // the projection is rounded to its type first, as when stored
                v1[e] = to_f32(from_f32<TC>(alpha * a1));
            }
            const int slot = rope.slots[m];
            const int pg = slot >= 0 ? slot / rope.page_size : 0, off = slot >= 0 ? slot - pg * rope.page_size : 0;
            if (rope_is_v) {
                if (slot < 0) continue;
                const int kh = rope_head - rope.nh - rope.nkvh;
                TC* dst = (TC*)rope.vcache + (((size_t)pg * rope.nkvh + kh) * rope.page_size + off) * rope.dh;
#pragma unroll
                for (int e = 0; e < 4; ++e) { dst[jj + e] = from_f32<TC>(v0[e]); dst[jj + rope.rr + e] = from_f32<TC>(v1[e]); }
                continue;
            }
            const float4 c = *reinterpret_cast<const float4*>(rope.cos_t + (size_t)rope.positions[m] * half + jj);
            const float4 s = *reinterpret_cast<const float4*>(rope.sin_t + (size_t)rope.positions[m] * half + jj);
            const float cc[4] = {c.x, c.y, c.z, c.w}, ss[4] = {s.x, s.y, s.z, s.w};
            TC* dst;
            if (rope_head < rope.nh) dst = C + (size_t)m * ldc + (size_t)rope_head * rope.dh;
            else {
                if (slot < 0) continue;
                dst = (TC*)rope.kcache + (((size_t)pg * rope.nkvh + (rope_head - rope.nh)) * rope.page_size + off) * rope.dh;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                dst[jj + e] = from_f32<TC>(v0[e] * cc[e] - v1[e] * ss[e]);
                dst[jj + half + e] = from_f32<TC>(v0[e] * ss[e] + v1[e] * cc[e]);
            }
        }
        return;
    }
    if (CRESID) {                                       // NT == MT == 1
        const int m = m0 + r;
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float v = acc[0][0][e];
#pragma unroll
            for (int w = 0; w < WPB - 1; ++w) v += red[w][0][lane][e];
            const int n = n0 + 4 * kq + e;
            if (m < M && n < rs_end) {
                const float d = to_f32(from_f32<TC>(alpha * v));     // the branch's output as it would be stored
                const float h = xres[e] + nf.rscale * d;
                nf.x[(size_t)m * nf.ldx + n] = h;
                C[(size_t)m * ldc + n] = from_f32<TC>(h * gres[e]);
                ss += h * h;
            }
        }
        ss += __shfl_xor(ss, 16, kWave);
        ss += __shfl_xor(ss, 32, kWave);
        if (kq == 0) nf.ss_out[blockIdx.x * 16 + r] = ss;
        return;
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m0 + 16 * mt + r;             // column j of D = l % 16
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float v = acc[nt][mt][e];
#pragma unroll
                for (int w = 0; w < WPB - 1; ++w) v += red[w][nt * MT + mt][lane][e];
                const int n = n0 + 16 * nt + 4 * kq + e;    // row i of D
                if (m < M && n < N) C[(size_t)m * ldc + n] = from_f32<TC>(alpha * v);
            }
        }
}

// What a caller of the *_variant entry points (tests and sweeps) asks for.  It holds for that one call on the calling
// thread and changes nothing for any other call: no setting outlives the call that made it.
struct Variant {
    int lines = 1;             // whole-line weight loads (LINES) where the sizes allow; 0: loads in operand layout
    int rope_tile_rows = 0;    // used weight rows per tile of ic_gemm_qkv_rope (16, 8, 4); 0: chosen from the number of heads
};
static thread_local Variant t_variant;
struct VariantScope {
    Variant saved;
    explicit VariantScope(const Variant& v) : saved(t_variant) { t_variant = v; }
    ~VariantScope() { t_variant = saved; }
};
static inline bool lines_apply(bool aligned, int K) { return aligned && t_variant.lines && K % 64 == 0; }

template <typename TC, int NT, int MT, int WPB, int UNROLL, int EPI = 0, bool OWN_K = false, int AG = 1>
static void launch_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                        int ldc, float alpha, bool aligned, const NormFuse& nf, hipStream_t stream, int blocks = 0) {
    dim3 grid(blocks > 0 ? blocks : (N + 16 * NT - 1) / (16 * NT), (M + 16 * MT - 1) / (16 * MT)), block(WPB * 64);
    if constexpr (UNROLL % 2 == 0) {
        if (lines_apply(aligned, K)) {
            hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, NT, MT, WPB, UNROLL, true, EPI, OWN_K, AG, true>), grid, block, 0, stream,
                               (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, alpha, RopeEpilogue{}, nf);
            return;
        }
    }
    if (aligned)
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, NT, MT, WPB, UNROLL, true, EPI, OWN_K, AG>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, alpha, RopeEpilogue{}, nf);
    else
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, NT, MT, WPB, UNROLL, false, EPI, OWN_K, AG>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, alpha, RopeEpilogue{}, nf);
}

// The gate/up projection with the activation in its epilogue: W [N, K] = [gate; up], C [M, N/2].
// G tiles of 16 gate rows (and as many of up rows) per block; `blocks` column blocks share the N/2 columns.
template <typename TC, int WPB, int UN = 2, int G = 1>
static void launch_gemm_swiglu(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                               int ldc, bool aligned, const NormFuse& nf, hipStream_t stream, int blocks = 0) {
    if (blocks <= 0) blocks = (N / 2 + 16 * G - 1) / (16 * G);
    dim3 grid(blocks, (M + 15) / 16), block(WPB * 64);
    constexpr int AG = (UN % 4 == 0) ? 4 : 2;                // up to 4 rows one token load serves AG k-steps
    if (lines_apply(aligned, K)) {
        if (M <= 4 && sizeof(TC) == 2)
            hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, 2 * G, 1, WPB, UN, true, 1, false, AG, true>), grid, block, 0, stream,
                               (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, 1.0f, RopeEpilogue{}, nf);
        else
            hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, 2 * G, 1, WPB, UN, true, 1, false, 1, true>), grid, block, 0, stream,
                               (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, 1.0f, RopeEpilogue{}, nf);
        return;
    }
    if (aligned && M <= 4 && sizeof(TC) == 2)
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, 2 * G, 1, WPB, UN, true, 1, false, AG>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, 1.0f, RopeEpilogue{}, nf);
    else if (aligned)
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, 2 * G, 1, WPB, UN, true, 1>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, 1.0f, RopeEpilogue{}, nf);
    else
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, 2 * G, 1, WPB, UN, false, 1>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, 1.0f, RopeEpilogue{}, nf);
}

// The same for 17..32 rows: two row tiles per block, 8 waves, whole-line weight loads (the caller has checked that they apply).
template <int G>
static void launch_gemm_swiglu_two_tiles(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                                         int ldc, const NormFuse& nf, hipStream_t stream, int blocks = 0) {
    if (blocks <= 0) blocks = (N / 2 + 16 * G - 1) / (16 * G);
    hipLaunchKernelGGL((gemm_nt_bf16_kernel<bf16, 2 * G, 2, 8, 2, true, 1, false, 1, true>), dim3(blocks, 1), dim3(512), 0, stream,
                       (const uint16_t*)A, (const uint16_t*)W, (bf16*)C, M, N, K, lda, ldw, ldc, 1.0f, RopeEpilogue{}, nf);
}

// Compute units of the current device, asked once.
static int compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
        else cus = 256;
    }
    return cus;
}

// Very many weight rows and at most 16 token rows (the output head over the vocabulary): there are enough 16-row
// weight tiles for every wave to own whole tiles, so nothing is summed across waves.  The token rows are staged in
// LDS once per block (zero-filled beyond K; rows padded by 32 bytes: the 16-byte reads of 16 rows by the 16 lanes of a
// k-quarter then run at the full 256 bytes a cycle, with 16 bytes of padding at half of it from 8 rows on); a wave
// walks K in groups of kWideDepth k-steps, with the next group's loads (of the same or of its next tile) issued
// before the current group is used, so its weight stream never pauses between tiles.  A block owns a run of whole
// tiles and its waves equal shares of the run's (tile, group) pairs, so that every wave reads the same number of
// bytes; where a share ends inside a tile, the two waves that hold the tile's halves add them through LDS.
// LINES: the weights come in whole cache lines as in the tiled kernel (a wave load covers 8 rows x 128 bytes, not kept
// in the caches) and pass through 2.3 KB of LDS of the wave's own into operand layout.  Alone, cold, 1 / 8 / 16 rows, a
// float32 result: 122,753 x 2,304 107 / 114 / 122 -> 95 / 101 / 107 us, 73,448 x 4,096 109 / 113 / 116 -> 101 / 101 / 104;
// 73,448 x 1,536 44.5 / 45.9 / 47.8 -> 46.6 / 47.4 / 49.8 (slower), and rows that do not start on a line (50,001 x 1,000)
// 27 -> 36: the launcher takes this way for rows of 4 KB and more that are whole lines.
constexpr int kWideDepth = 8;
constexpr int kWideLdsLimit = 160 * 1024;             // LDS of a compute unit

// WV waves a block: 8 when two blocks' token rows fit a compute unit's LDS, else 16 in one block
template <typename TC, int WV, bool LINES>
__global__ void __launch_bounds__(WV * 64)
gemm_wide_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W, TC* __restrict__ C, int M, int N, int K,
                 int lda, int ldw, int ldc, float alpha, NormFuse nf, int a_stride) {
    extern __shared__ __align__(16) unsigned char wide_smem[];
    uint16_t* As = reinterpret_cast<uint16_t*>(wide_smem);                       // [M][a_stride]
    float* part = reinterpret_cast<float*>(wide_smem + (size_t)M * a_stride * 2);    // [4 WV][16]
    float* rowf_s = part + 4 * WV * 16;                                          // [16]
    // per wave: after the loop the wave's unfinished tile lies here for its neighbour; LINES: during the loop 16 rows of
    // 128 bytes, kLineRowBytes apart, that pass the weights on
    constexpr int kWaveBuf = LINES ? 16 * kLineRowBytes : 64 * 16;
    unsigned char* const line_buf = reinterpret_cast<unsigned char*>(rowf_s + 16) + (size_t)(threadIdx.x >> 6) * kWaveBuf;
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int D = kWideDepth;
    const int steps = (K + 31) >> 5, groups = (steps + D - 1) / D, tiles = (N + 15) >> 4;
    // the block's tiles, and this wave's run of (tile, group) pairs among them
    const int t0 = (int)((long long)blockIdx.x * tiles / gridDim.x), t1 = (int)((long long)(blockIdx.x + 1) * tiles / gridDim.x);
    const int bg = (t1 - t0) * groups;
    const int run0 = (int)((long long)wave * bg / WV), total = (int)((long long)(wave + 1) * bg / WV) - run0;
    const int klast = K - 8;                                 // the last whole 16 bytes of a weight row
    // group L of this wave's run (clamped to its last one, so that loads are never conditional): weights only;
    // columns beyond K repeat the row's last 16 bytes and meet zeros of the staged token rows
    // LINES: w[2 j + h]: lane l holds 16 bytes of row 8 h + l / 8 of the tile, at byte 16 (l % 8) of the 128 that k-steps
    // 2 j and 2 j + 1 of the group cover; else w[u] is the lane's operand of k-step u
    auto issue = [&](uint4 (&w)[D], int L) {
        L = run0 + (L < total ? L : total - 1);
        const int ti = L / groups, g = L - ti * groups;
        if constexpr (!LINES) {
            const int n = (t0 + ti) * 16 + r;
            const uint16_t* p = W + (size_t)(n < N ? n : N - 1) * ldw;
#pragma unroll
            for (int u = 0; u < D; ++u) {
                const int k = 32 * (g * D + u) + 8 * kq;
                w[u] = *reinterpret_cast<const uint4*>(p + (k < klast ? k : klast));
            }
            return;
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int n = (t0 + ti) * 16 + 8 * h + (lane >> 3);
            const uint16_t* p = W + (size_t)(n < N ? n : N - 1) * ldw;
#pragma unroll
            for (int j = 0; j < D / 2; ++j) {
                const int k = 32 * (g * D + 2 * j) + 8 * (lane & 7);
                w[2 * j + h] = load_stream16(p + (k < klast ? k : klast));
            }
        }
    };
    uint4 w0[D], w1[D];
    if (total > 0) issue(w0, 0);                             // the weights do not wait for the token rows
    const int chunks = a_stride >> 3;                        // 16-byte pieces of a staged row
    for (int m = wave; m < M; m += WV) {                     // a wave stages whole rows, four loads at a time
        const uint16_t* src = A + (size_t)m * lda;
        uint16_t* dst = As + (size_t)m * a_stride;
        for (int c0 = lane; c0 < chunks; c0 += 256) {
            uint4 v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = c0 + 64 * j;
                v[j] = make_uint4(0u, 0u, 0u, 0u);
                if (8 * c + 8 <= K) v[j] = *reinterpret_cast<const uint4*>(src + 8 * c);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (c0 + 64 * j < chunks) *reinterpret_cast<uint4*>(dst + 8 * (c0 + 64 * j)) = v[j];
        }
    }
    if (nf.ss_in) {
        float t = 0.f;
        for (int b = tid >> 4; b < nf.n_parts_in; b += 4 * WV) t += nf.ss_in[b * 16 + (tid & 15)];
        part[(tid >> 4) * 16 + (tid & 15)] = t;
    }
    __syncthreads();
    if (tid < 16) {
        float f = 1.0f;
        if (nf.ss_in) {
            float t = 0.f;
            for (int j = 0; j < 4 * WV; ++j) t += part[j * 16 + tid];
            f = rsqrtf(t * nf.inv_width + nf.eps);
        }
        rowf_s[tid] = f;
    }
    __syncthreads();
    const float scale = alpha * rowf_s[r];                   // column j = r of D is token row r
    const uint16_t* arow = As + (size_t)(r < M ? r : M - 1) * a_stride + 8 * kq;

    // D[i = 4 kq + e][j = r]: weight row 16 tile + 4 kq + e, token row r
    auto store = [&](int tile, const v4f& v) {
        if (r < M) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = tile * 16 + 4 * kq + e;
                if (n < N) C[(size_t)r * ldc + n] = from_f32<TC>(scale * v[e]);
            }
        }
    };
    v4f acc = v4f{0.f, 0.f, 0.f, 0.f}, tail_acc = acc;
    int ct = t0 + run0 / groups, cg = run0 - (run0 / groups) * groups;       // tile and group the next use belongs to
    // A run that begins inside a tile holds that tile's tail; its head is the end of the previous wave's run.
    const bool has_tail = total > 0 && cg != 0;
    const int tail_tile = ct;
    bool in_tail = has_tail;
    auto use = [&](const uint4 (&w)[D]) {
        typedef __bf16 v8b __attribute__((ext_vector_type(8)));
        if constexpr (!LINES) {
#pragma unroll
            for (int u = 0; u < D; ++u) {
                const uint4 a = *reinterpret_cast<const uint4*>(arow + 32 * (cg * D + u));
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, w[u]), __builtin_bit_cast(v8b, a), acc, 0, 0, 0);
            }
        } else {
#pragma unroll
        for (int j = 0; j < D / 2; ++j) {
            // in as rows of 128 bytes, out as the operands of the pair's two k-steps; LDS serves a wave's requests in order
#pragma unroll
            for (int h = 0; h < 2; ++h)
                *reinterpret_cast<uint4*>(line_buf + (8 * h + (lane >> 3)) * kLineRowBytes + 16 * (lane & 7)) = w[2 * j + h];
            __builtin_amdgcn_wave_barrier();
            uint4 w2[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) w2[e] = *reinterpret_cast<const uint4*>(line_buf + r * kLineRowBytes + 16 * (4 * e + kq));
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const uint4 a = *reinterpret_cast<const uint4*>(arow + 32 * (cg * D + 2 * j + e));
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, w2[e]), __builtin_bit_cast(v8b, a), acc, 0, 0, 0);
            }
        }
        }
        if (++cg == groups) {
            if (in_tail) { tail_acc = acc; in_tail = false; }
            else store(ct, acc);
            acc = v4f{0.f, 0.f, 0.f, 0.f};
            cg = 0;
            ++ct;
        }
    };
    for (int L = 0; L < total; L += 2) {
        issue(w1, L + 1);
        use(w0);
        issue(w0, L + 2);
        if (L + 1 < total) use(w1);
    }
    // The launcher gives every wave at least `groups` pairs, so a tile is shared by two waves at most: the head
    // goes through LDS to the wave that holds the tail, which adds the two in this order and stores.
    if (total > 0 && cg != 0) reinterpret_cast<v4f*>(line_buf)[lane] = acc;
    __syncthreads();
    if (has_tail) {
        const v4f h = reinterpret_cast<const v4f*>(line_buf - kWaveBuf)[lane];     // (the wave before this one)
        store(tail_tile, h + tail_acc);
    }
}

// false when the wide kernel does not take the shape.
template <typename TC>
static bool launch_gemm_wide(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                             float alpha, const NormFuse& nf, hipStream_t stream) {
    const int steps = (K + 31) / 32, groups = (steps + kWideDepth - 1) / kWideDepth;
    const int a_stride = groups * kWideDepth * 32 + 16;
    const size_t rows_bytes = (size_t)M * a_stride * 2;
    const bool lines = t_variant.lines && K >= 2048 && K % 64 == 0 && ldw % 64 == 0 && ((uintptr_t)W & 127) == 0;
    auto lds_of = [&](int wv) { return rows_bytes + (4 * wv * 16 + 16) * sizeof(float) + (size_t)wv * (lines ? 16 * kLineRowBytes : 64 * 16); };
    // two blocks of 8 waves a compute unit; with many or long token rows one block of 16 waves, or of 8 when only that fits
    const bool two = 2 * lds_of(8) <= (size_t)kWideLdsLimit;
    const int wv = (two || lds_of(16) > (size_t)kWideLdsLimit) ? 8 : 16;
    const size_t lds = lds_of(wv);
    if (M > 16 || K < 8 || K % 8 || lds > (size_t)kWideLdsLimit) return false;
    static bool raised[2][2][2][64] = {};                    // per kernel and device: it may use more than 64 KB of LDS
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    bool& done = raised[sizeof(TC) == 2 ? 1 : 0][wv == 8 ? 1 : 0][lines ? 1 : 0][dev];
    const void* fn = wv == 8 ? (lines ? (const void*)gemm_wide_kernel<TC, 8, true> : (const void*)gemm_wide_kernel<TC, 8, false>)
                             : (lines ? (const void*)gemm_wide_kernel<TC, 16, true> : (const void*)gemm_wide_kernel<TC, 16, false>);
    if (!done) {
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kWideLdsLimit) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        done = true;
    }
    // as many blocks as are resident at once, each with a whole number of tiles and at least one tile per wave
    const int tiles = (N + 15) / 16, cus = compute_units();
    int blocks = cus * (two ? 2 : 1);
    if (blocks > tiles / wv) blocks = tiles / wv;
    if (blocks < 1) return false;
#define IC_WIDE(WV, LN)                                                                                                   \
    hipLaunchKernelGGL((gemm_wide_kernel<TC, WV, LN>), dim3(blocks), dim3(WV * 64), lds, stream, (const uint16_t*)A, \
                       (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, alpha, nf, a_stride)
    if (wv == 8) { if (lines) IC_WIDE(8, true); else IC_WIDE(8, false); }
    else { if (lines) IC_WIDE(16, true); else IC_WIDE(16, false); }
#undef IC_WIDE
    return true;
}

// NT weight tiles of 16 rows share one load of the A fragments; WPB waves split K.  Both are
// chosen so that (column blocks x waves) fills the chip's SIMDs about twice over.
template <typename TC>
static void dispatch_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                          int ldc, float alpha, bool aligned, const NormFuse& nf, hipStream_t stream) {
    const int tiles = (N + 15) / 16;
#define IC_GO(NT, MT, WPB, UN) launch_gemm<TC, NT, MT, WPB, UN>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, nf, stream)
    // tilings from a sweep over the projection shapes of 1B..8B models on MI355X
    if (M <= 16 && tiles >= 2048 && aligned &&
        launch_gemm_wide<TC>(A, W, C, M, N, K, lda, ldw, ldc, alpha, nf, stream)) return;
    if (M <= 16) {
        if (tiles < 400) IC_GO(1, 1, 16, 4);
        else if (tiles < 600) IC_GO(2, 1, 16, 4);
        else if (tiles < 2048) { if (M <= 4) IC_GO(1, 1, 8, 2); else IC_GO(1, 1, 4, 2); }
        else { if (M <= 8) IC_GO(1, 1, 16, 2); else IC_GO(4, 1, 4, 2); }
    } else if (M <= 32) {
        if (tiles < 600) IC_GO(1, 2, 8, 2);
        else IC_GO(2, 2, 4, 2);
    } else {
        if (tiles < 256) IC_GO(1, 4, 8, 1);
        else IC_GO(2, 4, 4, 1);
    }
#undef IC_GO
}

// The same product with the tiling chosen by the caller (for tuning and tests):
// nt in {1, 2, 4}, wpb in {4, 8, 16}, unroll in {2, 4}; mt follows from M.
template <typename TC, int NT, int WPB, int UN>
static int launch_cfg_m(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                        float alpha, bool aligned, hipStream_t stream) {
    if (M <= 16) launch_gemm<TC, NT, 1, WPB, UN>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, NormFuse{}, stream);
    else if (M <= 32) launch_gemm<TC, NT, 2, WPB, (UN > 2 ? 2 : UN)>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, NormFuse{}, stream);
    else {
        if (NT * WPB > 32) return IC_ERR_UNSUPPORTED;       // would not fit LDS
        launch_gemm<TC, (NT > 2 ? 2 : NT), 4, (WPB > 8 ? 8 : WPB), 1>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, NormFuse{}, stream);
    }
    return IC_OK;
}

IC_EXPORT int ic_gemm_nt_cfg(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda,
                             int ldw, int ldc, float alpha, int nt, int wpb, int unroll, hipStream_t stream) {
    if (M <= 0 || N <= 0) return IC_OK;
    if (K <= 0 || lda < K || ldw < K || c_dtype != IC_BF16) return IC_ERR_ARG;
    const bool aligned = (lda % 8 == 0) && (ldw % 8 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)W & 15) == 0);
    if (nt == 0) {                                  // nt == 0: the variant with SwiGLU in the epilogue
        if (M > 16 || (N & 1) || ldc < N / 2) return IC_ERR_ARG;
#define IC_SW(WPB, UN) if (wpb == WPB && unroll == UN) { launch_gemm_swiglu<bf16, WPB, UN>(A, W, C, M, N, K, lda, ldw, ldc, aligned, NormFuse{}, stream); return ic_launch_status(); }
        IC_SW(4, 2) IC_SW(4, 4) IC_SW(8, 2) IC_SW(8, 4) IC_SW(16, 2) IC_SW(16, 4)
#undef IC_SW
        return IC_ERR_UNSUPPORTED;
    }
    if (nt == -2) {                                 // the SwiGLU variant with two tiles per block, one block per compute unit
        if (M > 16 || (N & 1) || ldc < N / 2) return IC_ERR_ARG;
        const int cols = (N / 2 + compute_units() - 1) / compute_units();
        if (cols > 32) return IC_ERR_UNSUPPORTED;
        const int blocks = (N / 2 + cols - 1) / cols;
#define IC_SW(WPB, UN) if (wpb == WPB && unroll == UN) { launch_gemm_swiglu<bf16, WPB, UN, 2>(A, W, C, M, N, K, lda, ldw, ldc, aligned, NormFuse{}, stream, blocks); return ic_launch_status(); }
        IC_SW(4, 2) IC_SW(4, 4) IC_SW(8, 2) IC_SW(8, 4) IC_SW(16, 2)
#undef IC_SW
        return IC_ERR_UNSUPPORTED;
    }
    if (ldc < N) return IC_ERR_ARG;
    int st = IC_ERR_UNSUPPORTED;
#define IC_CFG(NT, WPB, UN) \
    if (nt == NT && wpb == WPB && unroll == UN) st = launch_cfg_m<bf16, NT, WPB, UN>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    IC_CFG(1, 4, 2) IC_CFG(1, 4, 4) IC_CFG(1, 8, 2) IC_CFG(1, 8, 4) IC_CFG(1, 16, 2) IC_CFG(1, 16, 4)
    IC_CFG(2, 4, 2) IC_CFG(2, 4, 4) IC_CFG(2, 8, 2) IC_CFG(2, 8, 4) IC_CFG(2, 16, 2) IC_CFG(2, 16, 4)
    IC_CFG(4, 4, 2) IC_CFG(4, 8, 2)
#undef IC_CFG
    if (st) return st;
    return ic_launch_status();
}

// Rows that the products with an epilogue take for this K and these row strides: 32 for kind 1 (SwiGLU) and kind 2 (rotary
// and cache write) where the weights can be read in whole cache lines (K a multiple of 64, strides multiples of 8: two row
// tiles per block), 16 otherwise.  Measured inside recorded steps of the 2B shape at batch 24 against the library's product
// followed by the kernel the epilogue replaces: QKV 12.7 us against 10.4 + 4.7, gate/up 14.4 against 13.8 + 4.8.  With four
// row tiles (64 rows) the QKV product took 20.5 us against 13.1 + 4.9, and gate/up 27..31 against 19.8 + 4.7: not built in.
IC_EXPORT int ic_gemm_nt_epilogue_rows(int kind, int K, int lda, int ldw) {
    const bool lines = lines_apply(lda % 8 == 0 && ldw % 8 == 0, K);
    return (kind == 1 || kind == 2) && lines ? 32 : 16;
}

IC_EXPORT int ic_gemm_nt_supported(int a_dtype, int w_dtype, int c_dtype) {
    return a_dtype == IC_BF16 && w_dtype == IC_BF16 && (c_dtype == IC_F32 || c_dtype == IC_BF16);
}

// Fills the kernel's description of a split norm from the C structs; false: an argument fault.
static bool norm_fuse_args(const IcRowFactor* rf, const IcResidualNorm* tail, int M, int N, int K, int c_dtype,
                           int col_blocks, NormFuse& nf) {
    if (rf) {
        if (M > 16 || !rf->sumsq || rf->n_parts <= 0 || rf->n_parts > kMaxSumParts || rf->width <= 0) return false;
        nf.ss_in = rf->sumsq; nf.n_parts_in = rf->n_parts; nf.inv_width = 1.0f / (float)rf->width; nf.eps = rf->eps;
    }
    if (tail) {
        if (M > 16 || c_dtype != IC_BF16 || !tail->x || !tail->weight || !tail->sumsq_out || tail->ldx < N ||
            tail->n_parts != col_blocks || col_blocks > kMaxSumParts) return false;
        nf.x = tail->x; nf.ldx = tail->ldx; nf.g = tail->weight; nf.rscale = tail->alpha; nf.ss_out = tail->sumsq_out;
    }
    return true;
}

// Column blocks (= sums of squares per row) that c_mode 2 writes for an N wide product.
// (one block per compute unit when 16-column tiles would be fewer than the units)
static int compute_units();
IC_EXPORT int ic_gemm_nt_residual_parts(int N) {
    const int tiles = (N + 15) / 16, cus = compute_units();
    if (tiles >= cus || N <= 0) return tiles;
    const int cols = (N + cus - 1) / cus;
    return (N + cols - 1) / cols;
}

// c_mode 0: C [M, N] = alpha * A W^T.  c_mode 1 (M <= 16, N even, alpha ignored): W = [gate; up] and
// C [M, N/2] = up * silu(gate), both projections rounded to C's type before the activation.
// c_mode 2 (M <= 16, bfloat16 C, `tail` given): x += tail->alpha * (alpha * A W^T); C = x * tail->weight;
// tail->sumsq_out[b * 16 + m] = sum of x[m]^2 over column block b.  row_factor (M <= 16, any c_mode): row m
// of the product is multiplied by rsqrt(sum_b sumsq[b * 16 + m] / width + eps) first.
IC_EXPORT int ic_gemm_nt(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                         int M, int N, int K, int lda, int ldw, int ldc, float alpha, int c_mode,
                         const IcRowFactor* row_factor, const IcResidualNorm* tail, hipStream_t stream) {
    if (M <= 0 || N <= 0) return IC_OK;
    if (K <= 0 || lda < K || ldw < K || c_mode < 0 || c_mode > 2) return IC_ERR_ARG;
    if (c_mode == 1 ? ((N & 1) || ldc < N / 2) : (ldc < N)) return IC_ERR_ARG;
    if ((c_mode == 2) != (tail != nullptr)) return IC_ERR_ARG;
    if (!ic_gemm_nt_supported(a_dtype, w_dtype, c_dtype)) return IC_ERR_UNSUPPORTED;
    if ((M + 63) / 64 > 65535) return IC_ERR_ARG;
    NormFuse nf{};
    if (!norm_fuse_args(row_factor, tail, M, N, K, c_dtype, ic_gemm_nt_residual_parts(N), nf)) return IC_ERR_ARG;
    const bool aligned = (lda % 8 == 0) && (ldw % 8 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)W & 15) == 0);
    if (c_mode == 1 && M > 16 && (M > 32 || c_dtype != IC_BF16 || row_factor || !lines_apply(aligned, K))) return IC_ERR_ARG;
    if (c_mode == 2) {
        // 16 waves a block throughout; up to 4 rows 4 k-steps in flight, above that 2 (from a sweep over the O and
        // down projections of the 1B..8B shapes with one block per compute unit)
        const int blocks = ic_gemm_nt_residual_parts(N);
        // rows of 16 KB and more: a wave owns one stretch of every row (8B shape's down projection: 36 -> 30 us)
        // up to 8 (4) rows one load of the token operand serves 2 (4) k-steps
#define IC_RES(UN, OWN, AG) launch_gemm<bf16, 1, 1, 16, UN, 3, OWN, AG>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, nf, stream, blocks)
        if (K >= kOwnKFrom) { if (M <= 8) IC_RES(2, true, 2); else IC_RES(2, true, 1); }
        else if (M > 8) IC_RES(2, false, 1);
        else if (M > 4) IC_RES(2, false, 2);
        else IC_RES(4, false, 4);
#undef IC_RES
        return ic_launch_status();
    }
    if (c_mode == 1) {
        const int tiles = (N / 2 + 15) / 16, cus = compute_units();
        // Between one and two 16-column tiles per compute unit the second round of blocks would be part-filled:
        // then every block takes ceil(columns / units) columns (two tiles, the second one partial) and one round does it.
        const int cols = (N / 2 + cus - 1) / cus;
        const bool one_round = tiles > cus && cols <= 32;
        const int blocks = one_round ? (N / 2 + cols - 1) / cols : 0;
        if (M > 16) {
            if (one_round) launch_gemm_swiglu_two_tiles<2>(A, W, C, M, N, K, lda, ldw, ldc, nf, stream, blocks);
            else launch_gemm_swiglu_two_tiles<1>(A, W, C, M, N, K, lda, ldw, ldc, nf, stream);
        } else if (c_dtype == IC_F32) {
            if (one_round) launch_gemm_swiglu<float, 8, 2, 2>(A, W, C, M, N, K, lda, ldw, ldc, aligned, nf, stream, blocks);
            else if (tiles < 300) launch_gemm_swiglu<float, 8>(A, W, C, M, N, K, lda, ldw, ldc, aligned, nf, stream);
            else launch_gemm_swiglu<float, 16, 4>(A, W, C, M, N, K, lda, ldw, ldc, aligned, nf, stream);
        } else {
            if (one_round) launch_gemm_swiglu<bf16, 8, 2, 2>(A, W, C, M, N, K, lda, ldw, ldc, aligned, nf, stream, blocks);
            else if (tiles < 300) launch_gemm_swiglu<bf16, 8>(A, W, C, M, N, K, lda, ldw, ldc, aligned, nf, stream);
            // many tiles (8B shape): 16 waves (61 -> 55 us against 4); with whole-line weight loads two k-steps in flight
            // per wave do better than four (batch 8: 1.266 -> 1.237 ms for 10 layers)
            else if (lines_apply(aligned, K)) launch_gemm_swiglu<bf16, 16, 2>(A, W, C, M, N, K, lda, ldw, ldc, aligned, nf, stream);
            else launch_gemm_swiglu<bf16, 16, 4>(A, W, C, M, N, K, lda, ldw, ldc, aligned, nf, stream);
        }
        return ic_launch_status();
    }
    if (c_dtype == IC_F32) dispatch_gemm<float>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, nf, stream);
    else dispatch_gemm<bf16>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, nf, stream);
    return ic_launch_status();
}

// The fused QKV projection of few rows (M <= 16) with the rotary encoding and the cache write in
// its epilogue: q heads land rotated in C[M, >= nh*dh] (row stride ldc), k heads rotated and v
// heads as they are in the token's cache slot.  bfloat16 throughout; full rotary (rot == dh);
// dh a multiple of 32.  W: [(nh + 2 nkvh) * dh, K].
IC_EXPORT int ic_gemm_qkv_rope_supported(int dtype, int dh) { return dtype == IC_BF16 && dh >= 32 && dh % 32 == 0; }

IC_EXPORT int ic_gemm_qkv_rope(const void* A, const void* W, void* C, int M, int K, int lda, int ldw, int ldc,
                               const int* positions, const int* slots, const float* cos_t, const float* sin_t,
                               void* kcache, void* vcache, int nh, int nkvh, int dh, int page_size,
                               const IcRowFactor* row_factor, hipStream_t stream) {
    if (M <= 0) return IC_OK;
    if (M > 32 || K <= 0 || lda < K || ldw < K || nh <= 0 || nkvh <= 0 || page_size <= 0 || ldc < nh * dh) return IC_ERR_ARG;
    if (!ic_gemm_qkv_rope_supported(IC_BF16, dh)) return IC_ERR_UNSUPPORTED;
    if (((uintptr_t)cos_t & 15) || ((uintptr_t)sin_t & 15)) return IC_ERR_ARG;
    const bool aligned = (lda % 8 == 0) && (ldw % 8 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)W & 15) == 0);
    // 17..32 rows: two row tiles per block, with whole-line weight loads only and no row factors
    if (M > 16 && (row_factor || !lines_apply(aligned, K))) return IC_ERR_ARG;
    // rows per tile: few heads make few blocks of 16 + 16 rows; tiles of 8 or 4 used rows make two or four times as
    // many.  The unused rows still cost load cycles, so it pays only well below one block per compute unit
    // (measured: 80 blocks on 256 units 7.6 -> 6.9 us with 8 rows; 144 blocks 16.1 -> 19.6, slower).
    const int pairs16 = (nh + 2 * nkvh) * (dh / 32), cus = compute_units();
    int rr = 16;
    if (t_variant.rope_tile_rows) rr = t_variant.rope_tile_rows;
    else if (5 * pairs16 < 2 * cus) rr = (6 * pairs16 <= cus) ? 4 : 8;
    const RopeEpilogue rope{positions, slots, cos_t, sin_t, kcache, vcache, nh, nkvh, dh, page_size, rr};
    const int N = (nh + 2 * nkvh) * dh;
    NormFuse nf{};
    if (!norm_fuse_args(row_factor, nullptr, M, N, K, IC_BF16, 0, nf)) return IC_ERR_ARG;
    const int blocks = pairs16 * (16 / rr);
    dim3 grid(blocks, 1);
#define IC_ROPE(WPB, UN, AL)                                                                             \
    hipLaunchKernelGGL((gemm_nt_bf16_kernel<bf16, 2, 1, WPB, UN, AL, 2>), grid, dim3(WPB * 64), 0, stream, \
                       (const uint16_t*)A, (const uint16_t*)W, (bf16*)C, M, N, K, lda, ldw, ldc, 1.0f, rope, nf)
    // 8 waves, 4 steps in flight: within 4 % of the best tiling at every shape swept, and it does not spill
    if (M > 16)
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<bf16, 2, 2, 8, 4, true, 2, false, 1, true>), grid, dim3(8 * 64), 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (bf16*)C, M, N, K, lda, ldw, ldc, 1.0f, rope, nf);
    else if (lines_apply(aligned, K)) {
        if (M <= 4)
            hipLaunchKernelGGL((gemm_nt_bf16_kernel<bf16, 2, 1, 8, 4, true, 2, false, 4, true>), grid, dim3(8 * 64), 0, stream,
                               (const uint16_t*)A, (const uint16_t*)W, (bf16*)C, M, N, K, lda, ldw, ldc, 1.0f, rope, nf);
        else
            hipLaunchKernelGGL((gemm_nt_bf16_kernel<bf16, 2, 1, 8, 4, true, 2, false, 1, true>), grid, dim3(8 * 64), 0, stream,
                               (const uint16_t*)A, (const uint16_t*)W, (bf16*)C, M, N, K, lda, ldw, ldc, 1.0f, rope, nf);
    } else if (aligned && M <= 4)                           // one token load serves the 4 k-steps of an iteration
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<bf16, 2, 1, 8, 4, true, 2, false, 4>), grid, dim3(8 * 64), 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (bf16*)C, M, N, K, lda, ldw, ldc, 1.0f, rope, nf);
    else if (aligned) IC_ROPE(8, 4, true);
    else IC_ROPE(8, 4, false);
#undef IC_ROPE
    return ic_launch_status();
}

// ---- the same entry points with a variant named by the caller (tests and sweeps; see infinicore_infer_variants.h) ----------
IC_EXPORT int ic_gemm_nt_variant(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype, int M, int N, int K,
                                 int lda, int ldw, int ldc, float alpha, int c_mode, const IcRowFactor* row_factor,
                                 const IcResidualNorm* tail, int whole_lines, hipStream_t stream) {
    Variant v;
    v.lines = whole_lines ? 1 : 0;
    VariantScope scope(v);
    return ic_gemm_nt(A, a_dtype, W, w_dtype, C, c_dtype, M, N, K, lda, ldw, ldc, alpha, c_mode, row_factor, tail, stream);
}

IC_EXPORT int ic_gemm_qkv_rope_variant(const void* A, const void* W, void* C, int M, int K, int lda, int ldw, int ldc,
                                       const int* positions, const int* slots, const float* cos_t, const float* sin_t,
                                       void* kcache, void* vcache, int nh, int nkvh, int dh, int page_size,
                                       const IcRowFactor* row_factor, int tile_rows, hipStream_t stream) {
    if (tile_rows != 0 && tile_rows != 4 && tile_rows != 8 && tile_rows != 16) return IC_ERR_ARG;
    Variant v;
    v.rope_tile_rows = tile_rows;
    VariantScope scope(v);
    return ic_gemm_qkv_rope(A, W, C, M, K, lda, ldw, ldc, positions, slots, cos_t, sin_t, kcache, vcache, nh, nkvh, dh, page_size,
                            row_factor, stream);
}

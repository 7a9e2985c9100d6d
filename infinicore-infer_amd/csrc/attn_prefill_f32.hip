// Attention of prompt portions over the paged cache in true float32 on the matrix cores
// (v_mfma_f32_32x32x2_f32: float32 operands, float32 accumulation, no reduced-precision mode).
//
// The 32-bit path's prompts otherwise run in the general kernel, one wave per (token, head) with scalar
// dot products: 3.5 ms a layer for a 2,048-token prompt of the 2B shape, two thirds of that path's prompt
// time.  Here a block of four waves owns up to 128 consecutive tokens of one request and one head, wave w
// rows 32 w .. 32 w + 31, and walks the keys 64 at a time through LDS, as the bfloat16 kernel does; the
// tile list is the same.  Scores are computed transposed, S^T = K Q^T, so a lane holds 32 keys of ONE query
// and the running softmax needs a single cross-lane step; the probabilities are then already the B operand
// of O^T = V^T P^T.
//
// 32x32x2 operand layout (lane l, h = l / 32): A[i = l % 32][k = h], B[k = h][j = l % 32],
// D[i = 8 (r / 4) + 4 h + r % 4][j = l % 32] for the 16 accumulators r.  Which two values of the summed
// dimension an instruction takes is free as long as A and B agree: in S^T = K Q^T instruction c takes head
// dims c and c + DH / 2 (so a lane's K operands are DH / 2 consecutive floats of its key's row), and in
// O^T = V^T P^T accumulator r of S^T is the B operand as it stands: it holds key 8 (r / 4) + r % 4 in the
// lower half of the wave and the key four further on in the upper half.
//
// Simple on purpose (the 32-bit path is for checking): one wave group, no cut walks, a tile is loaded
// when it is needed (the float32 matrix instructions take 16 times as long as the bfloat16 ones, so the
// loop is bound by them, not by the loads).
//
// Cache layout of one layer: K and V planes [num_pages, n_kv_heads, page_size, head_dim].
#include "common.h"

typedef float f32_v16 __attribute__((ext_vector_type(16)));

constexpr int kF32Threads = 256;
constexpr int kF32Rows = 128;     // query rows per block (must equal the bfloat16 kernel's tile height: one tile list serves both)
constexpr int kF32Keys = 64;      // keys per step

template <int DH>
__global__ void __launch_bounds__(kF32Threads, 2)
attn_prefill_f32_kernel(const float* __restrict__ q, int q_stride, float* __restrict__ out, int out_stride,
                        const float* __restrict__ kcache, const float* __restrict__ vcache,
                        const int* __restrict__ block_tables, int bt_stride, const int4* __restrict__ tiles,
                        int n_tiles, int nh, int nkvh, int page_shift, float scale_log2e, int window) {
    constexpr int HALF = DH / 2;          // matrix instructions per 32-key tile of S^T
    constexpr int ND = DH / 32;           // 32-row tiles of O^T
    constexpr int KS = DH + 4;            // row stride of the K tile (floats): 16-byte reads of 16 consecutive rows cover all banks
    constexpr int VS = DH + 8;            // row stride of the V tile: rows four apart (the wave's two halves) fall into different banks
    constexpr int NL = kF32Keys * (DH / 4) / kF32Threads;     // 16-byte loads per thread and plane
    __shared__ __attribute__((aligned(16))) float Ks[kF32Keys * KS];
    __shared__ __attribute__((aligned(16))) float Vs[kF32Keys * VS];

    const int slot = (int)blockIdx.x;                   // tile-major: all heads of the longest tile first
    const int h = slot % nh;
    const int4 tile = tiles[slot / nh];
    const int req = tile.x, row0 = tile.y, n_rows = tile.z, pos0 = tile.w;
    const int kvh = h / (nh / nkvh);
    const int* bt = block_tables + (size_t)req * bt_stride;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    const int page_size = 1 << page_shift, page_mask = page_size - 1;

    const int my_row = 32 * wave + lq;
    const bool row_ok = my_row < n_rows;
    const int qpos = pos0 + my_row;
    const bool wave_ok = 32 * wave < n_rows;
    const int wave_first = pos0 + 32 * wave;
    const int wave_last = pos0 + ((32 * wave + 31 < n_rows - 1) ? 32 * wave + 31 : n_rows - 1);
    const int last_key = pos0 + n_rows - 1;
    int first_key = 0;
    if (window > 0 && pos0 - window + 1 > 0) first_key = pos0 - window + 1;
    const int kb_begin = (first_key / kF32Keys) * kF32Keys;

    // Q operands: Q[query lq][HALF * half + c], scores in units of log 2 (the softmax scale folded in)
    float qf[HALF];
    {
        const float* qp = q + (size_t)(row0 + (row_ok ? my_row : 0)) * q_stride + (size_t)h * DH + HALF * half;
#pragma unroll
        for (int c = 0; c < HALF; c += 4) {
            const float4 v = *reinterpret_cast<const float4*>(qp + c);
            qf[c] = row_ok ? v.x * scale_log2e : 0.f; qf[c + 1] = row_ok ? v.y * scale_log2e : 0.f;
            qf[c + 2] = row_ok ? v.z * scale_log2e : 0.f; qf[c + 3] = row_ok ? v.w * scale_log2e : 0.f;
        }
    }
    f32_v16 oacc[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, l = 0.f;

    const size_t head_stride = (size_t)page_size * DH;
    const float* kbase = kcache + (size_t)kvh * head_stride;
    const float* vbase = vcache + (size_t)kvh * head_stride;
    const size_t page_stride = (size_t)nkvh * head_stride;

    for (int kb = kb_begin; kb <= last_key; kb += kF32Keys) {
        __syncthreads();                                // the previous step's readers are done
        // the step's 64 keys and values into LDS as rows (keys outside the tile's range as zeros: they are masked)
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int idx = tid + i * kF32Threads;
            const int key = idx / (DH / 4), quad = idx - key * (DH / 4);
            const int ka = kb + key;
            float4 kv = make_float4(0.f, 0.f, 0.f, 0.f), vv = kv;
            if (ka <= last_key && ka >= first_key) {
                const size_t off = (size_t)bt[ka >> page_shift] * page_stride + (size_t)(ka & page_mask) * DH + quad * 4;
                kv = *reinterpret_cast<const float4*>(kbase + off);
                vv = *reinterpret_cast<const float4*>(vbase + off);
            }
            *reinterpret_cast<float4*>(&Ks[key * KS + quad * 4]) = kv;
            *reinterpret_cast<float4*>(&Vs[key * VS + quad * 4]) = vv;
        }
        __syncthreads();
        if (!wave_ok || kb > wave_last) continue;       // nothing this wave may see
        if (window > 0 && kb + kF32Keys - 1 < wave_first - window + 1) continue;

        // ---- S^T = K Q^T : two tiles of 32 keys ----------------------------------------------------------
        f32_v16 sacc[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[tt][r] = 0.f;
            const float* kp = &Ks[(32 * tt + lq) * KS + HALF * half];
#pragma unroll
            for (int c = 0; c < HALF; c += 4) {
                const float4 kx = *reinterpret_cast<const float4*>(kp + c);
                sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kx.x, qf[c], sacc[tt], 0, 0, 0);
                sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kx.y, qf[c + 1], sacc[tt], 0, 0, 0);
                sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kx.z, qf[c + 2], sacc[tt], 0, 0, 0);
                sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kx.w, qf[c + 3], sacc[tt], 0, 0, 0);
            }
        }
        // ---- mask (only steps that touch the diagonal, the window's edge, or keys before the window) --------
        const bool need_mask = (kb + kF32Keys - 1 > wave_first) || (window > 0);
        if (need_mask) {
            // key kb + 4 half + e of this lane's accumulator (e a constant per accumulator) is seen when e <= lim
            const int lim = qpos - kb - 4 * half;
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (32 * tt + 8 * (r >> 2) + (r & 3) > lim) sacc[tt][r] = -INFINITY;
            if (window > 0) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (32 * tt + 8 * (r >> 2) + (r & 3) <= lim - window) sacc[tt][r] = -INFINITY;
            }
        }
        // ---- running softmax, base 2 -------------------------------------------------------------------
        float mloc = sacc[0][0];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, sacc[tt][r]);
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
        const float m_new = fmaxf(m, mloc);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = exp2f(m - m_use);            // 0 on the first step (m = -inf)
        float rs = 0.f;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = exp2f(sacc[tt][r] - m_use);
                sacc[tt][r] = p;
                rs += p;
            }
        rs += __shfl_xor(rs, 32, kWave);
        l = l * corr + rs;
        m = m_new;
#pragma unroll
        for (int i = 0; i < ND; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= corr;

        // ---- O^T += V^T P^T : accumulator r of S^T is the B operand as it stands -------------------------------
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float* vp = &Vs[(32 * tt + 8 * (r >> 2) + 4 * half + (r & 3)) * VS + lq];
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
                    oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[32 * dt], sacc[tt][r], oacc[dt], 0, 0, 0);
            }
    }

    if (!row_ok) return;
    const float inv = 1.0f / l;
    float* op = out + (size_t)(row0 + my_row) * out_stride + (size_t)h * DH;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            const int d = 32 * dt + 8 * rg + 4 * half;
            *reinterpret_cast<float4*>(op + d) = make_float4(oacc[dt][4 * rg] * inv, oacc[dt][4 * rg + 1] * inv,
                                                             oacc[dt][4 * rg + 2] * inv, oacc[dt][4 * rg + 3] * inv);
        }
}

// Called by ic_attn_prefill_split for float32 (attn_prefill_mfma.hip): the arguments are checked there.
int ic_attn_prefill_f32_launch(const void* q, int q_stride, void* out, int out_stride, const void* kcache, const void* vcache,
                               const int* block_tables, int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh,
                               int page_shift, float scale, int window, hipStream_t stream) {
    if (q_stride % 4 || out_stride % 4 || ((uintptr_t)q & 15) || ((uintptr_t)out & 15) || ((uintptr_t)kcache & 15) ||
        ((uintptr_t)vcache & 15) || ((uintptr_t)tiles & 15))
        return IC_ERR_ARG;
    const float sl2 = scale * 1.4426950408889634f;
    dim3 grid((unsigned)nh * (unsigned)n_tiles), block(kF32Threads);
#define IC_F32_LAUNCH(DD)                                                                                            \
    hipLaunchKernelGGL((attn_prefill_f32_kernel<DD>), grid, block, 0, stream, (const float*)q, q_stride, (float*)out, \
                       out_stride, (const float*)kcache, (const float*)vcache, block_tables, bt_stride,              \
                       (const int4*)tiles, n_tiles, nh, nkvh, page_shift, sl2, window)
    if (dh == 64) IC_F32_LAUNCH(64);
    else if (dh == 128) IC_F32_LAUNCH(128);
    else return IC_ERR_UNSUPPORTED;
#undef IC_F32_LAUNCH
    return ic_launch_status();
}

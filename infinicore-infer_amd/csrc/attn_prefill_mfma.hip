// Attention of prompt portions over the paged cache on the matrix cores
// (bfloat16 operands, float32 accumulation and softmax).
//
// Grid (query tiles, heads), 256 threads.  A tile is up to 128 consecutive
// tokens of one request; wave w owns rows 32w..32w+31.  Keys and values come
// in tiles of 64 through LDS (values transposed on the way in).  Scores are
// computed transposed, S^T = K Q^T, with v_mfma_f32_32x32x8_bf16: every lane
// then holds 16 keys of ONE query, so the running softmax needs a single
// cross-lane step, and the probabilities are already laid out as the B operand
// of O^T = V^T P^T.
//
// 32x32x8 operand layout (lane l): A[i = l%32][k = 4(l/32)..+3], B[k = 4(l/32)..+3][j = l%32],
// D[i = 8(r/4) + 4(l/32) + r%4][j = l%32] for the 16 accumulators r.
//
// Cache layout of one layer: K and V planes [num_pages, n_kv_heads, page_size, head_dim].
#include "common.h"

typedef short v4s __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kPfThreads = 256;
constexpr int kPfRows = 128;      // query rows per block
constexpr int kPfKeys = 64;       // keys per tile
constexpr int kPfPad = 8;         // elements of padding per LDS row

template <int DH>
__global__ void __launch_bounds__(kPfThreads)
attn_prefill_mfma_kernel(const uint16_t* __restrict__ q, int q_stride, uint16_t* __restrict__ out, int out_stride,
                         const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                         const int* __restrict__ block_tables, int bt_stride, const int4* __restrict__ tiles,
                         int nh, int nkvh, int page_size, float scale_log2e, int window) {
    constexpr int NC = DH / 8;            // 8-wide chunks of the head dimension
    constexpr int ND = DH / 32;           // 32-row tiles of O^T
    constexpr int KS = DH + kPfPad;       // row stride of Ks
    constexpr int VS = kPfKeys + kPfPad;  // row stride of Vt
    __shared__ __attribute__((aligned(16))) uint16_t Ks[kPfKeys * KS];
    __shared__ __attribute__((aligned(16))) uint16_t Vt[DH * VS];

    const int4 tile = tiles[blockIdx.x];
    const int req = tile.x, row0 = tile.y, n_rows = tile.z, pos0 = tile.w;
    const int h = blockIdx.y;
    const int kvh = h / (nh / nkvh);
    const int* bt = block_tables + (size_t)req * bt_stride;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;

    const int my_row = 32 * wave + lq;                       // row within the tile
    const bool row_ok = my_row < n_rows;
    const int qpos = pos0 + my_row;
    const bool wave_ok = 32 * wave < n_rows;
    const int wave_last = pos0 + ((32 * wave + 31 < n_rows - 1) ? 32 * wave + 31 : n_rows - 1);
    const int last_key = pos0 + n_rows - 1;
    int first_key = 0;
    if (window > 0 && pos0 - window + 1 > 0) first_key = pos0 - window + 1;

    // Q^T fragments: Q[query lq][8c + 4 half .. +3]
    v4s qf[NC];
    {
        const uint16_t* qp = q + (size_t)(row0 + my_row) * q_stride + (size_t)h * DH + 4 * half;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            if (row_ok) qf[c] = *reinterpret_cast<const v4s*>(qp + 8 * c);
            else qf[c] = v4s{0, 0, 0, 0};
        }
    }

    v16f oacc[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, l = 0.f;

    const size_t head_stride = (size_t)page_size * DH;
    for (int kt = (first_key / kPfKeys) * kPfKeys; kt <= last_key; kt += kPfKeys) {
        __syncthreads();                                     // previous tile's readers are done
        // ---- K tile: thread -> (key, octet), 16-byte rows pieces ----------------
        for (int idx = tid; idx < kPfKeys * NC; idx += kPfThreads) {
            const int key = idx / NC, oct = idx - key * NC;
            const int ka = kt + key;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (ka <= last_key) {
                const int pg = bt[ka / page_size];
                const int off = ka % page_size;
                v = *reinterpret_cast<const uint4*>(kcache + ((size_t)pg * nkvh + kvh) * head_stride + (size_t)off * DH + oct * 8);
            }
            *reinterpret_cast<uint4*>(&Ks[key * KS + oct * 8]) = v;
        }
        // ---- V tile, transposed: thread -> (octet, key) with keys along lanes ----
        for (int idx = tid; idx < kPfKeys * NC; idx += kPfThreads) {
            const int oct = idx / kPfKeys, key = idx - oct * kPfKeys;
            const int ka = kt + key;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (ka <= last_key) {
                const int pg = bt[ka / page_size];
                const int off = ka % page_size;
                v = *reinterpret_cast<const uint4*>(vcache + ((size_t)pg * nkvh + kvh) * head_stride + (size_t)off * DH + oct * 8);
            }
            uint16_t* vp = &Vt[(oct * 8) * VS + key];
            vp[0 * VS] = (uint16_t)(v.x & 0xffff); vp[1 * VS] = (uint16_t)(v.x >> 16);
            vp[2 * VS] = (uint16_t)(v.y & 0xffff); vp[3 * VS] = (uint16_t)(v.y >> 16);
            vp[4 * VS] = (uint16_t)(v.z & 0xffff); vp[5 * VS] = (uint16_t)(v.z >> 16);
            vp[6 * VS] = (uint16_t)(v.w & 0xffff); vp[7 * VS] = (uint16_t)(v.w >> 16);
        }
        __syncthreads();
        if (!wave_ok || kt > wave_last) continue;            // nothing this wave may see
        if (window > 0 && kt + kPfKeys - 1 < pos0 + 32 * wave - window + 1) continue;

        // ---- S^T = K Q^T : two tiles of 32 keys ----------------------------------
        v16f sacc[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[tt][r] = 0.f;
            const uint16_t* kp = &Ks[(32 * tt + lq) * KS + 4 * half];
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const v4s a = *reinterpret_cast<const v4s*>(kp + 8 * c);
                sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a, qf[c], sacc[tt], 0, 0, 0);
            }
        }
        // ---- mask, running softmax (base 2) ----------------------------------------
        float mloc = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ka = kt + 32 * tt + 8 * (r >> 2) + 4 * half + (r & 3);
                bool ok = ka <= qpos;
                if (window > 0) ok = ok && (ka > qpos - window);
                const float s = ok ? sacc[tt][r] * scale_log2e : -INFINITY;
                sacc[tt][r] = s;
                mloc = fmaxf(mloc, s);
            }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
        const float m_new = fmaxf(m, mloc);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m - m_use);
        float rs = 0.f;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = __builtin_amdgcn_exp2f(sacc[tt][r] - m_use);
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

        // ---- O^T += V^T P^T ------------------------------------------------------------
#pragma unroll
        for (int kc = 0; kc < 8; ++kc) {
            const int tt = kc >> 2, rg = kc & 3;
            v4s b;
            b[0] = (short)f32_to_bf16_bits(sacc[tt][4 * rg + 0]);
            b[1] = (short)f32_to_bf16_bits(sacc[tt][4 * rg + 1]);
            b[2] = (short)f32_to_bf16_bits(sacc[tt][4 * rg + 2]);
            b[3] = (short)f32_to_bf16_bits(sacc[tt][4 * rg + 3]);
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const v4s a = *reinterpret_cast<const v4s*>(&Vt[(32 * dt + lq) * VS + 8 * kc + 4 * half]);
                oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a, b, oacc[dt], 0, 0, 0);
            }
        }
    }

    if (!row_ok) return;
    const float inv = 1.0f / l;
    uint16_t* op = out + (size_t)(row0 + my_row) * out_stride + (size_t)h * DH;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            const int d = 32 * dt + 8 * rg + 4 * half;
            uint2 pk;
            pk.x = (uint32_t)f32_to_bf16_bits(oacc[dt][4 * rg + 0] * inv) | ((uint32_t)f32_to_bf16_bits(oacc[dt][4 * rg + 1] * inv) << 16);
            pk.y = (uint32_t)f32_to_bf16_bits(oacc[dt][4 * rg + 2] * inv) | ((uint32_t)f32_to_bf16_bits(oacc[dt][4 * rg + 3] * inv) << 16);
            *reinterpret_cast<uint2*>(op + d) = pk;
        }
}

IC_EXPORT int ic_attn_prefill_supported(int dtype, int dh) {
    return dtype == IC_BF16 && (dh == 64 || dh == 128);
}

IC_EXPORT int ic_attn_prefill_tile_rows() { return kPfRows; }

// tiles: int32 [n_tiles, 4] = (request row of block_tables, first token row, rows <= 128, position of the first row).
IC_EXPORT int ic_attn_prefill(const void* q, int q_stride, void* out, int out_stride, int dtype,
                              const void* kcache, const void* vcache, const int* block_tables,
                              int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh,
                              int page_size, float scale, int window, hipStream_t stream) {
    if (n_tiles <= 0) return IC_OK;
    if (dtype != IC_BF16) return IC_ERR_UNSUPPORTED;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || page_size <= 0 || nh > 65535) return IC_ERR_ARG;
    if (q_stride % 4 || out_stride % 4 || ((uintptr_t)q & 7) || ((uintptr_t)out & 7) ||
        ((uintptr_t)kcache & 15) || ((uintptr_t)vcache & 15) || ((uintptr_t)tiles & 15)) return IC_ERR_ARG;
    const float sl2 = scale * 1.4426950408889634f;
    dim3 grid(n_tiles, nh), block(kPfThreads);
    if (dh == 64)
        hipLaunchKernelGGL(attn_prefill_mfma_kernel<64>, grid, block, 0, stream, (const uint16_t*)q, q_stride,
                           (uint16_t*)out, out_stride, (const uint16_t*)kcache, (const uint16_t*)vcache,
                           block_tables, bt_stride, (const int4*)tiles, nh, nkvh, page_size, sl2, window);
    else if (dh == 128)
        hipLaunchKernelGGL(attn_prefill_mfma_kernel<128>, grid, block, 0, stream, (const uint16_t*)q, q_stride,
                           (uint16_t*)out, out_stride, (const uint16_t*)kcache, (const uint16_t*)vcache,
                           block_tables, bt_stride, (const int4*)tiles, nh, nkvh, page_size, sl2, window);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// Attention of single new tokens over the paged cache (decoding), split over
// the keys so that few requests still fill the chip.
//
// Pass 1, grid (splits, kv heads, tokens), 256 threads: a block streams its
// share of one request's keys and values of one kv head once and serves the
// query heads of that group, four at a time.  DH/VEC lanes share a key
// (VEC = 16 bytes of elements per lane), so a wave reads whole contiguous
// rows; every lane keeps a float32 running softmax for its keys, which are
// merged across the lane groups, the four waves, and (pass 2) the splits.
// Pass 2, grid (tokens * heads): combines the splits and writes the output.
//
// Cache layout of one layer: K and V planes [num_pages, n_kv_heads, page_size, head_dim].
#include "common.h"

constexpr int kDecThreads = 256;
constexpr int kDecWaves = kDecThreads / 64;
constexpr int kDecUnroll = 4;
constexpr int kDecMaxPages = 1024;   // page ids of one block's keys staged in LDS (else read from memory)

template <typename T> struct Vec16;
template <> struct Vec16<float> {
    static constexpr int N = 4;
    __device__ static uint4 raw(const float* p) { return load_stream16(p); }
    __device__ static void unpack(const uint4& v, float* o) {
        o[0] = __uint_as_float(v.x); o[1] = __uint_as_float(v.y);
        o[2] = __uint_as_float(v.z); o[3] = __uint_as_float(v.w);
    }
    __device__ static void load(const float* p, float* o) { unpack(raw(p), o); }
};
template <> struct Vec16<bf16> {
    static constexpr int N = 8;
    __device__ static uint4 raw(const bf16* p) { return load_stream16(p); }
    __device__ static void unpack(const uint4& v, float* o) {
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
        o[4] = __uint_as_float(v.z << 16); o[5] = __uint_as_float(v.z & 0xffff0000u);
        o[6] = __uint_as_float(v.w << 16); o[7] = __uint_as_float(v.w & 0xffff0000u);
    }
    __device__ static void load(const bf16* p, float* o) { unpack(raw(p), o); }
};

// merge running-softmax state b into a
__device__ __forceinline__ void merge_state(float& m, float& l, float* acc, int n,
                                            float mb, float lb, const float* accb) {
    const float mn = fmaxf(m, mb);
    if (mn == -INFINITY) return;                 // both empty
    const float ca = __builtin_amdgcn_exp2f(m - mn), cb = __builtin_amdgcn_exp2f(mb - mn);   // maxima in units of log 2
    l = l * ca + lb * cb;
    for (int i = 0; i < n; ++i) acc[i] = acc[i] * ca + accb[i] * cb;
    m = mn;
}

// Sum over the LPK consecutive lanes that share a key; every one of them gets the same total.
// Steps inside a row of 16 lanes are DPP operands of the add (no LDS round trip).
__device__ __forceinline__ float dpp_add(float v, int) = delete;
template <int CTRL> __device__ __forceinline__ float dpp_add(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int LPK> __device__ __forceinline__ float group_sum(float d) {
    if (LPK >= 64) d += __shfl_xor(d, 32, kWave);
    if (LPK >= 32) d += __shfl_xor(d, 16, kWave);
    if (LPK >= 16) d = dpp_add<0x128>(d);        // row_ror:8      lane i <- lane i ^ 8
    if (LPK >= 8) d = dpp_add<0x141>(d);         // row_half_mirror lane i <- lane 7 - i (of 8)
    if (LPK >= 4) d = dpp_add<0x4E>(d);          // quad_perm [2,3,0,1]
    if (LPK >= 2) d = dpp_add<0xB1>(d);          // quad_perm [1,0,3,2]
    return d;
}

template <typename T, int DH, int GQ, bool STAGED>
__global__ void __launch_bounds__(kDecThreads)
attn_decode_split_kernel(const T* __restrict__ q, int q_stride,
                         const T* __restrict__ kcache, const T* __restrict__ vcache,
                         const int* __restrict__ block_tables, int bt_stride,
                         const int* __restrict__ tok_list, const int* __restrict__ token_req,
                         const int* __restrict__ positions,
                         float* __restrict__ part_acc, float* __restrict__ part_ml,
                         int nh, int nkvh, int page_size, float scale, int window, int nsplit,
                         T* __restrict__ final_out, int out_stride) {
    constexpr int VEC = Vec16<T>::N;
    constexpr int LPK = DH / VEC;                 // lanes per key
    constexpr int KPW = 64 / LPK;                 // keys per wave per step
    constexpr int KPB = KPW * kDecWaves;          // keys per block per step
    static_assert(DH % VEC == 0 && 64 % LPK == 0, "head size must split a wave evenly");

    __shared__ float sm_acc[kDecWaves][GQ][DH];
    __shared__ float sm_ml[kDecWaves][GQ][2];
    __shared__ int pages[kDecMaxPages];

    const int split = blockIdx.x, kvh = blockIdx.y, n = blockIdx.z;
    const int t = tok_list ? tok_list[n] : n;
    const int g = nh / nkvh;
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const int lo0 = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int nkeys = pos + 1 - lo0;
    const int per = (nkeys + nsplit - 1) / nsplit;
    const int lo = lo0 + split * per;
    int hi = lo + per;
    if (hi > pos + 1) hi = pos + 1;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPK;                   // which 16-byte slice of the row
    const int grp = lane / LPK;                   // which key of the wave's step
    const size_t head_stride = (size_t)page_size * DH;
    const size_t page_stride = (size_t)nkvh * head_stride;
    const T* kbase = kcache + (size_t)kvh * head_stride + sub * VEC;
    const T* vbase = vcache + (size_t)kvh * head_stride + sub * VEC;

    // page ids of this block's keys, staged once: the loop then needs one memory hop per key.
    // STAGED is a compile-time choice (the host knows the block table's width): a run-time choice
    // between the two arrays would make every lookup a flat load, whose wait also waits for the
    // key and value loads in flight.
    const int page_lo = lo / page_size;
    const int n_pages = (hi > lo) ? (hi - 1) / page_size - page_lo + 1 : 0;
    if (STAGED)
        for (int i = threadIdx.x; i < n_pages; i += kDecThreads) pages[i] = bt[page_lo + i];
    __syncthreads();

    // element offset of a key's row piece in a plane
    auto row_of = [&](int key) -> size_t {
        const int lp = key / page_size;
        const int pg = STAGED ? pages[lp - page_lo] : bt[lp];
        return (size_t)pg * page_stride + (size_t)(key - lp * page_size) * DH;
    };

    for (int h0 = 0; h0 < g; h0 += GQ) {
        float qv[GQ][VEC], acc[GQ][VEC], m[GQ], l[GQ];
#pragma unroll
        for (int j = 0; j < GQ; ++j) {
            m[j] = -INFINITY; l[j] = 0.f;
            const int hh = (h0 + j < g) ? h0 + j : g - 1;
            Vec16<T>::load(q + (size_t)t * q_stride + (size_t)(kvh * g + hh) * DH + sub * VEC, qv[j]);
#pragma unroll
            for (int i = 0; i < VEC; ++i) { qv[j][i] *= scale * 1.4426950408889634f; acc[j][i] = 0.f; }   // scores in units of log 2
        }

        // keys kb, kb + KPB, ... of one step; the next step's loads are issued before this one is used
        uint4 kr[2][kDecUnroll], vr[2][kDecUnroll];
        // Loads are unconditional (keys beyond the share read its last key and are ignored), so the
        // loop is straight-line code and a stage waits only for its own loads.
        auto issue = [&](int kb, uint4* kk, uint4* vv) {
#pragma unroll
            for (int u = 0; u < kDecUnroll; ++u) {
                const int key = (kb + u * KPB < hi) ? kb + u * KPB : hi - 1;
                const size_t off = row_of(key);
                kk[u] = Vec16<T>::raw(kbase + off);
                vv[u] = Vec16<T>::raw(vbase + off);
            }
        };
        auto consume = [&](int kb, const uint4* kk, const uint4* vv) {
            float kf[kDecUnroll][VEC];
            bool ok[kDecUnroll];
#pragma unroll
            for (int u = 0; u < kDecUnroll; ++u) {
                ok[u] = kb + u * KPB < hi;
                Vec16<T>::unpack(kk[u], kf[u]);
            }
#pragma unroll
            for (int j = 0; j < GQ; ++j) {
                float s[kDecUnroll];
                float mx = m[j];
#pragma unroll
                for (int u = 0; u < kDecUnroll; ++u) {
                    float d = 0.f;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) d += qv[j][i] * kf[u][i];
                    d = group_sum<LPK>(d);
                    s[u] = ok[u] ? d : -INFINITY;
                    mx = fmaxf(mx, s[u]);
                }
                if (mx == -INFINITY) continue;     // this lane group has seen no key yet
                const float corr = __builtin_amdgcn_exp2f(m[j] - mx);
                float lsum = l[j] * corr;
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[j][i] *= corr;
#pragma unroll
                for (int u = 0; u < kDecUnroll; ++u) {
                    float vf[VEC];
                    Vec16<T>::unpack(vv[u], vf);
                    const float p = __builtin_amdgcn_exp2f(s[u] - mx);      // 0 for a key beyond the share
                    lsum += p;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) acc[j][i] += p * vf[i];
                }
                l[j] = lsum;
                m[j] = mx;
            }
        };
        constexpr int STEP = kDecUnroll * KPB;
        const int kb0 = lo + wave * KPW + grp;
        if (lo < hi) {                               // (block-uniform) an empty share has no key to read, not even a stand-in
            issue(kb0, kr[0], vr[0]);
            for (int kb = kb0; kb < hi; kb += 2 * STEP) {
                issue(kb + STEP, kr[1], vr[1]);
                consume(kb, kr[0], vr[0]);
                issue(kb + 2 * STEP, kr[0], vr[0]);
                consume(kb + STEP, kr[1], vr[1]);
            }
        }

        // merge the lane groups of the wave (lanes with the same `sub`)
#pragma unroll
        for (int j = 0; j < GQ; ++j) {
#pragma unroll
            for (int o = LPK; o < 64; o <<= 1) {
                const float mb = __shfl_xor(m[j], o, kWave);
                const float lb = __shfl_xor(l[j], o, kWave);
                float ab[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) ab[i] = __shfl_xor(acc[j][i], o, kWave);
                merge_state(m[j], l[j], acc[j], VEC, mb, lb, ab);
            }
        }
        __syncthreads();                            // LDS free from the previous head chunk
        if (grp == 0) {
#pragma unroll
            for (int j = 0; j < GQ; ++j) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) sm_acc[wave][j][sub * VEC + i] = acc[j][i];
                if (sub == 0) { sm_ml[wave][j][0] = m[j]; sm_ml[wave][j][1] = l[j]; }
            }
        }
        __syncthreads();
        // merge the waves: thread (j, d) for j < GQ, d < DH
        for (int idx = threadIdx.x; idx < GQ * DH; idx += kDecThreads) {
            const int j = idx / DH, d = idx - j * DH;
            if (h0 + j >= g) continue;
            float mm = -INFINITY;
            for (int w = 0; w < kDecWaves; ++w) mm = fmaxf(mm, sm_ml[w][j][0]);
            float a = 0.f, ll = 0.f;
            if (mm != -INFINITY) {
                for (int w = 0; w < kDecWaves; ++w) {
                    const float c = __builtin_amdgcn_exp2f(sm_ml[w][j][0] - mm);
                    a += sm_acc[w][j][d] * c;
                    ll += sm_ml[w][j][1] * c;
                }
            }
            const int h = kvh * g + h0 + j;
            if (final_out) {                        // a single split: this is the result, no second pass
                final_out[(size_t)t * out_stride + (size_t)h * DH + d] = from_f32<T>(a / ll);
                continue;
            }
            const size_t pidx = ((size_t)n * nh + h) * nsplit + split;
            part_acc[pidx * DH + d] = a;
            // the partial maximum leaves in natural units, as the second pass expects
            if (d == 0) { part_ml[pidx * 2] = mm * 0.6931471805599453f; part_ml[pidx * 2 + 1] = ll; }
        }
    }
}

// Grid (tokens * heads), four waves.  Lane s of every wave holds split s (at most 64 splits): the
// weights exp(m_s - max) come from one wave reduction.  Thread (d, g) sums output dim d over
// the splits g, g + G, .. (G = 256 / DH groups, CNT = ceil(splits / G) of them a thread), and the
// groups meet in LDS: with many splits (few kv heads, few requests) one wave alone would walk them
// one after the other.  The partial sums are loaded first, without condition (a slot beyond the
// splits reads the last split and is not added): they do not wait for the weights, so the kernel
// is one round trip to memory, not two.
constexpr int kRedThreads = 256;
template <typename T, int DH, int CNT>
__global__ void __launch_bounds__(kRedThreads)
attn_decode_reduce_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                          const int* __restrict__ tok_list, T* __restrict__ out,
                          int out_stride, int nh, int nsplit) {
    constexpr int G = kRedThreads / DH;
    static_assert(kRedThreads % DH == 0, "every thread has a (dim, group) place");
    __shared__ float wgt[64];
    __shared__ float grp[kRedThreads];
    const int n = blockIdx.x / nh, h = blockIdx.x % nh, tid = threadIdx.x, lane = tid & 63;
    const size_t base = ((size_t)n * nh + h) * nsplit;
    const int g = tid / DH, d = tid - g * DH;
    float pa[CNT];
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
        const int s = (g + i * G < nsplit) ? g + i * G : nsplit - 1;
        pa[i] = part_acc[(base + s) * DH + d];
    }
    const int ls_i = (lane < nsplit) ? lane : nsplit - 1;
    float ms = part_ml[(base + ls_i) * 2], ls = part_ml[(base + ls_i) * 2 + 1];
    const int t = tok_list ? tok_list[n] : n;
    if (lane >= nsplit) { ms = -INFINITY; ls = 0.f; }
    const float mm = wave_max(ms);
    const float w = (ms == -INFINITY) ? 0.f : expf(ms - mm);
    const float inv = 1.0f / wave_sum(ls * w);
    if (tid < 64) wgt[lane] = w;
    __syncthreads();
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < CNT; ++i)
        if (g + i * G < nsplit) a += pa[i] * wgt[g + i * G];
    grp[tid] = a;
    __syncthreads();
    if (tid < DH) {
#pragma unroll
        for (int j = 1; j < G; ++j) a += grp[j * DH + tid];
        out[(size_t)t * out_stride + (size_t)h * DH + tid] = from_f32<T>(a * inv);
    }
}

// ---------------------------------------------------------------------------------------------
// Grouped queries on the matrix cores (bfloat16): the query heads that share a kv head are the
// columns of one 16-wide tile, so keys and values are read once for the whole group.
//
// Same grid and partial-result layout as above.  A wave owns tiles of 32 keys of the block's
// share (tile i -> wave i % 4).  S^T = K Q^T with v_mfma_f32_16x16x32_bf16, keys as rows: the K
// operand comes straight from memory in operand layout (lane l: key l%16, dims 8(l/16)..+7 of a
// 32-dim chunk).  A lane then holds 4+4 keys of ONE head (l%16), so the running softmax needs two
// cross-lane steps.  O^T = V^T P^T: P^T is already the B operand (slot (l/16, e) stands for key
// 4(l/16) + e of the first 16 keys for e < 4, of the second 16 for e >= 4); V goes through LDS
// (written as rows, read as columns with ds_read_b64_tr_b16).  16x16x32 layout: A[i = l%16][k = 8(l/16)..+7],
// B[k = 8(l/16)..+7][j = l%16], D[i = 4(l/16) + e][j = l%16].
typedef __bf16 gq_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gq_v4f __attribute__((ext_vector_type(4)));
typedef float gq_v8f __attribute__((ext_vector_type(8)));
typedef short gq_v4s __attribute__((ext_vector_type(4)));
constexpr int kGqaKeys = 32;

union GqFrag {
    uint4 u;
    uint16_t h[8];
    gq_bf16x8 v;
};

template <int DH, bool STAGED>
__global__ void __launch_bounds__(kDecThreads)
attn_decode_gqa_kernel(const uint16_t* __restrict__ q, int q_stride,
                       const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                       const int* __restrict__ block_tables, int bt_stride,
                       const int* __restrict__ tok_list, const int* __restrict__ token_req,
                       const int* __restrict__ positions,
                       float* __restrict__ part_acc, float* __restrict__ part_ml,
                       int nh, int nkvh, int page_size, float scale, int window, int nsplit,
                       uint16_t* __restrict__ final_out, int out_stride) {
    constexpr int NC = DH / 32;                    // 32-dim chunks of the score product
    constexpr int ND = DH / 16;                    // 16-dim chunks of the output
    constexpr int VS = DH + 8;                     // LDS row stride of a V tile (elements)
    constexpr int NV = kGqaKeys * (DH / 8) / 64;   // 16-byte V loads per lane and tile
    __shared__ __attribute__((aligned(16))) uint16_t Vs[kDecWaves][kGqaKeys * VS];
    __shared__ float sm_ml[kDecWaves][16][2];
    __shared__ int pages[kDecMaxPages];
    static_assert(sizeof(uint16_t) * kGqaKeys * VS >= sizeof(float) * 16 * DH, "merge buffer fits in the V tiles");
    float* sm_o = reinterpret_cast<float*>(&Vs[0][0]);       // [waves][16 heads][DH] after the key loop

    const int split = blockIdx.x, kvh = blockIdx.y, n = blockIdx.z;
    const int t = tok_list ? tok_list[n] : n;
    const int g = nh / nkvh;
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const int lo0 = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int nkeys = pos + 1 - lo0;
    const int per = (nkeys + nsplit - 1) / nsplit;
    const int lo = lo0 + split * per;
    int hi = lo + per;
    if (hi > pos + 1) hi = pos + 1;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float scale2 = scale * 1.4426950408889634f;   // scores and running maxima in units of log 2: exp2 is one instruction
    const int lr = lane & 15, lg = lane >> 4;      // row / column of a tile, and the lane group
    const size_t head_stride = (size_t)page_size * DH;
    const size_t page_stride = (size_t)nkvh * head_stride;
    const uint16_t* kbase = kcache + (size_t)kvh * head_stride;
    const uint16_t* vbase = vcache + (size_t)kvh * head_stride;

    const int page_lo = lo / page_size;
    const int n_pages = (hi > lo) ? (hi - 1) / page_size - page_lo + 1 : 0;
    if (STAGED)
        for (int i = threadIdx.x; i < n_pages; i += kDecThreads) pages[i] = bt[page_lo + i];
    __syncthreads();
    auto row_of = [&](int key) -> size_t {
        const int lp = key / page_size;
        const int pg = STAGED ? pages[lp - page_lo] : bt[lp];
        return (size_t)pg * page_stride + (size_t)(key - lp * page_size) * DH;
    };

    const int n_tiles = (hi > lo) ? (hi - lo + kGqaKeys - 1) / kGqaKeys : 0;
    const int rounds = (n_tiles + kDecWaves - 1) / kDecWaves;

    for (int h0 = 0; h0 < g; h0 += 16) {
        // Q^T operand: head lr of this chunk, dims 32c + 8 lg .. +7
        GqFrag qf[NC];
        {
            const bool head_ok = h0 + lr < g;
            const uint16_t* qp = q + (size_t)t * q_stride + (size_t)(kvh * g + h0 + (head_ok ? lr : 0)) * DH + 8 * lg;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (head_ok) qf[c].u = *reinterpret_cast<const uint4*>(qp + 32 * c);
                else qf[c].u = make_uint4(0, 0, 0, 0);
            }
        }
        gq_v4f oacc[ND];
#pragma unroll
        for (int c = 0; c < ND; ++c) oacc[c] = gq_v4f{0.f, 0.f, 0.f, 0.f};
        float m = -INFINITY, l = 0.f;              // of head lr, the same in the four lane groups

        // Keys and values are read in whole rows (consecutive lanes take consecutive 16-byte pieces, so a wave's load
        // covers whole cache lines) with loads the caches do not keep.  The keys then pass through the wave's LDS tile
        // into operand layout (key 16 s2 + lr, dims 32 c + 8 lg .. +7) before the values take the tile over: loaded
        // straight in operand layout a wave's load covered 64 bytes of each of 16 rows, half a line.
        GqFrag kreg[2][NC];
        uint4 kraw[NV], vreg[NV];
        auto fetch = [&](int tile) {
            const int kt = lo + tile * kGqaKeys;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int idx = lane + 64 * i;
                const int vkey = idx / (DH / 8), oct = idx - vkey * (DH / 8);
                const int key = kt + vkey;
                kraw[i] = make_uint4(0, 0, 0, 0);
                vreg[i] = make_uint4(0, 0, 0, 0);
                if (tile < n_tiles && key < hi) {
                    const size_t at = row_of(key) + oct * 8;
                    kraw[i] = load_stream16(kbase + at);
                    vreg[i] = load_stream16(vbase + at);
                }
            }
        };
        auto stash = [&](const uint4* regs) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int idx = lane + 64 * i;
                const int vkey = idx / (DH / 8), oct = idx - vkey * (DH / 8);
                *reinterpret_cast<uint4*>(&Vs[wave][vkey * VS + oct * 8]) = regs[i];
            }
        };

        // A wave writes and reads only its own V tile in LDS, and LDS serves a wave's instructions
        // in order, so no block barrier is needed in this loop (wave_barrier keeps the compiler from
        // moving LDS accesses across it).
        fetch(wave);
        for (int r = 0; r < rounds; ++r) {
            const int tile = r * kDecWaves + wave;
            if (tile >= n_tiles) break;             // uniform in the wave
            const int kt = lo + tile * kGqaKeys;
            __builtin_amdgcn_wave_barrier();
            stash(kraw);
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                for (int c = 0; c < NC; ++c)
                    kreg[s2][c].u = *reinterpret_cast<const uint4*>(&Vs[wave][(16 * s2 + lr) * VS + 32 * c + 8 * lg]);
            __builtin_amdgcn_wave_barrier();
            stash(vreg);
            __builtin_amdgcn_wave_barrier();

            // ---- S^T = K Q^T, two subtiles of 16 keys ----------------------------------
            gq_v4f sacc[2];
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                sacc[s2] = gq_v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < NC; ++c)
                    sacc[s2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[s2][c].v, qf[c].v, sacc[s2], 0, 0, 0);
            }
            fetch(tile + kDecWaves);                // the next tile's loads fly during the rest of this one
            float sv[8];
            float mloc = -INFINITY;
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int key = kt + 16 * s2 + 4 * lg + e;
                    const float x = (key < hi) ? sacc[s2][e] * scale2 : -INFINITY;     // in units of log 2
                    sv[4 * s2 + e] = x;
                    mloc = fmaxf(mloc, x);
                }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 16, kWave));
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
            const float m_new = fmaxf(m, mloc);     // finite: every tile has at least one key
            const float corr = __builtin_amdgcn_exp2f(m - m_new);
            float rs = 0.f;
            gq_v8f pf;
#pragma unroll
            for (int e = 0; e < 8; ++e) { const float p = __builtin_amdgcn_exp2f(sv[e] - m_new); pf[e] = p; rs += p; }
            rs += __shfl_xor(rs, 16, kWave);
            rs += __shfl_xor(rs, 32, kWave);
            l = l * corr + rs;
            m = m_new;
            const gq_bf16x8 pb = __builtin_convertvector(pf, gq_bf16x8);

            // ---- O^T += V^T P^T ----------------------------------------------------------------
            // V^T operand by transposing LDS reads: lane 16 G + i receives, for e = 0..3, element i % 4 of the
            // 8-byte chunk that lane 16 G + i / 4 + 4 e pointed at; this lane points at key 4 lg + lr / 4 (and 16
            // keys on), dims 16 c + 4 (lr % 4) ..+3, and gets dim 16 c + lr of keys 4 lg + e (and 16 keys on)
            const uint16_t* vrow = &Vs[wave][(4 * lg + (lr >> 2)) * VS + 4 * (lr & 3)];
#pragma unroll
            for (int c = 0; c < ND; ++c) {
                GqFrag a;
                const gq_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gq_v4s __attribute__((address_space(3)))*)(vrow + 16 * c));
                const gq_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gq_v4s __attribute__((address_space(3)))*)(vrow + 16 * VS + 16 * c));
#pragma unroll
                for (int e = 0; e < 4; ++e) { a.h[e] = (uint16_t)lo[e]; a.h[4 + e] = (uint16_t)hi[e]; }
                oacc[c] *= corr;
                oacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pb, oacc[c], 0, 0, 0);
            }
        }

        // ---- merge the four waves; O^T[d = 16c + 4 lg + e][head lr] ---------------------------
        __syncthreads();
#pragma unroll
        for (int c = 0; c < ND; ++c)
#pragma unroll
            for (int e = 0; e < 4; ++e) sm_o[(wave * 16 + lr) * DH + 16 * c + 4 * lg + e] = oacc[c][e];
        if (lg == 0) { sm_ml[wave][lr][0] = m; sm_ml[wave][lr][1] = l; }
        __syncthreads();
        for (int idx = threadIdx.x; idx < 16 * DH; idx += kDecThreads) {
            const int j = idx / DH, d = idx - j * DH;
            if (h0 + j >= g) continue;
            float mm = -INFINITY;
            for (int w = 0; w < kDecWaves; ++w) mm = fmaxf(mm, sm_ml[w][j][0]);
            float a = 0.f, ll = 0.f;
            if (mm != -INFINITY) {
                for (int w = 0; w < kDecWaves; ++w) {
                    const float cw = __builtin_amdgcn_exp2f(sm_ml[w][j][0] - mm);
                    a += sm_o[(w * 16 + j) * DH + d] * cw;
                    ll += sm_ml[w][j][1] * cw;
                }
            }
            const int h = kvh * g + h0 + j;
            if (final_out) {                        // a single split: this is the result, no second pass
                final_out[(size_t)t * out_stride + (size_t)h * DH + d] = f32_to_bf16_bits(a / ll);
                continue;
            }
            const size_t pidx = ((size_t)n * nh + h) * nsplit + split;
            part_acc[pidx * DH + d] = a;
            if (d == 0) { part_ml[pidx * 2] = mm * 0.6931471805599453f; part_ml[pidx * 2 + 1] = ll; }   // natural units for the second pass
        }
        __syncthreads();                            // sm_o (the V tiles) is reused by the next chunk
    }
}

// Grouped queries in bfloat16 run the matrix-core kernel: the one place that says so (the key-split rule asks here too).
IC_EXPORT int ic_attn_decode_on_matrix_cores(int dtype, int n_heads, int n_kv_heads) { return dtype == IC_BF16 && n_heads != n_kv_heads; }

template <typename T, int DH>
static int launch_decode(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                         const void* vcache, const int* block_tables, int bt_stride, const int* tok_list,
                         const int* token_req, const int* positions, float* part_acc, float* part_ml,
                         int n_tok, int nh, int nkvh, int page_size, float scale, int window, int nsplit,
                         hipStream_t stream) {
    dim3 grid(nsplit, nkvh, n_tok), block(kDecThreads);
    const bool staged = bt_stride <= kDecMaxPages;      // a block never needs more page ids than a request has
    void* direct = (nsplit == 1) ? out : nullptr;       // one split writes the result itself
#define IC_DEC_LAUNCH(KERNEL, TQ)                                                                           \
    hipLaunchKernelGGL(KERNEL, grid, block, 0, stream, (const TQ*)q, q_stride, (const TQ*)kcache,           \
                       (const TQ*)vcache, block_tables, bt_stride, tok_list, token_req, positions, part_acc, \
                       part_ml, nh, nkvh, page_size, scale, window, nsplit, (TQ*)direct, out_stride)
    if (ic_attn_decode_on_matrix_cores(sizeof(T) == 2 ? IC_BF16 : IC_F32, nh, nkvh)) {
        if (staged) IC_DEC_LAUNCH((attn_decode_gqa_kernel<DH, true>), uint16_t);
        else IC_DEC_LAUNCH((attn_decode_gqa_kernel<DH, false>), uint16_t);
    } else if (nh == nkvh) {
        if (staged) IC_DEC_LAUNCH((attn_decode_split_kernel<T, DH, 1, true>), T);
        else IC_DEC_LAUNCH((attn_decode_split_kernel<T, DH, 1, false>), T);
    } else {
        if (staged) IC_DEC_LAUNCH((attn_decode_split_kernel<T, DH, 4, true>), T);
        else IC_DEC_LAUNCH((attn_decode_split_kernel<T, DH, 4, false>), T);
    }
#undef IC_DEC_LAUNCH
    int st = ic_launch_status();
    if (st || nsplit == 1) return st;
    const int per_thread = (nsplit + kRedThreads / DH - 1) / (kRedThreads / DH);    // splits a thread of the second pass sums
#define IC_RED_LAUNCH(CNT)                                                                                      \
    hipLaunchKernelGGL((attn_decode_reduce_kernel<T, DH, CNT>), dim3(n_tok * nh), dim3(kRedThreads), 0, stream, \
                       part_acc, part_ml, tok_list, (T*)out, out_stride, nh, nsplit)
    if (per_thread <= 2) IC_RED_LAUNCH(2);
    else if (per_thread <= 4) IC_RED_LAUNCH(4);
    else if (per_thread <= 8) IC_RED_LAUNCH(8);
    else if (per_thread <= 16) IC_RED_LAUNCH(16);
    else IC_RED_LAUNCH(32);                             // 64 splits, two groups
#undef IC_RED_LAUNCH
    return ic_launch_status();
}

// Head sizes with a tiled decode kernel.
IC_EXPORT int ic_attn_decode_supported(int dtype, int dh) {
    return (dtype == IC_F32 || dtype == IC_BF16) && (dh == 64 || dh == 128);
}

// part_acc: float32 [n_tok, nh, nsplit, dh]; part_ml: float32 [n_tok, nh, nsplit, 2].
// tok_list: rows of q/out that are decoded (nullptr: rows 0..n_tok-1).
IC_EXPORT int ic_attn_decode(const void* q, int q_stride, void* out, int out_stride, int dtype,
                             const void* kcache, const void* vcache, const int* block_tables,
                             int bt_stride, const int* tok_list, const int* token_req,
                             const int* positions, float* part_acc, float* part_ml, int n_tok, int nh,
                             int nkvh, int dh, int page_size, float scale, int window, int nsplit,
                             hipStream_t stream) {
    if (n_tok <= 0) return IC_OK;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || page_size <= 0 || nsplit <= 0 || nsplit > 64) return IC_ERR_ARG;
    if (nkvh > 65535 || n_tok > 65535) return IC_ERR_ARG;
    if (q_stride % 8 || ((uintptr_t)q & 15) || ((uintptr_t)kcache & 15) || ((uintptr_t)vcache & 15)) return IC_ERR_ARG;
#define IC_DECODE_CASE(TT, DD)                                                                          \
    return launch_decode<TT, DD>(q, q_stride, out, out_stride, kcache, vcache, block_tables, bt_stride, \
                                 tok_list, token_req, positions, part_acc, part_ml, n_tok, nh, nkvh,   \
                                 page_size, scale, window, nsplit, stream)
    if (dtype == IC_F32 && dh == 64) IC_DECODE_CASE(float, 64);
    if (dtype == IC_F32 && dh == 128) IC_DECODE_CASE(float, 128);
    if (dtype == IC_BF16 && dh == 64) IC_DECODE_CASE(bf16, 64);
    if (dtype == IC_BF16 && dh == 128) IC_DECODE_CASE(bf16, 128);
#undef IC_DECODE_CASE
    return IC_ERR_UNSUPPORTED;
}

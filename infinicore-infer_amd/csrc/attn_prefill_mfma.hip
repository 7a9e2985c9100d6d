// Attention of prompt portions over the paged cache on the matrix cores
// (bfloat16 operands, float32 accumulation and softmax).
//
// Grid (heads * query tiles), tile-major, 256 * GROUPS threads.  A tile is up to 128
// consecutive tokens of one request; wave w of a group owns rows 32w..32w+31.  With GROUPS == 2
// the two groups take the even and the odd key tiles of 64 and are merged through LDS at the
// end: the longest query tile of a prompt, which sets the kernel's time when there are few
// blocks, then walks half as many key tiles.  With many blocks GROUPS == 1 keeps more of them
// resident and is faster.  Keys and values come through LDS as rows, 64 * GROUPS keys a step, loaded
// from memory straight into LDS (no registers in between, one barrier a step); the next step's are on
// their way into a second stage while the current one is used.  The V^T operand is
// read with ds_read_b64_tr_b16, which transposes 16-bit elements across the lanes of a 16-lane
// group on the way out of LDS (lane 16G + i receives, for e = 0..3, element i % 4 of the 8-byte
// chunk that lane 16G + i / 4 + 4e pointed at).  Scores
// are computed transposed, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16: every
// lane then holds 32 keys of ONE query, so the running softmax needs a single
// cross-lane step, and the probabilities are already laid out as the B operand
// of O^T = V^T P^T.
//
// 32x32x16 operand layout (lane l, h = l/32): A[i = l%32][k = 8h..8h+7],
// B[k = 8h..8h+7][j = l%32], D[i = 8(r/4) + 4h + r%4][j = l%32] for the 16
// accumulators r.  A and B only have to agree on which k a slot means: in
// O^T = V^T P^T slot (h, e) of 16-key chunk c stands for key 16c + 4h + e
// (e < 4) and 16c + 8 + 4h + (e - 4) (e >= 4), which is where D left P^T.
//
// A query tile's walk over the keys may also be cut into parts that run as blocks of their own (GROUPS == 1): the
// grid then holds `parts` blocks per (tile, head), block `part` walks its share of the tile's key tiles (at least
// part_len of them a part; blocks beyond a tile's number of parts leave at once), writes its running maximum, sum
// and O^T to scratch memory and counts itself in; the block that arrives last merges the others' results into its
// own and writes the output.  Nobody waits for anybody.  With few blocks the longest tile's walk is the kernel's
// time (a 2,048-token prompt: 32 key tiles one after the other while most of the chip has run dry), and parts cut it
// without the 8-wave blocks of GROUPS == 2.
//
// Cache layout of one layer: K and V planes [num_pages, n_kv_heads, page_size, head_dim].
#include "common.h"
#include <type_traits>

// Arrival counters of the split walk, one per (tile, head), in memory of the caller's: zero before the first launch,
// and put back to zero by the block that merges, so launches that follow each other on a stream share one buffer.
constexpr int kPfCounters = 1 << 16;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v8f __attribute__((ext_vector_type(8)));
typedef short tr_v4s __attribute__((ext_vector_type(4)));

constexpr int kPfWaveThreads = 256;   // four waves own the 128 rows of a query tile
constexpr int kPfRows = 128;      // query rows per block
constexpr int kPfKeys = 64;       // keys per tile
constexpr int kPfMaxPages = 2048; // pages of one request whose ids are staged in LDS (else read from memory)

union Frag8 {
    uint4 u;
    uint2 h[2];
    bf16x8 v;
};

template <int DH, bool STAGED, int GROUPS, bool PAGE64>
__global__ void __launch_bounds__(256 * GROUPS, (GROUPS == 1 && DH <= 64) ? 3 : 2)
attn_prefill_mfma_kernel(const uint16_t* __restrict__ q, int q_stride, uint16_t* __restrict__ out, int out_stride,
                         const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                         const int* __restrict__ block_tables, int bt_stride, const int4* __restrict__ tiles,
                         int n_tiles, int nh, int nkvh, int page_shift, float scale_log2e, int window,
                         int parts, int part_len, float* __restrict__ scratch, int* __restrict__ counters) {
    constexpr int NC = DH / 16;           // 16-wide chunks of the head dimension
    constexpr int ND = DH / 32;           // 32-row tiles of O^T
    constexpr int CPR = DH / 8;           // 16-byte chunks of a row
    constexpr int kPfThreads = kPfWaveThreads * GROUPS;
    constexpr int STEP = kPfKeys * GROUPS;                 // keys staged per step
    constexpr int NL = STEP * CPR / kPfThreads;            // 16-byte loads per thread per plane and step
    constexpr int TILE = kPfKeys * DH;                     // elements of one group's K (or V) tile: rows without padding
    constexpr int STAGE = 2 * GROUPS * TILE;               // a step's tiles: K of every group, then V of every group
    constexpr int MERGE_F = 2 + ND * 16;                   // floats a lane hands over at the end
    static_assert(GROUPS == 1 || sizeof(uint16_t) * STAGE >= sizeof(float) * 256 * (2 + (ND / 2) * 16), "each half of the merge buffer fits in a stage");
    // Two stages: the loads of the next step write one while the other is read.  They go from memory straight into LDS
    // (global_load_lds_dwordx4: lane i of a wave writes 16 bytes at the wave's base + 16 i, no registers, no store
    // instructions), so rows cannot be padded; instead the 16-byte chunks of row r sit at position (chunk ^ f(r)), which a
    // lane arranges by fetching the chunk that belongs where it writes.  The LDS has 64 banks of 4 bytes: a 16-byte read of
    // a wave is conflict-free when 16 consecutive rows fall on 16 different 16-byte slots of the 256 bytes, so for the K
    // operand f(r) = r / 2 % 8 with rows of 128 bytes and r % 16 with rows of 256; the transposing 8-byte reads of the V
    // operand (4 rows x 32 bytes per 16 lanes) want f(r) = 2 (r % 4) + (r / 4) % 2.  Measured alone, cycles per read
    // instruction with four waves reading: K 20 (32 with f = r % 8, 22 with rows padded to 144 bytes, 128 with neither),
    // V 20 (19 with rows padded to 160 bytes).
    // (Two arrays, and the stage a compile-time constant wherever they are used: the compiler then knows that a load
    // in flight into one does not touch what is read from the other, and does not wait for it before every LDS read.)
    __shared__ __attribute__((aligned(16))) uint16_t stage0[STAGE];
    __shared__ __attribute__((aligned(16))) uint16_t stage1[STAGE];

    __shared__ int pages[kPfMaxPages];

    // Blocks start in index order and the host lists the tiles longest first: tile-major order (all heads
    // of the longest tile, then of the next one) therefore starts the long walks first everywhere, and since
    // blocks are dealt to the 8 XCDs in turn (block b runs on XCD b % 8) every XCD gets an equal share of
    // every length.  A head's tiles then meet on few XCDs (two of them with 36 heads), so its keys still
    // stay in those L2s.
    const int part = (GROUPS == 1 && parts > 1) ? (int)(blockIdx.x / ((unsigned)nh * (unsigned)n_tiles)) : 0;
    const int slot = (int)blockIdx.x - part * nh * n_tiles;          // (tile, head)
    const int h = slot % nh;
    const int4 tile = tiles[slot / nh];
    const int req = tile.x, row0 = tile.y, n_rows = tile.z, pos0 = tile.w;
    const int kvh = h / (nh / nkvh);
    const int* bt = block_tables + (size_t)req * bt_stride;
    const int tid = threadIdx.x, lane = tid & 63;
    const int grp = tid >> 8, wave = (tid >> 6) & 3;        // key-tile group, and the 32 rows this wave owns
    const int lq = lane & 31, half = lane >> 5;
    const int page_size = 1 << page_shift, page_mask = page_size - 1;     // pages are a power of two here

    const int my_row = 32 * wave + lq;                       // row within the tile
    const bool row_ok = my_row < n_rows;
    const int qpos = pos0 + my_row;
    const bool wave_ok = 32 * wave < n_rows;
    const int wave_first = pos0 + 32 * wave;
    const int wave_last = pos0 + ((32 * wave + 31 < n_rows - 1) ? 32 * wave + 31 : n_rows - 1);
    const int last_key = pos0 + n_rows - 1;
    int first_key = 0;
    if (window > 0 && pos0 - window + 1 > 0) first_key = pos0 - window + 1;

    // this block's share of the tile's key tiles
    const int kt0 = (first_key / kPfKeys) * kPfKeys;
    const int n_kt = (last_key - kt0) / kPfKeys + 1;
    int n_parts = 1;
    if (GROUPS == 1 && parts > 1) {
        n_parts = (n_kt + part_len - 1) / part_len;
        n_parts = n_parts < parts ? n_parts : parts;
        if (part >= n_parts) return;                         // (the whole block: nobody is left at a barrier)
    }
    const int kb_begin = kt0 + kPfKeys * (int)((long long)n_kt * part / n_parts);
    const int kb_end = kt0 + kPfKeys * (int)((long long)n_kt * (part + 1) / n_parts);      // one past this part's last tile

    // page ids of the keys this block reads, staged once (one memory hop less per tile)
    const int page_lo = (kb_begin > first_key ? kb_begin : first_key) >> page_shift;
    const int page_hi = (kb_end - 1 < last_key ? kb_end - 1 : last_key) >> page_shift;
    // STAGED is chosen by the host from the block table's width: a run-time choice between the
    // two arrays would turn every lookup into a flat load, and waiting for a flat load also
    // waits for the key and value loads in flight.
    if (STAGED)
        for (int i = tid; i <= page_hi - page_lo; i += kPfThreads) pages[i] = bt[page_lo + i];
    __syncthreads();
    auto page_of = [&](int ka) -> int { return STAGED ? pages[(ka >> page_shift) - page_lo] : bt[ka >> page_shift]; };

    // Q^T fragments: Q[query lq][16c + 8 half .. +7]
    Frag8 qf[NC];
    {
        const uint16_t* qp = q + (size_t)(row0 + my_row) * q_stride + (size_t)h * DH + 8 * half;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            if (row_ok) qf[c].u = *reinterpret_cast<const uint4*>(qp + 16 * c);
            else qf[c].u = make_uint4(0, 0, 0, 0);
        }
    }

    v16f oacc[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, l = 0.f;          // running maximum of the raw scores, running sum

    const size_t head_stride = (size_t)page_size * DH;
    const uint16_t* kbase = kcache + (size_t)kvh * head_stride;
    const uint16_t* vbase = vcache + (size_t)kvh * head_stride;
    const size_t page_stride = (size_t)nkvh * head_stride;

    // What a thread loads in a step never changes: LDS chunk tid + i * threads of the step's K (and V) tiles, that is key
    // `tkey` of the step's keys at chunk position idx % CPR, which holds the row's chunk `pos ^ f(key)`.
    auto swz_k = [](int row) -> int { return DH == 64 ? (row >> 1) & 7 : row & 15; };
    auto swz_v = [](int row) -> int { return ((row & 3) << 1) | ((row >> 2) & 1); };
    constexpr int KPI = kPfThreads / CPR;                     // keys one pass of loads covers (<= 64)
    static_assert(KPI <= kPfKeys && kPfKeys % KPI == 0, "a pass of loads stays inside a tile");
    int tkey[NL];
    uint32_t toffk[NL], toffv[NL], tcolk[NL], tcolv[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int idx = tid + i * kPfThreads;
        const int key = idx / CPR, colk = (idx - key * CPR) ^ swz_k(key), colv = (idx - key * CPR) ^ swz_v(key);
        tkey[i] = key;
        tcolk[i] = (uint32_t)(colk * 16);
        tcolv[i] = (uint32_t)(colv * 16);
        toffk[i] = (uint32_t)((key % kPfKeys) * DH * sizeof(uint16_t) + colk * 16);
        toffv[i] = (uint32_t)((key % kPfKeys) * DH * sizeof(uint16_t) + colv * 16);
    }
    typedef const void __attribute__((address_space(1)))* gptr_t;
    typedef void __attribute__((address_space(3)))* lptr_t;
    auto issue = [&](int kt, auto stage_c) {
        uint16_t* const kdst = (decltype(stage_c)::value ? stage1 : stage0) + (tid & ~63) * 8;       // this wave's 1 KB of the first pass
        uint16_t* const vdst = kdst + GROUPS * TILE;
        // PAGE64 (pages of 64 tokens and more): a 64-key tile lies in one page; when the whole step lies inside the keys
        // this tile may read, one page lookup per tile does, the same for every lane: the tile's first row is a scalar
        // address and a load adds the thread's constant offset to it.
        if (PAGE64 && kt >= first_key && kt + STEP - 1 <= last_key) {
            const char* krow[GROUPS];
            const char* vrow[GROUPS];
#pragma unroll
            for (int t = 0; t < GROUPS; ++t) {
                const int k0 = kt + kPfKeys * t;
                const int pg = __builtin_amdgcn_readfirstlane(page_of(k0));
                const size_t row = (size_t)pg * page_stride + (size_t)(k0 & page_mask) * DH;
                krow[t] = reinterpret_cast<const char*>(kbase + row);
                vrow[t] = reinterpret_cast<const char*>(vbase + row);
            }
#pragma unroll
            for (int i = 0; i < NL; ++i) {
                __builtin_amdgcn_global_load_lds((gptr_t)(krow[(i * KPI) / kPfKeys] + toffk[i]), (lptr_t)(kdst + i * kPfThreads * 8), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr_t)(vrow[(i * KPI) / kPfKeys] + toffv[i]), (lptr_t)(vdst + i * kPfThreads * 8), 16, 0, 0);
            }
            return;
        }
        // Otherwise every load looks its page up.  A key outside what the tile may read (before the window's first key,
        // beyond the last key) is replaced by the nearest one inside: its page may not be the request's any more, or not
        // written yet; the mask drops its score, and the value it is multiplied with is a real one.
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            int ka = kt + tkey[i];
            ka = ka < first_key ? first_key : ka;
            ka = ka > last_key ? last_key : ka;
            const size_t off = ((size_t)page_of(ka) * page_stride + (size_t)(ka & page_mask) * DH) * sizeof(uint16_t);
            __builtin_amdgcn_global_load_lds((gptr_t)(reinterpret_cast<const char*>(kbase) + off + tcolk[i]), (lptr_t)(kdst + i * kPfThreads * 8), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(reinterpret_cast<const char*>(vbase) + off + tcolv[i]), (lptr_t)(vdst + i * kPfThreads * 8), 16, 0, 0);
        }
    };

    // where this lane reads its operands: K row lq (and 32 on), chunks 2 c + half; V rows 4 half + (l % 16) / 4 of a
    // 16-key chunk (and 8 on), dims 32 dt + 16 (l / 16 % 2) + 4 (l % 4) ..+3
    int koff[NC], voff[ND];
    {
        const int fq = swz_k(lq);
#pragma unroll
        for (int c = 0; c < NC; ++c) koff[c] = lq * DH + ((2 * c + half) ^ fq) * 8;
        const int vrow = 4 * half + ((lane & 15) >> 2), fv = swz_v(vrow);
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) voff[dt] = vrow * DH + ((4 * dt + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1)) ^ fv) * 8 + 4 * (lane & 1);
    }

    // one step: wait for its tiles, send for the next step's, use it
    auto step = [&](int kb, auto stage_c) {
        constexpr int S = decltype(stage_c)::value;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this thread's loads of the step have reached LDS
        __syncthreads();                                     // everybody's have, and the other stage's readers are done
        if (kb + STEP < kb_end) issue(kb + STEP, std::integral_constant<int, 1 - S>{});      // in flight while this step is used
        const uint16_t* const Ks = (S ? stage1 : stage0) + grp * TILE;
        const uint16_t* const Vs = (S ? stage1 : stage0) + (GROUPS + grp) * TILE;
        const int kt = kb + kPfKeys * grp;                   // this group's key tile
        if (!wave_ok || kt > wave_last) return;              // nothing this wave may see
        if (window > 0 && kt + kPfKeys - 1 < wave_first - window + 1) return;

        // ---- S^T = K Q^T : two tiles of 32 keys ----------------------------------
        v16f sacc[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[tt][r] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                Frag8 a;
                a.u = *reinterpret_cast<const uint4*>(Ks + 32 * tt * DH + koff[c]);
                sacc[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, qf[c].v, sacc[tt], 0, 0, 0);
            }
        }
        // ---- mask (only tiles that touch the diagonal or the window's edge) -----------
        const bool need_mask = (kt + kPfKeys - 1 > wave_first) || (window > 0);
        if (need_mask) {
            // key kt + 4 half + e of this lane's accumulator (e a constant per accumulator) is seen when e <= lim
            const int lim = qpos - kt - 4 * half;
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
        // ---- running softmax, base 2: p = 2^(s c - m c) ---------------------------------
        float mloc = sacc[0][0];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, sacc[tt][r]);
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
        const float m_new = fmaxf(m, mloc);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float mc = m_use * scale_log2e;
        const float corr = __builtin_amdgcn_exp2f(m * scale_log2e - mc);       // 0 on the first tile (m = -inf)
        float rs = 0.f;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = __builtin_amdgcn_exp2f(fmaf(sacc[tt][r], scale_log2e, -mc));
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

        // ---- O^T += V^T P^T : four chunks of 16 keys ------------------------------------------
#pragma unroll
        for (int kc = 0; kc < 4; ++kc) {
            const int tt = kc >> 1, r0 = 8 * (kc & 1);
            v8f pf;
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[e] = sacc[tt][r0 + e];
            const bf16x8 b = __builtin_convertvector(pf, bf16x8);
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                // this lane's chunk: key 16 kc + 4 half + (l % 16) / 4 (and 8 keys on), dims 32 dt + 16 (l / 16 % 2) + 4 (l % 4) ..+3;
                // what comes back is dim 32 dt + lq of keys 16 kc + 4 half + e (and 8 keys on), e = 0..3
                const uint16_t* vp = Vs + 16 * kc * DH + voff[dt];
                Frag8 a;
                a.h[0] = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_v4s __attribute__((address_space(3)))*)vp));
                a.h[1] = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_v4s __attribute__((address_space(3)))*)(vp + 8 * DH)));
                oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b, oacc[dt], 0, 0, 0);
            }
        }
    };
    issue(kb_begin, std::integral_constant<int, 0>{});
    for (int kb = kb_begin; kb < kb_end; kb += 2 * STEP) {
        step(kb, std::integral_constant<int, 0>{});
        if (kb + STEP < kb_end) step(kb + STEP, std::integral_constant<int, 1>{});
    }

    // ---- the odd-tile group hands its state to the even-tile group (same lane, same rows) ----------
    if (GROUPS == 2) {
    __syncthreads();                                         // every wave is done with the tiles
    // (the maximum, the sum and the first half of O^T's tiles through one stage's memory, the other half through the other's)
    constexpr int H0 = ND / 2, F0 = 2 + 16 * H0, F1 = 16 * (ND - H0);
    float* const mbuf0 = reinterpret_cast<float*>(stage0) + (size_t)(wave * 64 + lane) * F0;
    float* const mbuf1 = reinterpret_cast<float*>(stage1) + (size_t)(wave * 64 + lane) * F1;
    if (grp == 1) {
        mbuf0[0] = m; mbuf0[1] = l;
#pragma unroll
        for (int i = 0; i < ND; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) (i < H0 ? mbuf0[2 + 16 * i + r] : mbuf1[16 * (i - H0) + r]) = oacc[i][r];
    }
    __syncthreads();
    if (grp == 1) return;
    {
        const float m1 = mbuf0[0], l1 = mbuf0[1];
        const float m_new = fmaxf(m, m1);
        const float mc = ((m_new == -INFINITY) ? 0.f : m_new) * scale_log2e;
        const float c0 = __builtin_amdgcn_exp2f(m * scale_log2e - mc), c1 = __builtin_amdgcn_exp2f(m1 * scale_log2e - mc);
        l = l * c0 + l1 * c1;
#pragma unroll
        for (int i = 0; i < ND; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] = oacc[i][r] * c0 + (i < H0 ? mbuf0[2 + 16 * i + r] : mbuf1[16 * (i - H0) + r]) * c1;
    }
    }
    // ---- a walk cut into parts: hand the state over, and the block that arrives last merges and writes ----------
    if (GROUPS == 1 && n_parts > 1) {
        __shared__ int arrived;
        constexpr int PF = kPfWaveThreads * MERGE_F;          // floats of one part: [field][thread], so that stores coalesce
        // The parts of a tile run on different XCDs, whose L2 caches do not see each other's lines: the state goes out
        // with device-scope stores (written through) and comes in with device-scope loads (not served from this XCD's
        // L2), so that no cache has to be written back or invalidated as a whole, which a device-scope fence would do
        // (with fences the kernel took three times as long).  The count is a device-scope atomic.
        float* const mine = scratch + ((size_t)slot * parts + part) * PF;
        auto put = [](float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
        auto get = [](const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
        put(mine + tid, m);
        put(mine + kPfWaveThreads + tid, l);
#pragma unroll
        for (int i = 0; i < ND; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) put(mine + (2 + 16 * i + r) * kPfWaveThreads + tid, oacc[i][r]);
        // a thread's stores must have completed before the block counts itself in: the barrier alone does not wait
        // for stores to memory (waves of a block share their unit's cache, so a barrier need not)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) arrived = atomicAdd(&counters[slot], 1);
        __syncthreads();
        if (arrived != n_parts - 1) return;
        if (tid == 0) counters[slot] = 0;                    // for the next launch
        for (int p = 0; p < n_parts; ++p) {
            if (p == part) continue;
            const float* other = scratch + ((size_t)slot * parts + p) * PF;
            const float m1 = get(other + tid), l1 = get(other + kPfWaveThreads + tid);
            const float m_new = fmaxf(m, m1);
            const float mc = ((m_new == -INFINITY) ? 0.f : m_new) * scale_log2e;
            const float c0 = __builtin_amdgcn_exp2f(m * scale_log2e - mc), c1 = __builtin_amdgcn_exp2f(m1 * scale_log2e - mc);
            l = l * c0 + l1 * c1;
            m = m_new;
#pragma unroll
            for (int i = 0; i < ND; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    oacc[i][r] = oacc[i][r] * c0 + get(other + (2 + 16 * i + r) * kPfWaveThreads + tid) * c1;
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

// bfloat16: the kernel above.  float32: the true-float32 kernel of attn_prefill_f32.hip (same tiles, one wave group, walks never cut).
IC_EXPORT int ic_attn_prefill_supported(int dtype, int dh, int page_size) {
    return (dtype == IC_BF16 || dtype == IC_F32) && (dh == 64 || dh == 128) && page_size > 0 && (page_size & (page_size - 1)) == 0;
}

int ic_attn_prefill_f32_launch(const void* q, int q_stride, void* out, int out_stride, const void* kcache, const void* vcache,
                               const int* block_tables, int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh,
                               int page_shift, float scale, int window, hipStream_t stream);

IC_EXPORT int ic_attn_prefill_tile_rows() { return kPfRows; }
IC_EXPORT int ic_attn_prefill_counter_ints() { return kPfCounters; }

// Floats of scratch memory that a walk cut into `parts` needs: every (tile, head, part) keeps a maximum, a sum and O^T per row.
IC_EXPORT long long ic_attn_prefill_scratch_floats(int n_tiles, int nh, int dh, int parts) {
    if (n_tiles <= 0 || nh <= 0 || parts <= 1 || (dh != 64 && dh != 128)) return 0;
    return (long long)n_tiles * nh * parts * kPfWaveThreads * (2 + dh / 2);
}

// How to cut the walks of a step whose longest query tile sees `max_keys` keys: parts per tile (1: no cut) and key tiles
// per part.  From sweeps over 16..48 heads of 64 and 32..40 of 128, prompts of 300..4,096 tokens and portions of 256..1,024
// after 256..3,584 tokens, against one and two wave groups:
//  * with many blocks, parts pay when walks are long (24 key tiles and more): as many parts as keep about 4.5 blocks a compute
//    unit at head size 64 and 2 at head size 128 (what stays resident there), at most 4, each of 6 key tiles or more; two
//    parts do no better than two wave groups where those run (up to 2 blocks a unit), so they keep that case;
//  * with few blocks (a portion or two beside decoded tokens) shorter walks are cut too: head size 64, up to half a block a
//    unit, from 12 key tiles on into 3 parts (4 from 20 key tiles on when four parts of every block still fit the units at once), and up to 1.25 blocks a unit
//    from 20 key tiles on into 3; head size 128, up to half a block a unit, walks of 8..23 key tiles into 2 parts, and up to a
//    quarter block a unit from 16 key tiles on into 4.  Against two wave groups, portions of 512 tokens after 512..768:
//    24:8 x 64 (96 blocks) 17.6 -> 14.7 and 20.0 -> 17.0 us, 32:2 x 128 (128 blocks) 25.9 -> 22.0 and 29.8 -> 25.1; 256
//    tokens after 1,024: 19.8 -> 13.9 and 29.2 -> 19.9;
//  * portions after a long past gain most (16 heads, 512 tokens after 3,584: 54 -> 26 us; 36 heads: 54 -> 41; 32:2 x 128: 83 -> 52),
//    whole prompts little (36 heads, 2,048 tokens: 43 -> 41 us) or nothing.
IC_EXPORT int ic_attn_prefill_parts(int n_tiles, int nh, int dh, int max_keys, int compute_units, int* part_len) {
    const int longest = (max_keys + kPfKeys - 1) / kPfKeys;
    const long long blocks = (long long)n_tiles * nh, cu = compute_units;
    int len = longest > 0 ? longest : 1, parts = 1;
    if (compute_units > 0 && blocks > 0 && blocks <= kPfCounters && (dh == 64 || dh == 128)) {
        long long p = 1;
        int least = 6;                                      // key tiles a part has at least
        bool few = false;
        if (dh == 64) {
            if (2 * blocks <= cu && longest >= 12) { p = (4 * blocks <= cu && longest >= 20) ? 4 : 3; few = true; }
            else if (4 * blocks <= 5 * cu && longest >= 20) { p = 3; few = true; }
        } else {
            if (4 * blocks <= cu && longest >= 16) { p = 4; few = true; }
            else if (2 * blocks <= cu && longest >= 8 && longest < 24) { p = 2; few = true; }
        }
        if (few) least = 4;
        else if (longest >= 24) {
            const long long room = dh == 64 ? 9LL * cu / 2 : 2LL * cu;
            p = room / blocks;
            p = p > 4 ? 4 : p;
            if (p == 2 && blocks <= 2LL * cu) p = 1;
        }
        p = p > longest / least ? longest / least : p;
        if (p >= 2) {
            parts = (int)p;
            len = (longest + parts - 1) / parts;
            len = len < least ? least : len;
        }
    }
    if (part_len) *part_len = len;
    return parts;
}

// The same question for a step: its largest position and the mixer's window (0: none) give the most keys a tile sees.
// (float32 walks are never cut.)
IC_EXPORT int ic_attn_prefill_parts_of_step(int dtype, int n_tiles, int nh, int dh, int max_position, int window, int compute_units, int* part_len) {
    int keys = max_position + 1;
    if (dtype != IC_BF16) {
        if (part_len) *part_len = (keys + kPfKeys - 1) / kPfKeys;
        return 1;
    }
    if (window > 0 && window + kPfRows < keys) keys = window + kPfRows;
    return ic_attn_prefill_parts(n_tiles, nh, dh, keys, compute_units, part_len);
}

// tiles: int32 [n_tiles, 4] = (request row of block_tables, first token row, rows <= 128, position of the first row).
// groups: 1 or 2 wave groups per query tile, 0 = chosen from the number of blocks.  parts > 1 (one group only): the grid
// holds `parts` blocks per (tile, head) and a tile's walk is cut into up to that many parts of at least part_len key
// tiles; scratch then holds ic_attn_prefill_scratch_floats(...) floats.
IC_EXPORT int ic_attn_prefill_split(const void* q, int q_stride, void* out, int out_stride, int dtype,
                                    const void* kcache, const void* vcache, const int* block_tables,
                                    int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh,
                                    int page_size, float scale, int window, int groups, int parts, int part_len,
                                    float* scratch, long long scratch_floats, int* counters, hipStream_t stream) {
    if (n_tiles <= 0) return IC_OK;
    if (!ic_attn_prefill_supported(dtype, dh, page_size)) return IC_ERR_UNSUPPORTED;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || page_size <= 0 || nh > 65535 || groups < 0 || groups > 2) return IC_ERR_ARG;
    if (dtype == IC_F32)                                  // (groups, parts and scratch do not apply: its walks are never cut)
        return ic_attn_prefill_f32_launch(q, q_stride, out, out_stride, kcache, vcache, block_tables, bt_stride, tiles, n_tiles, nh,
                                          nkvh, dh, page_shift, scale, window, stream);
    if (q_stride % 8 || out_stride % 4 || ((uintptr_t)q & 15) || ((uintptr_t)out & 7) ||
        ((uintptr_t)kcache & 15) || ((uintptr_t)vcache & 15) || ((uintptr_t)tiles & 15)) return IC_ERR_ARG;
    if (parts < 1) parts = 1;
    if (parts > 1) {
        if (groups == 2 || part_len < 1 || parts > 64 || (long long)nh * n_tiles > kPfCounters || !scratch || !counters ||
            ((uintptr_t)scratch & 15) || scratch_floats < ic_attn_prefill_scratch_floats(n_tiles, nh, dh, parts) ||
            (long long)nh * n_tiles * parts > 0x7fffffffLL) return IC_ERR_ARG;
        groups = 1;
    }
    const float sl2 = scale * 1.4426950408889634f;
    const bool staged = bt_stride <= kPfMaxPages;       // a block never needs more page ids than a request has
    // Few blocks (up to 2 per compute unit; measured with 16..64 heads of 64 and 32..40 of 128 over 512..4,096
    // tokens: two groups win up to 2.0 blocks a unit by 5..25 %, one group from 2.25 on by 2..25 %): the longest
    // tile's walk over the keys sets the time, so two wave groups share it.  Many blocks: one group, more blocks resident.
    static int cus = 0;                                 // compute units of the device, asked once
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
        else cus = 256;
    }
    const bool two_groups = groups ? groups == 2 : (long long)nh * n_tiles <= 2LL * cus;
    dim3 grid((unsigned)nh * (unsigned)n_tiles * (unsigned)parts);
    const bool page64 = page_size >= kPfKeys;            // (a power of two) a 64-key tile lies in one page
#define IC_PF_LAUNCH(DD, ST, GG, PP)                                                                                   \
    hipLaunchKernelGGL((attn_prefill_mfma_kernel<DD, ST, GG, PP>), grid, dim3(256 * GG), 0, stream, (const uint16_t*)q, \
                       q_stride, (uint16_t*)out, out_stride, (const uint16_t*)kcache, (const uint16_t*)vcache,      \
                       block_tables, bt_stride, (const int4*)tiles, n_tiles, nh, nkvh, page_shift, sl2, window,      \
                       parts, part_len, scratch, counters)
#define IC_PF_GROUPS(DD, ST) do { if (two_groups) { if (page64) IC_PF_LAUNCH(DD, ST, 2, true); else IC_PF_LAUNCH(DD, ST, 2, false); } \
                                  else { if (page64) IC_PF_LAUNCH(DD, ST, 1, true); else IC_PF_LAUNCH(DD, ST, 1, false); } } while (0)
    if (dh == 64) { if (staged) IC_PF_GROUPS(64, true); else IC_PF_GROUPS(64, false); }
    else if (dh == 128) { if (staged) IC_PF_GROUPS(128, true); else IC_PF_GROUPS(128, false); }
#undef IC_PF_GROUPS
#undef IC_PF_LAUNCH
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

IC_EXPORT int ic_attn_prefill_groups(const void* q, int q_stride, void* out, int out_stride, int dtype,
                                     const void* kcache, const void* vcache, const int* block_tables,
                                     int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh,
                                     int page_size, float scale, int window, int groups, hipStream_t stream) {
    return ic_attn_prefill_split(q, q_stride, out, out_stride, dtype, kcache, vcache, block_tables, bt_stride, tiles,
                                 n_tiles, nh, nkvh, dh, page_size, scale, window, groups, 1, 0, nullptr, 0, nullptr, stream);
}

IC_EXPORT int ic_attn_prefill(const void* q, int q_stride, void* out, int out_stride, int dtype,
                              const void* kcache, const void* vcache, const int* block_tables,
                              int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh,
                              int page_size, float scale, int window, hipStream_t stream) {
    return ic_attn_prefill_groups(q, q_stride, out, out_stride, dtype, kcache, vcache, block_tables, bt_stride, tiles,
                                  n_tiles, nh, nkvh, dh, page_size, scale, window, 0, stream);
}

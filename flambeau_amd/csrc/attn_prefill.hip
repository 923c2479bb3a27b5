// Tiled grouped-query attention over the paged cache for prompt portions: bf16 storage, float
// softmax, matrix cores (v_mfma_f32_16x16x32_bf16).
//
// A block of four waves takes 64 consecutive query tokens of one request (16 per wave) and, for
// one kv head, QT of the query heads that share it (QT = 4, 2 or 1, a divisor of the group size):
// each wave holds QT query tiles and reuses every key/value operand it reads from LDS QT times.
// Keys are walked in stages of 64 from the first key any of the block's queries may see to the
// last, through a ring of LDS stages filled straight from the cache pages
// (global_load_lds_dwordx4: each lane names its own 16 bytes, the wave's kilobyte lands in tile
// order), one bare barrier per stage.  The block's part of the block table sits in LDS.
//
// Everything is computed transposed, so that a query is a lane column:
//   S^T[key][query] = K . Q^T        A = K tile (LDS, stored as matrix-core tiles), B = Q (registers)
//   softmax per column: the base m of the exponents and the sum l live in the lanes that own the
//       column; rescaling the output needs no broadcast and happens only when a base moves, which
//       it does lazily (when a score exceeds it by more than a factor of 256): the usual chunk
//       costs no exchange between lanes
//   O^T[d][query] += V^T . P^T       A = V^T tile (the cache stores values transposed inside a
//       page, so its rows are runs of keys), B = P straight from the S^T accumulator
// Scores are scaled by scale * log2(e) and exponentiated with exp2.  Query at position p sees keys
// [max(0, p - window + 1), p]; keys outside are excluded, never scored.
//
// Reference: crates/kernels-hip/src/kernels/attention_prefill_flash_tile_f16.cu:43-330 (tiled
// prefill, 4 query rows per tile), attention_prefill_f16_paged.cu:50-150 (paged addressing).
#include "common.h"
#include "api.h"
#include "recordable.h"
#include "attn_merge.h"

#define PF_TOKENS 64          // query tokens per block
#define PF_STAGE 64           // keys per LDS stage
#define PF_MAX_PAGES 16384    // block-table entries a block keeps in LDS (64 KB; beyond 4,096 one block per compute unit)
#define PF_LDS_BYTES (160 * 1024)     // LDS of a compute unit: the ring of key/value stages and the table share it

// Which key sits in row i of the two 16-key score tiles of a 32-key chunk: tile a holds keys
// 8 (i / 4) + i % 4, tile b the same + 4.  A lane (query, g) of the score accumulators then owns
// the eight consecutive keys 8 g .. 8 g + 7 of the chunk (four from each tile), which is one
// 16-byte run of a row of the transposed values: the value operand needs no gathering.
__device__ __forceinline__ int pf_key_of_row(int i, int ab) { return 8 * (i >> 2) + 4 * ab + (i & 3); }

__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

template <int HDP, int QT, int NS>
__global__ __launch_bounds__(256, QT * HDP <= 256 ? 2 : 1) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, PagedCache cache,
    const int* __restrict__ tiles, const int* __restrict__ positions,
    const int* __restrict__ block_table, int max_blocks, int nh, float scale_log2e, int window,
    int log2_ps, int mirror_from, float* __restrict__ part_o, float* __restrict__ part_ml) {
    constexpr int QS = HDP / 32;              // k-steps of the score product
    constexpr int DT = HDP / 16;              // tiles of head dims in the output
    constexpr int KT = 4 * QS;                // 1 KB tiles of a K stage: [chunk (2)][a/b (2)][k-step]
    constexpr int VT = 2 * DT;                // of a V stage: [chunk (2)][dim tile]
    constexpr int LPW = (KT + VT) / 4;        // tile loads per wave and stage
    extern __shared__ __attribute__((aligned(16))) bf16_t ring[];       // [NS][KT + VT][512], then the pages
    int* s_pages = (int*)(ring + (size_t)NS * (KT + VT) * 512);         // [max_blocks]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);          // the same for the whole wave: branches on it are scalar
    const int j = lane & 15, g = lane >> 4;
    const int hd = cache.head_dim, ps = cache.page_size;
    const int G = nh / cache.n_kv_heads;
    const int hgroups = G / QT;
    // Tiles late in a prompt have the most keys: they are started first.  When the whole grid is on
    // the chip at once (two blocks per compute unit, the second half of the grid beside the first),
    // the second half runs the other way round, so that a long tile shares its unit with a short one.
    // A grid that comes in several rounds (mirror_from < 0) starts all head groups of the longest tile,
    // then all of the next: no long tile is left for the end.
    const int lin = blockIdx.y * gridDim.x + blockIdx.x;
    const int by = mirror_from < 0 ? lin % gridDim.y : blockIdx.y;
    const int tile = mirror_from < 0 ? gridDim.x - 1 - lin / gridDim.y
                                     : (lin < mirror_from ? gridDim.x - 1 - blockIdx.x : blockIdx.x);
    const int kvh = by / hgroups, hg = by % hgroups;
    const int seq = tiles[4 * tile], row0 = tiles[4 * tile + 1], cnt = tiles[4 * tile + 2], item0 = tiles[4 * tile + 3];
    const int* table = block_table + (size_t)seq * max_blocks;
    const bf16_t* kv = (const bf16_t*)cache.base;

    const int p_first = positions[row0], p_last = p_first + cnt - 1;
    const int lo = window > 0 ? max(0, p_first - window + 1) : 0;     // first key anyone here sees
    const int qtok = 16 * wave + j;
    const bool q_ok = qtok < cnt;
    const int p = q_ok ? p_first + qtok : -1;
    const int my_lo = window > 0 ? max(0, p - window + 1) : 0;
    const bool wave_on = 16 * wave < cnt;
    const int wp_first = p_first + 16 * wave, wp_last = min(p_last, wp_first + 15);
    const int w_lo = window > 0 ? max(0, wp_first - window + 1) : 0;

    // ---- the pages of the keys [lo, p_last] go to LDS; a missing page (a hole below a window,
    // or beyond the request) is replaced by the page of the last key: what is read from it is
    // finite and never used (such keys are masked)
    const int page0 = lo >> log2_ps, n_pg = (p_last >> log2_ps) - page0 + 1;
    const int safe_page = table[p_last >> log2_ps];
    for (int i = tid; i < n_pg; i += 256) {
        const int pg = table[page0 + i];
        s_pages[i] = (pg >= 0 && pg < cache.n_pages) ? pg : safe_page;
    }

    // ---- Q as B operand, QT tiles: lane (query j, g) holds Q[token][head][32 s + 8 g ..]
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8 qreg[QT][QS];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const int head = kvh * G + hg * QT + t;
#pragma unroll
        for (int s = 0; s < QS; ++s) {
            const int d = 32 * s + 8 * g;
            qreg[t][s] = (q_ok && d + 8 <= hd) ? *(const bf16x8*)(q + ((size_t)(row0 + qtok) * nh + head) * hd + d) : zero8;
        }
    }
    f32x4 o[QT][DT];
    f32x4 l[QT];                              // sums of the exponentials: every row of the tile holds the column's sum
    float m[QT], thr[QT];                     // base of the exponents and the score that moves the base
    const bf16_t one = (bf16_t)1.0f;
    const bf16x8 ones8 = {one, one, one, one, one, one, one, one};
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        m[t] = -INFINITY;
        thr[t] = -INFINITY;
        l[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < DT; ++d) o[t][d] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

    // ---- what this wave loads per stage: tiles tl = wave + 4 u of [K tiles | V tiles]; per lane the
    // key offset inside the stage and the offset inside the (page, head) block are fixed
    // (KT is a multiple of 4, so load u of every wave is a K tile for u < QS and a V tile from there on)
    int key_off[LPW], blk_off[LPW];
    const int head_k = kvh * ps * hd, head_v = (cache.n_kv_heads + kvh) * ps * hd;      // inside a page: below 2^31
    const unsigned page_stride = 2u * cache.n_kv_heads * ps * hd;
#pragma unroll
    for (int u = 0; u < LPW; ++u) {
        const int tl = wave + 4 * u;
        if (u < QS) {                                          // K tile: chunk, a/b, k-step
            // the four lanes of a quad copy 64 consecutive bytes of one key row (a quad spread over
            // four rows costs four cache lookups); the pieces of a row are exchanged by (row / 2) % 4
            // so that the operand reads meet no bank twice (see gemm_tiled.hip)
            const int c2 = tl / (2 * QS), ab = (tl / QS) & 1, s = tl % QS;
            key_off[u] = 32 * c2 + pf_key_of_row(lane >> 2, ab);
            int d = 32 * s + 8 * ((lane & 3) ^ ((lane >> 3) & 3));
            if (d + 8 > hd) d = 0;                             // padding dims: any finite data (Q is zero there)
            blk_off[u] = head_k + d;                           // + row * hd, row known per stage
        } else {                                               // V tile: chunk, dim tile
            const int tv = tl - KT;
            const int c2 = tv / DT, dt = tv % DT;
            key_off[u] = 32 * c2 + 8 * g;
            int d = 16 * dt + j;
            if (d >= hd) d = 0;                                // padding dims are never stored
            blk_off[u] = head_v + d * ps;                      // + row
        }
    }
    // operand lane (key row j, k-piece g) finds its 16 bytes of a K tile here
    const int k_read = 32 * j + 8 * (g ^ ((j >> 1) & 3));
    // the keys are walked in stages of 64; with gridDim.z > 1 this block takes one part of the stages
    // and leaves its result unnormalised for the merge (a short portion behind a long context gives
    // few tiles, and splitting the keys is what fills the chip then)
    const int all_stages = (p_last / PF_STAGE) - (lo / PF_STAGE) + 1;
    const int per_split = (all_stages + gridDim.z - 1) / gridDim.z;
    const int first_stage = min(all_stages, (int)blockIdx.z * per_split);
    const int n_stage = min(all_stages, first_stage + per_split) - first_stage;
    const int t_base = (lo / PF_STAGE) * PF_STAGE + first_stage * PF_STAGE;
    // A stage whose 64 keys all lie in [lo, p_last] needs no clamping, and then little arithmetic:
    // the keys of a load sit in one of the stage's two chunks of 32, at a row of its page that is
    // the same in every stage (pages divide 64 or are multiples of it), and the page a lane needs
    // within a chunk depends on lane / 16 only (keys 8 (lane / 16) .. + 7 of the chunk, for K and V
    // tiles alike).  So two look-ups and two multiplications per stage serve all loads.
    int in_page_c[LPW];
    bool second_chunk[LPW];
#pragma unroll
    for (int u = 0; u < LPW; ++u) {
        const int r = key_off[u] & (ps - 1);
        in_page_c[u] = blk_off[u] + (u < QS ? __mul24(r, hd) : r);
        second_chunk[u] = (u < QS ? (wave + 4 * u) / (2 * QS) : (wave + 4 * u - KT) / DT) != 0;      // the same for the wave
    }
    const int lane_pg = (8 * g) >> log2_ps;
    auto issue = [&](int i) {
        const int t0 = t_base + i * PF_STAGE;
        bf16_t* slot = ring + (size_t)(i % NS) * (KT + VT) * 512;
        const bf16_t* src[LPW];
        if (t0 >= lo && t0 + PF_STAGE - 1 <= p_last) {
            const bf16_t* base0 = kv + (uint64_t)(unsigned)s_pages[(t0 >> log2_ps) - page0 + lane_pg] * page_stride;
            const bf16_t* base1 = kv + (uint64_t)(unsigned)s_pages[((t0 + 32) >> log2_ps) - page0 + lane_pg] * page_stride;
            const int row_shift = t0 & (ps - 1);              // pages longer than a stage: where the stage begins in its page
            const int shift_k = row_shift * hd;
#pragma unroll
            for (int u = 0; u < LPW; ++u)
                src[u] = (second_chunk[u] ? base1 : base0) + (in_page_c[u] + (u < QS ? shift_k : row_shift));
        } else {
            // first every load's page is looked up (the compiler keeps an LDS read behind a copy into
            // LDS that precedes it: looked up one by one, each would wait for its own read), then the
            // copies are started
#pragma unroll
            for (int u = 0; u < LPW; ++u) {
                // keys outside [lo, p_last] are masked: read any valid one instead.  A value piece is a run
                // of 8 keys and keeps its place if any of its keys is needed (its page is alive then)
                int t = t0 + key_off[u];
                if (u < QS) t = min(max(t, lo), p_last);
                else if (t + 7 < lo || t > p_last) t = p_last & ~7;
                const unsigned page = (unsigned)s_pages[(t >> log2_ps) - page0];
                const int row = t & (ps - 1);
                // 32-bit arithmetic inside the page (24-bit factors: one full-rate multiply), one 32 x 32 -> 64
                // multiply for the page
                const int in_page = blk_off[u] + (u < QS ? __mul24(row, hd) : row);
                src[u] = kv + (uint64_t)page * page_stride + in_page;
            }
        }
#pragma unroll
        for (int u = 0; u < LPW; ++u)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src[u],
                                             (__attribute__((address_space(3))) void*)(slot + (wave + 4 * u) * 512), 16, 0, 0);
    };
    __syncthreads();                                            // s_pages is complete
#pragma unroll
    for (int i = 0; i < NS - 1; ++i)
        if (i < n_stage) issue(i);

    for (int i = 0; i < n_stage; ++i) {
        if (i + NS - 2 < n_stage) {
            __builtin_amdgcn_s_waitcnt(0xF70 | ((LPW * (NS - 2)) & 0xF) | ((((LPW * (NS - 2)) >> 4) & 3) << 14));
        } else {
            __builtin_amdgcn_s_waitcnt(0xF70);
        }
        asm volatile("s_barrier" ::: "memory");
        if (i + NS - 1 < n_stage) issue(i + NS - 1);
        const bf16_t* slot = ring + (size_t)(i % NS) * (KT + VT) * 512;
        // The scores of both halves of the stage go to the matrix cores first: the softmax of the
        // first half (vector unit) then runs while the second half's products are still in flight,
        // and the second softmax beside the first half's value products.
        bool act[2];
        f32x4 sa[2][QT], sb[2][QT];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int t0 = t_base + i * PF_STAGE + 32 * half;
            // wave-uniform: does any query of this wave see any key of this chunk?
            act[half] = wave_on && t0 <= wp_last && t0 + 31 >= w_lo;
            if (!act[half]) continue;
#pragma unroll
            for (int t = 0; t < QT; ++t) { sa[half][t] = (f32x4){0.f, 0.f, 0.f, 0.f}; sb[half][t] = sa[half][t]; }
            // all key tiles of the half are asked for at once: the later ones arrive behind the first products
            bf16x8 ka[QS], kb[QS];
#pragma unroll
            for (int s = 0; s < QS; ++s) {
                ka[s] = *(const bf16x8*)(slot + ((2 * half) * QS + s) * 512 + k_read);
                kb[s] = *(const bf16x8*)(slot + ((2 * half + 1) * QS + s) * 512 + k_read);
            }
#pragma unroll
            for (int s = 0; s < QS; ++s) {
#pragma unroll
                for (int t = 0; t < QT; ++t) {
                    sa[half][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[s], qreg[t][s], sa[half][t], 0, 0, 0);
                    sb[half][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[s], qreg[t][s], sb[half][t], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            if (!act[half]) continue;
            const int t0 = t_base + i * PF_STAGE + 32 * half;
            const bool need_mask = (t0 + 31 > wp_first) || (t0 < (window > 0 ? max(0, wp_last - window + 1) : 0));
            // the value tiles of this half are asked for now and arrive during the softmax (where
            // the registers allow it)
            constexpr bool EARLY_V = QT * HDP <= 256 && QT <= 2;
            bf16x8 vt[EARLY_V ? DT : 1];
            if (EARLY_V) {
#pragma unroll
                for (int d = 0; d < DT; ++d) vt[EARLY_V ? d : 0] = *(const bf16x8*)(slot + (KT + half * DT + d) * 512 + lane * 8);
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- softmax per query column; this lane holds keys t0 + 8 g + r (a) and + 4 + r (b).
            // m holds the raw (unscaled) score that the exponents are taken against.  It follows the
            // running maximum lazily: only when a score exceeds it by more than 8 in the exponent (a
            // factor of 256, harmless in float) does the column move its base and rescale what it
            // has summed.  With 64 columns per wave some running maximum moves in nearly every
            // chunk, a base almost never after the first ones; and whether any base has to move
            // is a vote of the lanes over their own scores, so the usual chunk needs no exchange
            // between lanes at all.
            if (need_mask) {
#pragma unroll
                for (int t = 0; t < QT; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int ka = t0 + 8 * g + r, kb = ka + 4;
                        sa[half][t][r] = (ka > p || ka < my_lo) ? -INFINITY : sa[half][t][r];
                        sb[half][t][r] = (kb > p || kb < my_lo) ? -INFINITY : sb[half][t][r];
                    }
            }
            float mx[QT];
            bool above = false;
#pragma unroll
            for (int t = 0; t < QT; ++t) {
                const f32x4 a = sa[half][t], b = sb[half][t];
                mx[t] = max3(max3(a[0], a[1], a[2]), max3(a[3], b[0], b[1]), fmaxf(b[2], b[3]));
                above = above || mx[t] > thr[t];
            }
            if (__any(above)) {
#pragma unroll
                for (int t = 0; t < QT; ++t) {
                    float cm = fmaxf(mx[t], __shfl_xor(mx[t], 16, 64));
                    cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
                    if (cm > thr[t]) {                          // the same for the four lanes of a column
                        // exp2(-inf) = 0: a column that had no key yet forgets its (empty) sums
                        const float corr = __builtin_amdgcn_exp2f((m[t] - cm) * scale_log2e);
                        l[t] *= corr;
#pragma unroll
                        for (int d = 0; d < DT; ++d) o[t][d] *= corr;
                        m[t] = cm;
                        thr[t] = cm + 8.0f / scale_log2e;
                    }
                }
            }
            bf16x8 pmat[QT];
#pragma unroll
            for (int t = 0; t < QT; ++t) {
                // the scale (with log2 e folded in) enters inside the exponent: one fma per value.  A
                // column that has seen no key yet keeps m = -inf: its base is 0 then (its scores
                // are all -inf, their exponentials 0)
                const float base = m[t] == -INFINITY ? 0.f : m[t] * scale_log2e;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pmat[t][r] = (bf16_t)__builtin_amdgcn_exp2f(fmaf(sa[half][t][r], scale_log2e, -base));
                    pmat[t][4 + r] = (bf16_t)__builtin_amdgcn_exp2f(fmaf(sb[half][t][r], scale_log2e, -base));
                }
                // the column's sum of exponentials (of the rounded ones, which are what the values
                // are weighted with) comes from the matrix cores too: a value tile of ones
                l[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones8, pmat[t], l[t], 0, 0, 0);
            }
            // ---- O^T += V^T P^T.  In a chunk at an end of [lo, p_last] the values of keys outside it
            // (rows of a page that were never written, or belong to whoever holds the page now) are
            // zeroed: their weights are 0, but 0 * NaN would not be
            const bool edge = t0 < lo || t0 + 31 > p_last;             // the same for the whole block
            u32x4 keep = {~0u, ~0u, ~0u, ~0u};
            if (edge) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int k0 = t0 + 8 * g + 2 * e;
                    keep[e] = ((k0 >= lo && k0 <= p_last) ? 0x0000FFFFu : 0u) | ((k0 + 1 >= lo && k0 + 1 <= p_last) ? 0xFFFF0000u : 0u);
                }
            }
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                bf16x8 vd = EARLY_V ? vt[EARLY_V ? d : 0] : *(const bf16x8*)(slot + (KT + half * DT + d) * 512 + lane * 8);
                if (edge) vd = __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, vd) & keep);
#pragma unroll
                for (int t = 0; t < QT; ++t)
                    o[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vd, pmat[t], o[t][d], 0, 0, 0);
            }
        }
    }

    if (!q_ok) return;
    if (gridDim.z > 1) {
        // ---- one part of the keys: the unnormalised output, the base of its exponents (in natural-log
        // units, as the merge wants it) and its sum go to the workspace
#pragma unroll
        for (int t = 0; t < QT; ++t) {
            const int head = kvh * G + hg * QT + t;
            const size_t at = ((size_t)(item0 + qtok) * nh + head) * gridDim.z + blockIdx.z;
            float* prow = part_o + at * HDP;
#pragma unroll
            for (int d = 0; d < DT; ++d) *(f32x4*)(prow + 16 * d + 4 * g) = o[t][d];
            if (g == 0) {
                part_ml[at * 2] = m[t] * scale_log2e * 0.6931471805599453f;
                part_ml[at * 2 + 1] = l[t][0];
            }
        }
        return;
    }
    // ---- normalise and store: lane (query j, g) holds dims 16 d + 4 g + r
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const float ll = l[t][0];
        const float inv = ll > 0.f ? 1.0f / ll : 0.f;
        const int head = kvh * G + hg * QT + t;
        bf16_t* orow = out + ((size_t)(row0 + qtok) * nh + head) * hd;
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            const int dd = 16 * d + 4 * g;
            if (dd + 4 <= hd) {
                const f32x4 v = o[t][d];
                bf16x4 ov = {(bf16_t)(v[0] * inv), (bf16_t)(v[1] * inv), (bf16_t)(v[2] * inv), (bf16_t)(v[3] * inv)};
                *(bf16x4*)(orow + dd) = ov;
            }
        }
    }
}

template <int HDP, int QT, int NS>
static void launch_prefill_one(dim3 grid, hipStream_t stream, const bf16_t* q, bf16_t* out, PagedCache c,
                               const int* tiles, const int* positions, const int* block_table, int max_blocks,
                               int nh, float scale_log2e, int window, int log2_ps, float* part_o, float* part_ml, int lds_pages) {
    // blocks that the chip holds at one time: one or two per compute unit
    const int units = fl_units();
    const int total = (int)(grid.x * grid.y * grid.z);
    constexpr int RING = NS * (4 * (HDP / 32) + 2 * (HDP / 16)) * 1024;
    const int lds = RING + lds_pages * (int)sizeof(int);
    const int resident = units * ((QT * HDP <= 256 && 2 * lds <= PF_LDS_BYTES) ? 2 : 1);
    // (whole rows of the grid: every tile of a head group is taken exactly once either way)
    const int mirror_from = (resident == 2 * units && grid.z == 1 && total <= resident && total > units) ? (int)((grid.y / 2) * grid.x)
                            : (grid.z == 1 && total > resident) ? -1 : (int)(grid.x * grid.y);
    static bool configured = false;
    auto kern = attn_prefill_kernel<HDP, QT, NS>;
    if (!configured) {
        (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  min(RING + PF_MAX_PAGES * (int)sizeof(int), PF_LDS_BYTES));
        configured = true;
    }
    kern<<<grid, 256, lds, stream>>>(q, out, c, tiles, positions, block_table, max_blocks, nh, scale_log2e, window, log2_ps, mirror_from, part_o, part_ml);
}

template <int HDP, int NS>
static void launch_prefill(int qt, dim3 grid, hipStream_t stream, const bf16_t* q, bf16_t* out, PagedCache c,
                           const int* tiles, const int* positions, const int* block_table, int max_blocks, int nh,
                           float scale_log2e, int window, int log2_ps, float* part_o, float* part_ml, int lds_pages) {
    if constexpr (HDP <= 64) {            // four heads per wave only where two blocks still fit a compute unit
        if (qt == 4) {
            launch_prefill_one<HDP, 4, NS>(grid, stream, q, out, c, tiles, positions, block_table, max_blocks, nh, scale_log2e, window, log2_ps, part_o, part_ml, lds_pages);
            return;
        }
    }
    if (qt >= 2)
        launch_prefill_one<HDP, 2, NS>(grid, stream, q, out, c, tiles, positions, block_table, max_blocks, nh, scale_log2e, window, log2_ps, part_o, part_ml, lds_pages);
    else
        launch_prefill_one<HDP, 1, NS>(grid, stream, q, out, c, tiles, positions, block_table, max_blocks, nh, scale_log2e, window, log2_ps, part_o, part_ml, lds_pages);
}

// Query heads per wave (QT, a divisor of the group size) and parts of the keys for a batch of n_tiles
// tiles whose longest context has max_keys keys.
//  * At most as many heads as leave room for two blocks per compute unit (two waves per SIMD hide each
//    other's waits: 906 against 1314 us at 8192 tokens with 2 heads instead of 4 at head size 128).
//  * A grid of fewer than two blocks per unit is filled by splitting the keys, as long as every part keeps
//    12 stages of 64 keys or so, rather than by fewer heads per wave: a block of two heads reads its keys
//    and values once for both (512 tokens behind 7,680 keys: 99 us with two heads and 4 parts against 125
//    with one head and 2; behind 32,256: 314 against 422; 64 tokens behind 32,704: 83 against 115).
//  * Where the keys are too few for that (a whole prompt of 1,024 tokens: 16 stages at most), fewer heads
//    per wave give the blocks (29 us with one head, 35 with two).
struct PrefillPlan { int qt, splits; };
static PrefillPlan pf_plan(int n_tiles, int nh, int nkv, int hd, int max_keys) {
    const int G = nh / nkv;
    const int hdp = ceil_div(hd, 32) * 32;
    int qt = (G % 4 == 0) ? 4 : (G % 2 == 0 ? 2 : 1);
    const int qt_max = hdp <= 64 ? 4 : 2;
    while (qt > qt_max) qt /= 2;
    const int slots = 2 * fl_units();
    const int by_keys = max(1, ceil_div(max(max_keys, 1), PF_STAGE) / 12);
    for (;; qt /= 2) {
        const int blocks = max(1, n_tiles * nkv * (G / qt));
        if (blocks >= slots) return {qt, 1};
        const int splits = max(1, min(min(slots / blocks, by_keys), 16));
        // (at the most parts there are, fewer heads would only read the keys more often)
        if (qt == 1 || splits == 16 || blocks * splits >= slots * 5 / 8) return {qt, splits};
    }
}

// query heads per wave for fl_attn_prefill: qt_hint (1, 2 or 4) at most that many; else what goes with
// the parts the caller has chosen
static int pf_heads_per_wave(int n_tiles, int nh, int nkv, int hd, int qt_hint, int n_split) {
    const int G = nh / nkv;
    const int hdp = ceil_div(hd, 32) * 32;
    int qt = (G % 4 == 0) ? 4 : (G % 2 == 0 ? 2 : 1);
    const int qt_max = hdp <= 64 ? 4 : 2;
    while (qt > qt_max) qt /= 2;
    if (qt_hint == 1 || qt_hint == 2 || qt_hint == 4) {
        while (qt > qt_hint) qt /= 2;
        return qt;
    }
    while (qt > 1 && n_tiles * nkv * (G / qt) * n_split < 3 * fl_units() / 2) qt /= 2;
    return qt;
}

// Query heads per wave for a batch of this shape (what fl_attn_prefill takes as its hint), and into how
// many parts its keys are split (1: not at all).
extern "C" int fl_attn_prefill_heads(int n_tiles, int nh, int nkv, int hd, int max_keys) {
    if (n_tiles <= 0 || nh <= 0 || nkv <= 0 || nh % nkv) return 1;
    return pf_plan(n_tiles, nh, nkv, hd, max_keys).qt;
}
extern "C" int fl_attn_prefill_splits(int n_tiles, int nh, int nkv, int hd, int max_keys) {
    if (n_tiles <= 0 || nh <= 0 || nkv <= 0 || nh % nkv) return 1;
    return pf_plan(n_tiles, nh, nkv, hd, max_keys).splits;
}

// Block-table entries per request that the kernel takes at a head size: the table of a request sits in
// LDS beside the ring of two stages of 64 keys and values (256 bytes per padded head dim and stage).
extern "C" int fl_attn_prefill_max_pages(int hd) {
    if (hd <= 0 || hd > 256) return 0;
    const int hdp = ceil_div(hd, 32) * 32;
    return min(PF_MAX_PAGES, (PF_LDS_BYTES - 2 * hdp * 256) / (int)sizeof(int));
}

// Entries of a request's table that a block may need: all of them, or with a window the pages of the
// window + 63 keys that its 64 queries see between them.
static int pf_table_need(int max_blocks, int page_size, int window) {
    if (window <= 0) return max_blocks;
    return min(max_blocks, (window + PF_TOKENS - 2) / page_size + 2);
}

// Whether fl_attn_prefill takes a cache of this shape with block tables max_blocks wide.
extern "C" int fl_attn_prefill_takes(int hd, int page_size, int max_blocks, int window) {
    if (hd <= 0 || hd > 256 || hd % 8 || page_size < 8 || (page_size & (page_size - 1)) || max_blocks < 0 || window < 0) return 0;
    return pf_table_need(max_blocks, page_size, window) <= fl_attn_prefill_max_pages(hd) ? 1 : 0;
}

// Workspace of the split form, in floats: part_o and part_ml for n_rows rows of tiles.
extern "C" int fl_attn_prefill_workspace(int n_rows, int nh, int hd, int n_split, long* o_floats, long* ml_floats) {
    const int hdp = ceil_div(hd, 32) * 32;
    *o_floats = (long)n_rows * nh * n_split * hdp;
    *ml_floats = (long)n_rows * nh * n_split * 2;
    return 0;
}

// Merge of the parts of the keys (at most 16): out[d] = sum_s part_o[s][d] e^(m_s - m) / sum_s l_s e^(m_s - m),
// m = max m_s, the sums in rising s.  A thread owns four head dims of one (row, head); a tile's 64 rows
// x heads x dims are dealt to its blocks in that order, so a wave reads whole rows of the partial
// outputs side by side.
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml,
                                                                 bf16_t* __restrict__ out, const int* __restrict__ tiles,
                                                                 int nh, int hd, int hdp, int n_split, int blocks_per_tile) {
    const int tile = blockIdx.x / blocks_per_tile;
    const int row0 = tiles[4 * tile + 1], cnt = tiles[4 * tile + 2], item0 = tiles[4 * tile + 3];
    const int quads = hdp >> 2;
    const int idx = (blockIdx.x % blocks_per_tile) * 256 + threadIdx.x;       // (row of the tile, head, quad of dims)
    const int q4 = idx % quads, head = (idx / quads) % nh, qtok = idx / (quads * nh);
    if (qtok >= cnt) return;
    const size_t base = ((size_t)(item0 + qtok) * nh + head) * n_split;
    float ms[16], ls[16];
    float mm = -INFINITY;
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        if (s < n_split) {
            const float2 ml = *(const float2*)(part_ml + (base + s) * 2);
            ms[s] = ml.x;
            ls[s] = ml.y;
            mm = fmaxf(mm, ml.x);
        }
    }
    float ll = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        if (s < n_split) {
            const float f = ms[s] == -INFINITY ? 0.f : expf(ms[s] - mm);
            ll += ls[s] * f;
            acc += *(const f32x4*)(part_o + (base + s) * hdp + 4 * q4) * f;
        }
    }
    const float inv = ll > 0.f ? 1.0f / ll : 0.f;
    const int d = 4 * q4;
    bf16_t* orow = out + ((size_t)(row0 + qtok) * nh + head) * hd;
    if (d + 4 <= hd) {
        const bf16x4 ov = {(bf16_t)(acc[0] * inv), (bf16_t)(acc[1] * inv), (bf16_t)(acc[2] * inv), (bf16_t)(acc[3] * inv)};
        *(bf16x4*)(orow + d) = ov;
    } else {
        for (int r = 0; r < 4 && d + r < hd; ++r) orow[d + r] = (bf16_t)(acc[r] * inv);
    }
}

// tiles[n_tiles][4] = (row of the request in the block table, first row, rows (at most 64), index of
// the first row among all rows of tiles).  n_split > 1 (fl_attn_prefill_splits): the keys are split,
// part_o and part_ml hold fl_attn_prefill_workspace floats.
extern "C" int fl_attn_prefill(const void* q, void* out, const void* cache_base, const int* tiles,
                               int n_tiles, const int* positions, const int* block_table,
                               int max_blocks, int nh, int nkv, int hd, int page_size, int n_pages,
                               float scale, int window, int qt_hint, float* part_o, float* part_ml, int n_split,
                               hipStream_t stream) {
    FL_CHECK(n_tiles >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attn_prefill: bad head counts %d/%d", nh, nkv);
    FL_CHECK(hd > 0 && hd <= 256 && hd % 8 == 0, "attn_prefill: head size %d must be a multiple of 8 up to 256", hd);
    FL_CHECK(page_size >= 8 && (page_size & (page_size - 1)) == 0,
             "attn_prefill: page size %d must be a power of two, at least 8", page_size);
    FL_CHECK((long long)2 * nkv * page_size * hd < (1ll << 31), "attn_prefill: a page of %d heads x %d keys x %d is too large (2^31 values)", nkv, page_size, hd);
    FL_CHECK(window >= 0, "attn_prefill: negative window");
    const int lds_pages = pf_table_need(max_blocks, page_size, window);
    FL_CHECK(lds_pages <= fl_attn_prefill_max_pages(hd), "attn_prefill: %d pages per request in reach of a block, at most %d with heads of %d",
             lds_pages, fl_attn_prefill_max_pages(hd), hd);
    FL_CHECK(scale > 0.f, "attn_prefill: the score scale must be positive");
    FL_CHECK(n_split >= 1 && n_split <= 16, "attn_prefill: %d splits (at most 16)", n_split);
    FL_CHECK(n_split == 1 || (part_o && part_ml && (uintptr_t)part_o % 16 == 0), "attn_prefill: splits need a 16-byte aligned workspace");
    FL_CHECK(n_split == 1 || (long long)n_tiles * PF_TOKENS * nh * (ceil_div(hd, 32) * 8) / 256 < (1ll << 31),
             "attn_prefill: %d tiles are too many to split", n_tiles);
    if (n_tiles == 0) return 0;
    PagedCache c{(void*)cache_base, nkv, page_size, hd, n_pages};
    const int G = nh / nkv;
    const int hdp = ceil_div(hd, 32) * 32;
    int log2_ps = 0;
    while ((1 << log2_ps) < page_size) ++log2_ps;
    const int qt = pf_heads_per_wave(n_tiles, nh, nkv, hd, qt_hint, n_split);
    dim3 grid(n_tiles, nkv * (G / qt), n_split);
    const float sl = scale * 1.4426950408889634f;
    // a ring of two stages: two blocks then fit a compute unit (three stages were no faster)
#define FL_PF(HDP_)                                                                                            \
    launch_prefill<HDP_, 2>(qt, grid, stream, (const bf16_t*)q, (bf16_t*)out, c, tiles, positions, block_table, \
                            max_blocks, nh, sl, window, log2_ps, part_o, part_ml, lds_pages)
    switch (hdp) {
        case 32: FL_PF(32); break;
        case 64: FL_PF(64); break;
        case 96: FL_PF(96); break;
        case 128: FL_PF(128); break;
        case 160: FL_PF(160); break;
        case 192: FL_PF(192); break;
        case 224: FL_PF(224); break;
        default: FL_PF(256); break;
    }
#undef FL_PF
    FL_LAUNCH_CHECK();
    if (n_split > 1) {
        const int blocks_per_tile = ceil_div(PF_TOKENS * nh * (hdp / 4), 256);
        attn_prefill_merge_kernel<<<n_tiles * blocks_per_tile, 256, 0, stream>>>(part_o, part_ml, (bf16_t*)out, tiles, nh, hd,
                                                                                 hdp, n_split, blocks_per_tile);
        FL_LAUNCH_CHECK();
    }
    return 0;
}
FL_RECORDABLE(fl_attn_prefill)

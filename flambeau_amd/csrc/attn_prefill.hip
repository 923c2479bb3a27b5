// Tiled grouped-query attention over the paged cache for prompt portions: bf16 storage, float
// softmax, matrix cores (v_mfma_f32_16x16x32_bf16).
//
// A block of four waves takes 64 consecutive query tokens of one request (16 per wave) and, for
// one kv head, QT of the query heads that share it (QT = 4, 2 or 1, a divisor of the group size):
// each wave holds QT query tiles and reuses every key/value operand it reads from LDS QT times.
// Keys are walked in stages of 64 from the first key any of the block's queries may see to the
// last; the next stage is fetched from the cache pages into registers while the current one is
// multiplied, and put into the other LDS buffer.
//
// Everything is computed transposed, so that a query is a lane column:
//   S^T[key][query] = K . Q^T        A = K tile (LDS, stored as matrix-core tiles), B = Q (registers)
//   softmax per column: running max m and sum l live in the lanes that own the column; rescaling
//       the output needs no broadcast and is skipped when no maximum moved
//   O^T[d][query] += V^T . P^T       A = V^T tile (the cache stores values transposed inside a
//       page, so its rows are runs of keys), B = P straight from the S^T accumulator
// Scores are scaled by scale * log2(e) and exponentiated with exp2.  Query at position p sees keys
// [max(0, p - window + 1), p]; keys outside are excluded, never scored.
//
// Reference: crates/kernels-hip/src/kernels/attention_prefill_flash_tile_f16.cu:43-330 (tiled
// prefill, 4 query rows per tile), attention_prefill_f16_paged.cu:50-150 (paged addressing).
#include "common.h"
#include "api.h"

#define PF_TOKENS 64          // query tokens per block
#define PF_STAGE 64           // keys per LDS stage

typedef __attribute__((ext_vector_type(4))) unsigned int pf_u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int pf_u32x2;

template <int HDP, int QT, int NBUF>
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, PagedCache cache,
    const int* __restrict__ tiles, const int* __restrict__ positions,
    const int* __restrict__ block_table, int max_blocks, int nh, float scale_log2e, int window) {
    constexpr int QS = HDP / 32;              // k-steps of the score product
    constexpr int DT = HDP / 16;              // tiles of head dims in the output
    constexpr int KCH = PF_STAGE * HDP / 8;   // 16-byte chunks of a K stage
    constexpr int VPC = PF_STAGE * HDP / 4;   // 8-byte pieces of a V stage
    constexpr int KPT = KCH / 256, VPT = VPC / 256;
    // K stage: [key tile (4)][k-step (QS)][512]; V stage: [32-key chunk (2)][dim tile (DT)][512]
    __shared__ __attribute__((aligned(16))) bf16_t ks[NBUF][PF_STAGE / 16][QS][512];
    __shared__ __attribute__((aligned(16))) bf16_t vs[NBUF][PF_STAGE / 32][DT][512];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int j = lane & 15, g = lane >> 4;
    const int hd = cache.head_dim, ps = cache.page_size;
    const int G = nh / cache.n_kv_heads;
    const int hgroups = G / QT;
    const int kvh = blockIdx.y / hgroups, hg = blockIdx.y % hgroups;
    const int seq = tiles[3 * blockIdx.x], row0 = tiles[3 * blockIdx.x + 1], cnt = tiles[3 * blockIdx.x + 2];
    const int* table = block_table + (size_t)seq * max_blocks;
    const bf16_t* kv = (const bf16_t*)cache.base;

    const int p_first = positions[row0], p_last = p_first + cnt - 1;
    const int lo = window > 0 ? max(0, p_first - window + 1) : 0;     // first key anyone here sees
    // this lane's query
    const int qtok = 16 * wave + j;
    const bool q_ok = qtok < cnt;
    const int p = q_ok ? p_first + qtok : -1;
    const int my_lo = window > 0 ? max(0, p - window + 1) : 0;
    // this wave's span of positions (wave-uniform)
    const bool wave_on = 16 * wave < cnt;
    const int wp_first = p_first + 16 * wave, wp_last = min(p_last, wp_first + 15);
    const int w_lo = window > 0 ? max(0, wp_first - window + 1) : 0;

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
    float m[QT], l[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        m[t] = -INFINITY;
        l[t] = 0.f;
#pragma unroll
        for (int d = 0; d < DT; ++d) o[t][d] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

    // ---- staging of one 64-key stage
    pf_u32x4 kr[KPT];
    pf_u32x2 vr[VPT];
    const int PP = ps < PF_STAGE ? ps : PF_STAGE;        // keys of a page that lie in one stage
    const int v_per_part = HDP * (PP / 4);               // 8-byte pieces of one page part
    auto fetch = [&](int t0) {
#pragma unroll
        for (int u = 0; u < KPT; ++u) {
            const int c = tid + 256 * u;
            const int kk = c / (HDP / 8), dc = c % (HDP / 8);
            const int t = t0 + kk;
            int page = (t >= lo && t <= p_last) ? table[t / ps] : -1;
            if (page >= cache.n_pages) page = -1;
            kr[u] = (page >= 0 && dc * 8 + 8 <= hd)
                        ? *(const pf_u32x4*)(kv + cache_k_offset(cache, page, kvh, t % ps, dc * 8))
                        : (pf_u32x4){0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const int c = tid + 256 * u;
            const int part = c / v_per_part, rem = c % v_per_part;
            const int d = rem / (PP / 4), r4 = rem % (PP / 4);
            const int t = t0 + part * PP + 4 * r4;
            int page = (t + 3 >= lo && t <= p_last) ? table[t / ps] : -1;
            if (page >= cache.n_pages) page = -1;
            vr[u] = (page >= 0 && d < hd) ? *(const pf_u32x2*)(kv + cache_v_offset(cache, page, kvh, t % ps, d))
                                           : (pf_u32x2){0u, 0u};
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int u = 0; u < KPT; ++u) {
            const int c = tid + 256 * u;
            const int kk = c / (HDP / 8), dc = c % (HDP / 8);
            *(pf_u32x4*)&ks[buf][kk >> 4][dc >> 2][(16 * (dc & 3) + (kk & 15)) * 8] = kr[u];
        }
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const int c = tid + 256 * u;
            const int part = c / v_per_part, rem = c % v_per_part;
            const int d = rem / (PP / 4), r4 = rem % (PP / 4);
            const int q4 = (part * PP) / 4 + r4;          // group of 4 keys within the stage, 0..15
            // 32-key chunk q4 / 8; within it tile a/b = (q4 / 4) % 2, lane group g = q4 % 4
            *(pf_u32x2*)&vs[buf][q4 >> 3][d >> 4][(16 * (q4 & 3) + (d & 15)) * 8 + 4 * ((q4 >> 2) & 1)] = vr[u];
        }
    };

    const int st_first = lo / PF_STAGE, st_last = p_last / PF_STAGE;
    int buf = 0;
    fetch(st_first * PF_STAGE);
    stash(0);
    __syncthreads();
    for (int st = st_first; st <= st_last; ++st) {
        const bool more = st < st_last;
        if (more) fetch((st + 1) * PF_STAGE);
        if (NBUF == 1) __syncthreads();       // (single buffer: computed below before it is overwritten)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int t0 = st * PF_STAGE + 32 * half;
            // wave-uniform: does any query of this wave see any key of this chunk?
            if (!wave_on || t0 > wp_last || t0 + 31 < w_lo) continue;
            const bool need_mask = (t0 + 31 > wp_first) || (t0 < (window > 0 ? max(0, wp_last - window + 1) : 0));
            // ---- scores
            f32x4 sa[QT], sb[QT];
#pragma unroll
            for (int t = 0; t < QT; ++t) { sa[t] = (f32x4){0.f, 0.f, 0.f, 0.f}; sb[t] = sa[t]; }
#pragma unroll
            for (int s = 0; s < QS; ++s) {
                const bf16x8 ka = *(const bf16x8*)&ks[buf][2 * half][s][lane * 8];
                const bf16x8 kb = *(const bf16x8*)&ks[buf][2 * half + 1][s][lane * 8];
#pragma unroll
                for (int t = 0; t < QT; ++t) {
                    sa[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qreg[t][s], sa[t], 0, 0, 0);
                    sb[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, qreg[t][s], sb[t], 0, 0, 0);
                }
            }
            // ---- softmax per query column; this lane holds keys t0 + 4 g + r (a) and + 16 (b)
            bf16x8 pmat[QT];
            bool moved = false;
            float corr[QT];
#pragma unroll
            for (int t = 0; t < QT; ++t) {
                float mx = -INFINITY;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float va = sa[t][r] * scale_log2e, vb = sb[t][r] * scale_log2e;
                    if (need_mask) {
                        const int ka = t0 + 4 * g + r, kb = ka + 16;
                        if (ka > p || ka < my_lo) va = -INFINITY;
                        if (kb > p || kb < my_lo) vb = -INFINITY;
                    }
                    sa[t][r] = va;
                    sb[t][r] = vb;
                    mx = fmaxf(mx, fmaxf(va, vb));
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                const float m_new = fmaxf(m[t], mx);
                // a column that has seen no key yet keeps m = -inf: use 0 as the base then
                const float base = m_new == -INFINITY ? 0.f : m_new;
                corr[t] = __builtin_amdgcn_exp2f(m[t] - base);        // exp2(-inf) = 0
                if (m_new != m[t]) moved = true;
                float ls = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float ea = __builtin_amdgcn_exp2f(sa[t][r] - base);
                    const float eb = __builtin_amdgcn_exp2f(sb[t][r] - base);
                    ls += ea + eb;
                    pmat[t][r] = (bf16_t)ea;
                    pmat[t][4 + r] = (bf16_t)eb;
                }
                l[t] = l[t] * corr[t] + ls;
                m[t] = m_new;
            }
            // ---- rescale the output only if some maximum in the wave moved
            if (__any(moved)) {
#pragma unroll
                for (int t = 0; t < QT; ++t)
#pragma unroll
                    for (int d = 0; d < DT; ++d) o[t][d] *= corr[t];
            }
            // ---- O^T += V^T P^T
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                const bf16x8 vt = *(const bf16x8*)&vs[buf][half][d][lane * 8];
#pragma unroll
                for (int t = 0; t < QT; ++t)
                    o[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt, pmat[t], o[t][d], 0, 0, 0);
            }
        }
        if (more) {
            if (NBUF == 1) __syncthreads();
            stash(NBUF == 1 ? 0 : buf ^ 1);
        }
        __syncthreads();
        if (NBUF == 2) buf ^= 1;
    }

    // ---- normalise and store: lane (query j, g) holds dims 16 d + 4 g + r
    if (!q_ok) return;
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        float ll = l[t];
        ll += __shfl_xor(ll, 16, 64);
        ll += __shfl_xor(ll, 32, 64);
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

template <int HDP, int NBUF>
static void launch_prefill(int qt, dim3 grid, hipStream_t stream, const bf16_t* q, bf16_t* out, PagedCache c,
                           const int* tiles, const int* positions, const int* block_table, int max_blocks, int nh,
                           float scale_log2e, int window) {
    if (qt == 4)
        attn_prefill_kernel<HDP, 4, NBUF><<<grid, 256, 0, stream>>>(q, out, c, tiles, positions, block_table, max_blocks, nh, scale_log2e, window);
    else if (qt == 2)
        attn_prefill_kernel<HDP, 2, NBUF><<<grid, 256, 0, stream>>>(q, out, c, tiles, positions, block_table, max_blocks, nh, scale_log2e, window);
    else
        attn_prefill_kernel<HDP, 1, NBUF><<<grid, 256, 0, stream>>>(q, out, c, tiles, positions, block_table, max_blocks, nh, scale_log2e, window);
}

extern "C" int fl_attn_prefill(const void* q, void* out, const void* cache_base, const int* tiles,
                               int n_tiles, const int* positions, const int* block_table,
                               int max_blocks, int nh, int nkv, int hd, int page_size, int n_pages,
                               float scale, int window, int qt_hint, hipStream_t stream) {
    FL_CHECK(n_tiles >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attn_prefill: bad head counts %d/%d", nh, nkv);
    FL_CHECK(hd > 0 && hd <= 256 && hd % 8 == 0, "attn_prefill: head size %d must be a multiple of 8 up to 256", hd);
    FL_CHECK(page_size >= 4 && (PF_STAGE % page_size == 0 || page_size % PF_STAGE == 0),
             "attn_prefill: page size %d must divide %d or be a multiple of it", page_size, PF_STAGE);
    FL_CHECK(window >= 0, "attn_prefill: negative window");
    if (n_tiles == 0) return 0;
    PagedCache c{(void*)cache_base, nkv, page_size, hd, n_pages};
    const int G = nh / nkv;
    const int hdp = ceil_div(hd, 32) * 32;
    // query heads per wave: a divisor of the group size, as many as the registers hold
    int qt = (G % 4 == 0) ? 4 : (G % 2 == 0 ? 2 : 1);
    const int qt_max = hdp <= 128 ? 4 : (hdp <= 192 ? 2 : 1);
    while (qt > qt_max) qt /= 2;
    if (qt_hint == 1 || qt_hint == 2 || qt_hint == 4)
        while (qt > qt_hint) qt /= 2;
    dim3 grid(n_tiles, nkv * (G / qt));
    const float sl = scale * 1.4426950408889634f;
#define FL_PF(HDP_, NBUF_)                                                                                     \
    launch_prefill<HDP_, NBUF_>(qt, grid, stream, (const bf16_t*)q, (bf16_t*)out, c, tiles, positions, block_table, \
                                max_blocks, nh, sl, window)
    switch (hdp) {
        case 32: FL_PF(32, 2); break;
        case 64: FL_PF(64, 2); break;
        case 96: FL_PF(96, 2); break;
        case 128: FL_PF(128, 2); break;
        case 160: FL_PF(160, 1); break;
        case 192: FL_PF(192, 1); break;
        case 224: FL_PF(224, 1); break;
        default: FL_PF(256, 1); break;
    }
#undef FL_PF
    FL_LAUNCH_CHECK();
    return 0;
}

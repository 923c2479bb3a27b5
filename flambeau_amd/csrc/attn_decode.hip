// Split-K grouped-query attention over the paged cache for single query rows (decode rows, and
// the rows of short prompt portions): bf16 storage, float arithmetic, matrix cores.
//
// Work item = (query row, kv head, split); a query row comes as (row, position, request, 0), or, with
// splits of its own, once per split as (row, position, request, split + 256 * splits): the caller
// then gives long contexts more splits than short ones, and the blocks take about equally long
// (with one number of splits for all, the longest context of a ragged batch ends the kernel alone).  A
// block of four waves handles the (up to 16) query heads that share one kv head over the keys of
// its split, 32 keys per wave at a time:
//
//   S^T[key][head] = K[key][:] . Q[head][:]     v_mfma_f32_16x16x32_bf16, A = K rows read
//                                               straight from the cache pages (head dims are
//                                               contiguous), B = Q (kept in registers)
//   per head (one lane column): running max and sum; scores and their exponentials never leave
//   the lane that owns the column, so no broadcast is needed to rescale
//   O^T[d][head]  += V^T[d][key] . P^T[key][head]   A = values, which the cache stores transposed
//                                               inside a page (keys contiguous: one 16-byte load
//                                               per lane), B = P from the S^T accumulator without
//                                               any data movement
//
// The four waves' states are merged through LDS; with more than one split the block writes a
// partial (max, sum, O) and a second kernel merges the splits (same rule: exp(m_c - m_max)).
// (Merging in the block that finishes last was tried twice: with a device-wide release fence in every
// block it is far slower, since each fence writes the L2 back, one block after the other; with
// device-scope loads and stores and a relaxed counter instead of fences it takes as long as the second
// kernel that it saves.)  Keys and values are loaded with the non-temporal hint: a step reads each
// byte of them once, and streaming reads are a tenth faster with the hint.
// Which keys a row sees depends on its own position only: [max(0, p - window + 1), p].
//
// Reference: crates/kernels-hip/src/kernels/attention_decode_f16_paged.cu:49-158 (paged decode),
// attention_decode_f16_splitk.cu:31-256 (partials and merge).
#include "common.h"
#include "api.h"
#include "recordable.h"
#include "attn_merge.h"
#include <mutex>

#define DEC_WAVES 4
#define DEC_CHUNK 32

// items[i] = (row of q and out, position, request, 0 or split + 256 * splits): everything a block needs
// to find its keys comes with one load.
template <int HDP>
__global__ __launch_bounds__(256, HDP <= 128 ? 2 : 1) void attn_decode_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, float* part_o,
    float* part_ml, PagedCache cache, const int4* __restrict__ items,
    const int* __restrict__ block_table, int max_blocks, int nh, float scale, int window,
    int n_split, int q_tiles, int ps_shift, int item_base) {
    constexpr int QS = HDP / 32;     // k-steps of the score product
    constexpr int DT = HDP / 16;     // 16-wide tiles of head dims in the output
    constexpr bool PIPELINED = HDP <= 128;       // two chunks of keys and values fit the registers
    __shared__ float s_m[DEC_WAVES][16], s_l[DEC_WAVES][16];
    __shared__ f32x4 s_o[DEC_WAVES - 1][DT][64];     // wave 0 keeps its own in registers

    // (the items are the slow index of the grid: the places of a list that no row uses come last)
    const int item = item_base + blockIdx.y;
    const int kvh = blockIdx.x / q_tiles, qt = blockIdx.x % q_tiles;
    const int4 it = items[item];
    if (it.x < 0) return;                              // a place in the list that no row uses
    // an item with splits of its own says which split it is; its partial result lies in the slot of the item
    const bool own_splits = it.w != 0;
    const int split = own_splits ? (it.w & 255) : (int)blockIdx.z;
    if (own_splits) n_split = it.w >> 8;
    const int token = it.x, p = it.y;
    const int hd = cache.head_dim, ps = cache.page_size;
    const int G = nh / cache.n_kv_heads;
    const int* table = block_table + (size_t)it.z * max_blocks;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);      // the same for the whole wave: what depends on it is scalar
    const int li = lane & 15, g = lane >> 4;
    const bf16_t* kv = (const bf16_t*)cache.base;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // this split's chunks of 32 keys
    const int c_lo = lo / DEC_CHUNK, c_hi = p / DEC_CHUNK;
    const int per = (c_hi - c_lo + n_split) / n_split;
    const int c0 = c_lo + split * per, c1 = min(c_hi + 1, c0 + per);

    // Q as B operand: lane (head li, group g) holds Q[head][32 s + 8 g .. +7]
    const int head = kvh * G + qt * 16 + li;
    const bool head_ok = qt * 16 + li < G;
    bf16x8 qreg[QS];
#pragma unroll
    for (int s = 0; s < QS; ++s) {
        const int d = 32 * s + 8 * g;
        qreg[s] = (head_ok && d + 8 <= hd) ? *(const bf16x8*)(q + ((size_t)token * nh + head) * hd + d) : zero8;
    }

    f32x4 o[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) o[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    // Row i of score tile a is key t0 + 8 (i / 4) + i % 4, of tile b the same + 4: a lane (head, g)
    // of the accumulators then owns the 8 consecutive keys t0 + 8 g .. + 7, one 16-byte run of a
    // row of the transposed values.  The two keys of a lane lie in one page (pages hold multiples of 8).
    const int k_off = 8 * (li >> 2) + (li & 3), v_off = 8 * g;
    struct Chunk { bf16x8 xa[QS], xb[QS], wv[DT]; };
    auto page_of = [&](int key) { return ps_shift >= 0 ? key >> ps_shift : key / ps; };
    auto row_of = [&](int key) { return ps_shift >= 0 ? key & (ps - 1) : key % ps; };
    // Loads carry no conditions (a branch around a load would make every wait a wait for all loads
    // in flight): keys outside [lo, p] are clamped into it, page ids outside the pool to a page of
    // the pool, chunks beyond the split to its last chunk; what such a load brings is masked in
    // compute().  Pages of chunk c for this lane: of its two keys and of its eight values.
    const int c_last = c1 - 1;
    auto page_ids = [&](int c, int& pk, int& pv) {
        c = min(c, c_last);
        const int ka = min(max(c * DEC_CHUNK + k_off, lo), p), vk = min(max(c * DEC_CHUNK + v_off, lo), p);
        pk = table[page_of(ka)];
        pv = table[page_of(vk)];
    };
    auto load_chunk = [&](Chunk& f, int c, int pk, int pv) {
        c = min(c, c_last);
        const int ka = c * DEC_CHUNK + k_off, vk = c * DEC_CHUNK + v_off;
        pk = (int)min((unsigned)pk, (unsigned)cache.n_pages - 1u);
        pv = (int)min((unsigned)pv, (unsigned)cache.n_pages - 1u);
        const bf16_t* rowa = kv + cache_k_offset(cache, pk, kvh, row_of(ka), 0);
        const bf16_t* rowb = rowa + 4 * hd;          // key ka + 4: the same page
#pragma unroll
        for (int s = 0; s < QS; ++s) {
            const int d = min(32 * s + 8 * g, hd - 8);       // head dims beyond hd: q is zero there
            f.xa[s] = __builtin_nontemporal_load((const bf16x8*)(rowa + d));
            f.xb[s] = __builtin_nontemporal_load((const bf16x8*)(rowb + d));
        }
        const bf16_t* vrow = kv + cache_v_offset(cache, pv, kvh, row_of(vk), 0);
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            const int d = min(16 * t + li, hd - 1);          // rows beyond hd are never stored
            f.wv[t] = __builtin_nontemporal_load((const bf16x8*)(vrow + (size_t)d * ps));
        }
    };
    auto compute = [&](const Chunk& f, int c) {
        const int t0 = c * DEC_CHUNK;
        f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < QS; ++s) {
            sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.xa[s], qreg[s], sa, 0, 0, 0);
            sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.xb[s], qreg[s], sb, 0, 0, 0);
        }
        // online softmax; this lane holds keys t0 + 8 g + r (tile a) and + 4 + r (tile b) for head li
        float mt = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int ka = t0 + 8 * g + r, kb = ka + 4;
            sa[r] = (ka >= lo && ka <= p) ? sa[r] * scale : -INFINITY;
            sb[r] = (kb >= lo && kb <= p) ? sb[r] * scale : -INFINITY;
            mt = fmaxf(mt, fmaxf(sa[r], sb[r]));
        }
        mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const float m_new = fmaxf(m, mt);          // finite: every chunk holds a visible key
        const float corr = expf(m - m_new);
        bf16x8 pb8;
        float ls = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float ea = expf(sa[r] - m_new), eb = expf(sb[r] - m_new);
            ls += ea + eb;
            pb8[r] = (bf16_t)ea;
            pb8[4 + r] = (bf16_t)eb;
        }
        l = l * corr + ls;
        m = m_new;
        if (t0 < lo || t0 + DEC_CHUNK - 1 > p) {
            // a chunk at an end of the range: values of keys outside it (whatever the page holds
            // there) are zeroed, since 0 * NaN would not be 0
            u32x4 keep;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int k0 = t0 + 8 * g + 2 * e;
                keep[e] = ((k0 >= lo && k0 <= p) ? 0x0000FFFFu : 0u) | ((k0 + 1 >= lo && k0 + 1 <= p) ? 0xFFFF0000u : 0u);
            }
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                o[t] *= corr;
                const u32x4 v = __builtin_bit_cast(u32x4, f.wv[t]) & keep;
                o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, v), pb8, o[t], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                o[t] *= corr;
                o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.wv[t], pb8, o[t], 0, 0, 0);
            }
        }
    };

    // The wave's chunks are c0 + wave, + 4, ...  What bounds a short split is the chain page id ->
    // key and value loads -> arithmetic, so the chain is pipelined: page ids two chunks ahead, keys
    // and values one chunk ahead, in two register sets that swap roles.  The loop body has no
    // branch, so the compiler's count of the loads in flight is exact.
    int c = c0 + wave;
    if (c < c1) {
        if (PIPELINED) {
            Chunk fa, fb;
            int pk0, pv0, pk1, pv1;
            page_ids(c, pk0, pv0);
            page_ids(c + DEC_WAVES, pk1, pv1);
            load_chunk(fa, c, pk0, pv0);
            for (; c + 2 * DEC_WAVES < c1; c += 2 * DEC_WAVES) {
                page_ids(c + 2 * DEC_WAVES, pk0, pv0);
                load_chunk(fb, c + DEC_WAVES, pk1, pv1);
                compute(fa, c);
                page_ids(c + 3 * DEC_WAVES, pk1, pv1);
                load_chunk(fa, c + 2 * DEC_WAVES, pk0, pv0);
                compute(fb, c + DEC_WAVES);
            }
            if (c + DEC_WAVES < c1) {               // two chunks left
                load_chunk(fb, c + DEC_WAVES, pk1, pv1);
                compute(fa, c);
                compute(fb, c + DEC_WAVES);
            } else {
                compute(fa, c);
            }
        } else {
            Chunk f;
            for (; c < c1; c += DEC_WAVES) {
                int pk, pv;
                page_ids(c, pk, pv);
                load_chunk(f, c, pk, pv);
                compute(f, c);
            }
        }
    }
    // sum over the four key groups of a head
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);

    // ---- merge the waves
    if (g == 0) { s_m[wave][li] = m; s_l[wave][li] = l; }
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < DT; ++t) s_o[wave - 1][t][lane] = o[t];
    }
    __syncthreads();
    if (wave == 0) {
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) mm = fmaxf(mm, s_m[w][li]);
        float f[DEC_WAVES], ll = 0.f;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) {
            f[w] = s_m[w][li] == -INFINITY ? 0.f : expf(s_m[w][li] - mm);
            ll += s_l[w][li] * f[w];
        }
        // lane (head li, group g) holds dims 16 t + 4 g + r
        if (head_ok && n_split == 1) {
            const float inv = ll > 0.f ? 1.0f / ll : 0.f;
            bf16_t* orow = out + ((size_t)token * nh + head) * hd;
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                f32x4 acc = o[t] * f[0];
#pragma unroll
                for (int w = 1; w < DEC_WAVES; ++w) acc += s_o[w - 1][t][lane] * f[w];
                const int d = 16 * t + 4 * g;
                if (d + 4 <= hd) {
                    bf16x4 ov = {(bf16_t)(acc[0] * inv), (bf16_t)(acc[1] * inv), (bf16_t)(acc[2] * inv), (bf16_t)(acc[3] * inv)};
                    *(bf16x4*)(orow + d) = ov;
                }
            }
        } else if (head_ok) {
            const size_t slot = own_splits ? (size_t)item * nh + head : ((size_t)item * nh + head) * n_split + split;
            if (g == 0) { part_ml[slot * 2] = mm; part_ml[slot * 2 + 1] = ll; }
            float* prow = part_o + slot * HDP;
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                f32x4 acc = o[t] * f[0];
#pragma unroll
                for (int w = 1; w < DEC_WAVES; ++w) acc += s_o[w - 1][t][lane] * f[w];
                *(f32x4*)(prow + 16 * t + 4 * g) = acc;
            }
        }
    }
}

// Merge of the splits: one block per (item, head) (attn_merge.h).
__global__ __launch_bounds__(256) void attn_decode_merge_kernel(const float* __restrict__ part_o,
                                                                const float* __restrict__ part_ml,
                                                                bf16_t* __restrict__ out,
                                                                const int4* __restrict__ items, int nh,
                                                                int hd, int hdp, int n_split) {
    const int item = blockIdx.x, head = blockIdx.y;
    const int token = items[item].x;
    attn_merge_splits(part_o, part_ml, out + ((size_t)token * nh + head) * hd, ((size_t)item * nh + head) * n_split, hd, hdp,
                      n_split);
}

// The same for items with splits of their own, which lie nh slots apart: one block per (row, head); firsts[r] =
// (row, index of the row's first item, its splits, 0).
__global__ __launch_bounds__(256) void attn_decode_merge_items_kernel(const float* __restrict__ part_o,
                                                                      const float* __restrict__ part_ml,
                                                                      bf16_t* __restrict__ out,
                                                                      const int4* __restrict__ items,
                                                                      const int4* __restrict__ firsts, int nh,
                                                                      int hd, int hdp) {
    const int head = blockIdx.y;
    const int4 row = firsts[blockIdx.x];
    const int first = row.y, n_split = row.z;
    if (n_split <= 1) return;
    attn_merge_splits(part_o, part_ml, out + ((size_t)row.x * nh + head) * hd, (size_t)first * nh + head, hd, hdp, n_split,
                      (size_t)nh);
}

extern "C" int fl_attn_decode_workspace(int n_items, int nh, int hd, int n_split, long* o_floats,
                                        long* ml_floats) {
    const int hdp = ceil_div(hd, 32) * 32;
    *o_floats = (long)n_items * nh * n_split * hdp;
    *ml_floats = (long)n_items * nh * n_split * 2;
    return 0;
}

static int attn_decode_launch(const char* who, const void* q, void* out, float* part_o, float* part_ml,
                              const void* cache_base, const int* items, int n_items, const int* block_table,
                              int max_blocks, int nh, int nkv, int hd, int page_size, int n_pages,
                              float scale, int window, int n_split, hipStream_t stream, bool own_splits = false,
                              const int* firsts = nullptr, int n_rows = 0) {
    FL_CHECK(n_items >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "%s: bad head counts %d/%d", who, nh, nkv);
    FL_CHECK(hd > 0 && hd <= 256 && hd % 8 == 0, "%s: head size %d must be a multiple of 8 up to 256", who, hd);
    FL_CHECK(page_size % 8 == 0, "%s: page size %d must be a multiple of 8", who, page_size);
    FL_CHECK(n_split >= 1 && n_split <= 256, "%s: %d splits", who, n_split);
    FL_CHECK(n_split == 1 || (part_o && part_ml), "%s: splits need a workspace", who);
    FL_CHECK(window >= 0, "%s: negative window", who);
    FL_CHECK((uintptr_t)items % 16 == 0, "%s: the items must be 16-byte aligned", who);
    if (n_items == 0) return 0;
    int ps_shift = -1;
    if ((page_size & (page_size - 1)) == 0)
        for (ps_shift = 0; (1 << ps_shift) < page_size; ++ps_shift) {}
    PagedCache c{(void*)cache_base, nkv, page_size, hd, n_pages};
    const int G = nh / nkv;
    const int q_tiles = ceil_div(G, 16);
    const int hdp = ceil_div(hd, 32) * 32;
    // a grid's slow index holds 65,535 places: longer lists of items take several launches
    for (int item_base = 0; item_base < n_items; item_base += 65535) {
        dim3 grid(nkv * q_tiles, min(n_items - item_base, 65535), own_splits ? 1 : n_split);
#define FL_DEC(HDP_)                                                                                  \
    attn_decode_kernel<HDP_><<<grid, 256, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, part_o, part_ml, c,       \
                                                       (const int4*)items, block_table, max_blocks, nh, scale,   \
                                                       window, n_split, q_tiles, ps_shift, item_base)
        switch (hdp) {
            case 32: FL_DEC(32); break;
            case 64: FL_DEC(64); break;
            case 96: FL_DEC(96); break;
            case 128: FL_DEC(128); break;
            case 160: FL_DEC(160); break;
            case 192: FL_DEC(192); break;
            case 224: FL_DEC(224); break;
            default: FL_DEC(256); break;
        }
#undef FL_DEC
        FL_LAUNCH_CHECK();
    }
    if (own_splits) {
        if (firsts && n_rows > 0) {              // (without: the caller knows that no row has more than one split)
            FL_CHECK((uintptr_t)firsts % 16 == 0, "%s: the rows' first items must be 16-byte aligned", who);
            dim3 mg(n_rows, nh);
            attn_decode_merge_items_kernel<<<mg, 256, 0, stream>>>(part_o, part_ml, (bf16_t*)out, (const int4*)items,
                                                                   (const int4*)firsts, nh, hd, hdp);
            FL_LAUNCH_CHECK();
        }
    } else if (n_split > 1) {
        dim3 mg(n_items, nh);
        attn_decode_merge_kernel<<<mg, 256, 0, stream>>>(
            part_o, part_ml, (bf16_t*)out, (const int4*)items, nh, hd, hdp, n_split);
        FL_LAUNCH_CHECK();
    }
    return 0;
}

extern "C" int fl_attn_decode(const void* q, void* out, float* part_o, float* part_ml,
                              const void* cache_base, const int* items, int n_items, const int* block_table,
                              int max_blocks, int nh, int nkv, int hd, int page_size, int n_pages,
                              float scale, int window, int n_split, hipStream_t stream) {
    return attn_decode_launch("attn_decode", q, out, part_o, part_ml, cache_base, items, n_items, block_table, max_blocks,
                              nh, nkv, hd, page_size, n_pages, scale, window, n_split, stream);
}
FL_RECORDABLE(fl_attn_decode)

// Items with splits of their own: items[i] = (row, position, request, split + 256 * splits), the splits of
// a row one after the other from split 0 on (up to 255), row < 0 for a place that is not used.  part_o
// holds n_items * nh * (head size rounded up to 32) floats, part_ml n_items * nh * 2.  firsts[r] = (row,
// index of the row's first item, its splits, 0) for the n_rows rows; without it no row has more
// than one split (a list with a place per row and no more) and the kernel that merges is left out.
extern "C" int fl_attn_decode_items(const void* q, void* out, float* part_o, float* part_ml, const void* cache_base,
                                    const int* items, int n_items, const int* block_table, int max_blocks, int nh,
                                    int nkv, int hd, int page_size, int n_pages, float scale, int window,
                                    const int* firsts, int n_rows, hipStream_t stream) {
    FL_CHECK(!firsts || (part_o && part_ml), "attn_decode_items: needs a workspace");
    return attn_decode_launch("attn_decode_items", q, out, part_o, part_ml, cache_base, items, n_items, block_table, max_blocks,
                              nh, nkv, hd, page_size, n_pages, scale, window, 1, stream, true, firsts, n_rows);
}
FL_RECORDABLE(fl_attn_decode_items)

// ---- the same without any allocation: the splits' partial results go to an array that is part of
// the library's image on every GPU.  `scratch` is a host-side stand-in for that array, not a device
// address; its address on the current device is asked for once per device and kept.
static __device__ __align__(256) float scratch[FL_ATTN_DECODE_STATIC_FLOATS];

#define FL_MAX_DEVICES 64
static float* g_scratch_ptr[FL_MAX_DEVICES];       // per device: where `scratch` lies there
static std::mutex g_scratch_mutex;

static int static_scratch(float** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    FL_CHECK(e == hipSuccess, "attn_decode_static: hipGetDevice failed: %s", hipGetErrorString(e));
    FL_CHECK(dev >= 0 && dev < FL_MAX_DEVICES, "attn_decode_static: device %d, at most %d are known", dev, FL_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        FL_CHECK(e == hipSuccess && p, "attn_decode_static: hipGetSymbolAddress failed on device %d: %s", dev,
                 hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

extern "C" long fl_attn_decode_static_capacity(void) { return (long)FL_ATTN_DECODE_STATIC_FLOATS; }

extern "C" int fl_attn_decode_static(const void* q, void* out, const void* cache_base, const int* items, int n_items,
                                     const int* block_table, int max_blocks, int nh, int nkv, int hd, int page_size,
                                     int n_pages, float scale, int window, int n_split, hipStream_t stream) {
    float* part_o = nullptr;
    float* part_ml = nullptr;
    if (n_split > 1 && n_items > 0) {
        FL_CHECK(nh > 0 && hd > 0 && hd <= 256 && n_split <= 256, "attn_decode_static: bad sizes (%d heads, head size %d, %d splits)",
                 nh, hd, n_split);
        const long hdp = ceil_div(hd, 32) * 32;
        const long slots = (long)n_items * nh * n_split;
        const long o_floats = (slots * hdp + 63) / 64 * 64;          // the pairs start 256-byte aligned
        const long need = o_floats + slots * 2;
        FL_CHECK(need <= (long)FL_ATTN_DECODE_STATIC_FLOATS,
                 "attn_decode_static: %d rows x %d heads x %d splits need %ld floats of scratch, the static array holds %ld "
                 "(use fl_attn_decode with a workspace, or fewer splits)",
                 n_items, nh, n_split, need, (long)FL_ATTN_DECODE_STATIC_FLOATS);
        float* base = nullptr;
        if (static_scratch(&base) != 0) return -1;
        part_o = base;
        part_ml = base + o_floats;
    }
    return attn_decode_launch("attn_decode_static", q, out, part_o, part_ml, cache_base, items, n_items, block_table,
                              max_blocks, nh, nkv, hd, page_size, n_pages, scale, window, n_split, stream);
}
FL_RECORDABLE(fl_attn_decode_static)

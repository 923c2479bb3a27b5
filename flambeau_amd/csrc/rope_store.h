// Epilogue shared by the matrix-product kernels: the product is the joined q/k/v projection with
// its rows in paired order (fl: rotary_paired_rows in kernels/packing.py), and instead of storing
// it the kernel rotates q and k (split-half rotation, crates/kernels-hip/src/kernels/
// rope_neox_partial_f16.cu:37-52), writes q to its buffer and k and v into the pages of the cache
// at the tokens' positions (crates/forward/src/core/composites/standard_attn.rs:485-500).
//
// The accumulators of v_mfma_f32_16x16x32_bf16 leave lane (token, g) with features 16 * group +
// 4 g .. + 3 of its token.  In paired order a group of 16 features of a rotated head is 8 dims
// (lanes g = 0, 1) and their 8 partners (g = 2, 3): the partner of a value sits in the lane 32
// further on (or back), one exchange per value.
#pragma once
#include "common.h"

struct RopeStore {
    const int* positions;     // [n]
    const int* tok_seq;       // [n] row of the block table
    const int* block_table;   // [requests][max_blocks]
    int max_blocks;
    const float2* cs;         // [n][rot / 2] cosine and sine of every (token, pair)
    bf16_t* q_out;            // [n][nh * hd]
    PagedCache cache;
    int nh;
    int rot;
    int write_cache;
};

struct TokenPlace {           // where a token's key and value go
    int page;                 // -1: nowhere (a padding row, a layer that reads another's cache)
    int row;
};

__device__ __forceinline__ TokenPlace rope_token_place(const RopeStore& rs, int tok) {
    TokenPlace tp;
    const int pos = rs.positions[tok];
    const int ps = rs.cache.page_size;
    int page = rs.write_cache ? rs.block_table[(size_t)rs.tok_seq[tok] * rs.max_blocks + pos / ps] : -1;
    if (page >= rs.cache.n_pages) page = -1;
    tp.page = page;
    tp.row = pos % ps;
    return tp;
}

// Where the tokens of COUNT lanes-rows go, all look-ups of one kind issued together (one wait for
// all of them instead of one per token).  toks beyond n_tokens are clamped and get page -1.
template <int COUNT>
__device__ __forceinline__ void rope_token_places(const RopeStore& rs, const int (&toks)[COUNT], int n_tokens,
                                                  TokenPlace (&places)[COUNT]) {
    const int ps = rs.cache.page_size;
    int pos[COUNT], seq[COUNT];
#pragma unroll
    for (int i = 0; i < COUNT; ++i) {
        const int t = min(toks[i], n_tokens - 1);
        pos[i] = rs.positions[t];
        seq[i] = rs.write_cache ? rs.tok_seq[t] : 0;
    }
#pragma unroll
    for (int i = 0; i < COUNT; ++i) {
        int page = rs.write_cache ? rs.block_table[(size_t)seq[i] * rs.max_blocks + pos[i] / ps] : -1;
        if (page >= rs.cache.n_pages || toks[i] >= n_tokens) page = -1;
        places[i].page = page;
        places[i].row = pos[i] % ps;
    }
}

struct RopeAngles {           // cosine and sine of a lane's four pairs: (c0, s0, c1, s1), (c2, s2, c3, s3)
    float4 a, b;
};

// The angles of the four pairs of lane (token, g) at features f0 .. f0 + 3.  The address is clamped
// into the token's row, so this may be called (and its result ignored) for features that are not
// rotated; tok must be a valid token and rs.rot at least 8.
__device__ __forceinline__ RopeAngles rope_angles(const RopeStore& rs, int tok, int f0, int g) {
    const int hd = rs.cache.head_dim;
    const int within = f0 % hd, half = rs.rot >> 1;
    const int pair0 = min(8 * (within >> 4) + 4 * (g & 1), half - 4);
    const float4* t = (const float4*)(rs.cs + (size_t)tok * half + pair0);
    RopeAngles an;
    an.a = t[0];
    an.b = t[1];
    return an;
}

// v: this lane's four features f0 .. f0 + 3 (f0 = 16 * group + 4 g, in paired order) of token tok;
// every lane of the wave calls this together (the exchange needs all of them), `live` says whether
// this lane's token and features exist.  PRELOADED: an holds rope_angles of this lane (else they
// are read here, where the lane rotates).
template <bool PRELOADED = false>
__device__ __forceinline__ void rope_store4(const RopeStore& rs, int tok, const TokenPlace& tp, int f0, int g,
                                            f32x4 v, bool live, RopeAngles an = RopeAngles{}) {
    const int hd = rs.cache.head_dim, nkv = rs.cache.n_kv_heads;
    f32x4 partner;
#pragma unroll
    for (int r = 0; r < 4; ++r) partner[r] = __shfl_xor(v[r], 32, 64);
    if (!live) return;
    const int head = f0 / hd, within = f0 - head * hd;
    const bool is_v = head >= rs.nh + nkv;
    int dim = within;
    f32x4 o = v;
    if (!is_v && within < rs.rot) {
        const int half = rs.rot >> 1;
        const int pair0 = 8 * (within >> 4) + 4 * (g & 1);          // first of this lane's four pairs
        dim = g < 2 ? pair0 : half + pair0;
        if (!PRELOADED) an = rope_angles(rs, tok, f0, g);
        const float4 cs01 = an.a, cs23 = an.b;
        const float c[4] = {cs01.x, cs01.z, cs23.x, cs23.z}, s[4] = {cs01.y, cs01.w, cs23.y, cs23.w};
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = g < 2 ? v[r] * c[r] - partner[r] * s[r] : v[r] * c[r] + partner[r] * s[r];
    }
    const bf16x4 ob = {(bf16_t)o[0], (bf16_t)o[1], (bf16_t)o[2], (bf16_t)o[3]};
    if (head < rs.nh) {
        *(bf16x4*)(rs.q_out + ((size_t)tok * rs.nh + head) * hd + dim) = ob;
    } else if (tp.page >= 0) {
        bf16_t* base = (bf16_t*)rs.cache.base;
        if (!is_v) {
            *(bf16x4*)(base + cache_k_offset(rs.cache, tp.page, head - rs.nh, tp.row, dim)) = ob;
        } else {
            bf16_t* p = base + cache_v_offset(rs.cache, tp.page, head - rs.nh - nkv, tp.row, dim);
#pragma unroll
            for (int r = 0; r < 4; ++r) p[(size_t)r * rs.cache.page_size] = ob[r];
        }
    }
}

// Plain kernels: one straightforward kernel for every op of the decoder, templated on
// the storage type.  The 32-bit path of the engine runs on these alone (float storage,
// float arithmetic, precise expf/sinf/cosf/powf, a fixed reduction order per output
// element that does not depend on the batch), and every tuned bf16 kernel is tested
// against its plain kernel.
//
// Formulas follow the reference's kernels:
//   rmsnorm   crates/kernels-hip/src/kernels/rmsnorm_f16.cu:40-85
//   rotation  crates/kernels-hip/src/kernels/rope_neox_partial_f16.cu:37-52
//   attention crates/kernels-hip/src/kernels/attention_prefill_f16.cu:50-133
//   paging    crates/kernels-hip/src/kernels/attention_decode_f16_paged.cu:110-115
//   SiLU gate crates/kernels-hip/src/kernels/swiglu_f32_to_f16.cu:21-23
#include "common.h"
#include "api.h"
#include "recordable.h"

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ __launch_bounds__(256) void embed_kernel(const T* __restrict__ table,
                                                    const int* __restrict__ tokens,
                                                    float* __restrict__ out, int H, int V) {
    const int r = blockIdx.x;
    int tok = tokens[r];
    if (tok < 0 || tok >= V) tok = 0;  // the host rejects such ids before the launch
    const T* src = table + (size_t)tok * H;
    float* dst = out + (size_t)r * H;
    if (H % 4 == 0 && ((uintptr_t)table % 16 == 0) && ((uintptr_t)out % 16 == 0)) {       // four values per load
        for (int i = 4 * threadIdx.x; i < H; i += 4 * blockDim.x) {
            f32x4 v;
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = to_f32(src[i + u]);
            *(f32x4*)(dst + i) = v;
        }
    } else {
        for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = to_f32(src[i]);
    }
}

extern "C" int fl_embed(const void* table, int dtype, const int* tokens, float* out, int n, int H,
                        int V, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && V > 0, "embed: bad sizes n=%d H=%d V=%d", n, H, V);
    if (n == 0) return 0;
    if (dtype == FL_F32)
        embed_kernel<float><<<n, 256, 0, stream>>>((const float*)table, tokens, out, H, V);
    else if (dtype == FL_BF16)
        embed_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)table, tokens, out, H, V);
    else
        FL_CHECK(false, "embed: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_embed)

// ------------------------------------------------------------------ RMSNorm
// out[r,:] = v * w * rsqrt(mean(v^2) + eps), v = x[src,:] (+ delta[src,:]); src = rows ? rows[r] : r.
// With resid_out the sum v is stored back (the residual stream, 32-bit).
template <typename TOut>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x,
                                                      const float* __restrict__ delta,
                                                      float* resid_out, const int* __restrict__ rows,
                                                      const float* __restrict__ w,
                                                      TOut* __restrict__ out, int H, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    const float* xr = x + (size_t)src * H;
    const float* dr = delta ? delta + (size_t)src * H : nullptr;
    float* ro = resid_out ? resid_out + (size_t)src * H : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
        float v = xr[i];
        if (dr) v += dr[i];
        if (ro) ro[i] = v;
        ss += v * v;
    }
    const float total = block_sum<4>(ss, red);
    const float inv = 1.0f / sqrtf(total / (float)H + eps);
    TOut* orow = out + (size_t)r * H;
    for (int i = threadIdx.x; i < H; i += 256) {
        float v = ro ? ro[i] : (dr ? xr[i] + dr[i] : xr[i]);
        orow[i] = from_f32<TOut>(v * w[i] * inv);
    }
}

// The same with 16-byte accesses and the row kept in registers between the two passes
// (H <= 1024 * VPT, H a multiple of 4): every load of a thread is issued before the first use.
template <typename TOut, int VPT>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(const float* __restrict__ x,
                                                          const float* __restrict__ delta,
                                                          float* resid_out, const int* __restrict__ rows,
                                                          const float* __restrict__ w,
                                                          TOut* __restrict__ out, int H, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    const f32x4* xr = (const f32x4*)(x + (size_t)src * H);
    const f32x4* dr = delta ? (const f32x4*)(delta + (size_t)src * H) : nullptr;
    const int n4 = H >> 2;
    f32x4 v[VPT], d[VPT], g[VPT];
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
        const int i = threadIdx.x + 256 * u;
        v[u] = i < n4 ? xr[i] : (f32x4){0.f, 0.f, 0.f, 0.f};
        d[u] = (dr && i < n4) ? dr[i] : (f32x4){0.f, 0.f, 0.f, 0.f};
        g[u] = i < n4 ? ((const f32x4*)w)[i] : (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
        v[u] += d[u];
        ss += v[u][0] * v[u][0] + v[u][1] * v[u][1] + v[u][2] * v[u][2] + v[u][3] * v[u][3];
    }
    if (resid_out) {
        f32x4* ro = (f32x4*)(resid_out + (size_t)src * H);
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const int i = threadIdx.x + 256 * u;
            if (i < n4) ro[i] = v[u];
        }
    }
    const float total = block_sum<4>(ss, red);
    const float inv = 1.0f / sqrtf(total / (float)H + eps);
    TOut* orow = out + (size_t)r * H;
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
        const int i = threadIdx.x + 256 * u;
        if (i < n4) {
            const f32x4 y = v[u] * g[u] * inv;
            if constexpr (sizeof(TOut) == 4) {
                *(f32x4*)(orow + 4 * i) = y;
            } else {
                bf16x4 o = {(bf16_t)y[0], (bf16_t)y[1], (bf16_t)y[2], (bf16_t)y[3]};
                *(bf16x4*)(orow + 4 * i) = o;
            }
        }
    }
}

template <typename TOut>
static void launch_rmsnorm(const float* x, const float* delta, float* resid_out, const int* rows, const float* w,
                           TOut* out, int n_rows, int H, float eps, hipStream_t stream) {
    const bool aligned = H % 4 == 0 && ((uintptr_t)x % 16 == 0) && (!delta || (uintptr_t)delta % 16 == 0) &&
                         ((uintptr_t)w % 16 == 0) && ((uintptr_t)out % 8 == 0);
    if (aligned && H <= 4096)
        rmsnorm_vec_kernel<TOut, 4><<<n_rows, 256, 0, stream>>>(x, delta, resid_out, rows, w, out, H, eps);
    else if (aligned && H <= 8192)
        rmsnorm_vec_kernel<TOut, 8><<<n_rows, 256, 0, stream>>>(x, delta, resid_out, rows, w, out, H, eps);
    else if (aligned && H <= 16384)
        rmsnorm_vec_kernel<TOut, 16><<<n_rows, 256, 0, stream>>>(x, delta, resid_out, rows, w, out, H, eps);
    else
        rmsnorm_kernel<TOut><<<n_rows, 256, 0, stream>>>(x, delta, resid_out, rows, w, out, H, eps);
}

extern "C" int fl_rmsnorm(const float* x, const float* delta, float* resid_out, const int* rows,
                          const float* w, void* out, int out_dtype, int n_rows, int H, float eps,
                          hipStream_t stream) {
    FL_CHECK(n_rows >= 0 && H > 0, "rmsnorm: bad sizes rows=%d H=%d", n_rows, H);
    FL_CHECK(!(rows && resid_out), "rmsnorm: gathered rows cannot be stored back");
    if (n_rows == 0) return 0;
    if (out_dtype == FL_F32)
        launch_rmsnorm<float>(x, delta, resid_out, rows, w, (float*)out, n_rows, H, eps, stream);
    else if (out_dtype == FL_BF16)
        launch_rmsnorm<bf16_t>(x, delta, resid_out, rows, w, (bf16_t*)out, n_rows, H, eps, stream);
    else
        FL_CHECK(false, "rmsnorm: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_rmsnorm)

// ------------------------------------------------------------------ residual add
__global__ __launch_bounds__(256) void add_kernel(float* __restrict__ x, const float* __restrict__ d, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) x[i] += d[i];
}

extern "C" int fl_add_inplace(float* x, const float* delta, long n, hipStream_t stream) {
    FL_CHECK(n >= 0, "add: bad size");
    if (n == 0) return 0;
    add_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, delta, (size_t)n);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_add_inplace)

// ------------------------------------------------------------------ plain GEMM
// out[m, n] = sum_k x[m,k] * w[n,k]; 64x64 tile per block, 4x4 per thread, k in steps of 16.
// Each output element is summed in a fixed order (rising k): the result of a row does not depend on
// how many rows the call has.  The 16 products of a step are added in a chain of their own and the
// steps' sums with a compensated (Kahan) addition, still all in float: over K = 14336 a single
// chain loses about sqrt(K) roundings, which is what showed in the 32-bit path's logits (6.6e-5 at
// 7B layer sizes against a float64 reference, against a bound of 1e-4).
template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const TIn* __restrict__ x,
                                                         const TIn* __restrict__ w,
                                                         TOut* __restrict__ out, int M, int N, int K,
                                                         int ldo) {
    __shared__ float xs[16][68];
    __shared__ float ws[16][68];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    float acc[4][4], lost[4][4];              // the running sums and what their roundings have lost so far
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) { acc[i][j] = 0.f; lost[i][j] = 0.f; }
    for (int k0 = 0; k0 < K; k0 += 16) {
        for (int e = threadIdx.x; e < 1024; e += 256) {
            const int row = e >> 4, kk = e & 15;
            const int gk = k0 + kk;
            const int gm = m0 + row, gn = n0 + row;
            xs[kk][row] = (gm < M && gk < K) ? to_f32(x[(size_t)gm * K + gk]) : 0.f;
            ws[kk][row] = (gn < N && gk < K) ? to_f32(w[(size_t)gn * K + gk]) : 0.f;
        }
        __syncthreads();
        float part[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) part[i][j] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) part[i][j] = fmaf(a[i], b[j], part[i][j]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float y = part[i][j] - lost[i][j];
                const float t = acc[i][j] + y;
                lost[i][j] = (t - acc[i][j]) - y;
                acc[i][j] = t;
            }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + ty * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn < N) out[(size_t)gm * ldo + gn] = from_f32<TOut>(acc[i][j]);
        }
    }
}

extern "C" int fl_gemm_plain(const void* x, const void* w, void* out, int in_dtype, int out_dtype,
                             int M, int N, int K, hipStream_t stream) {
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    dim3 grid(ceil_div(N, 64), ceil_div(M, 64));
    if (in_dtype == FL_F32 && out_dtype == FL_F32)
        gemm_plain_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)x, (const float*)w, (float*)out, M, N, K, N);
    else if (in_dtype == FL_BF16 && out_dtype == FL_F32)
        gemm_plain_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, (float*)out, M, N, K, N);
    else if (in_dtype == FL_BF16 && out_dtype == FL_BF16)
        gemm_plain_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)out, M, N, K, N);
    else
        FL_CHECK(false, "gemm: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_plain)

// ------------------------------------------------------------------ rotation + cache write
// cos and sin of every (token, pair) of a step: cs[token][i] = (cos, sin)(position * theta^(-2 i / rot)).
// Made once per step, read by every layer's rotation.
__global__ __launch_bounds__(64) void rope_table_kernel(const int* __restrict__ positions, int rot, float theta,
                                                        float2* __restrict__ cs) {
    const int token = blockIdx.x, half = rot >> 1;
    // The angle is formed in double: in float a position of some thousands times a frequency near 1
    // is already off by 1e-4 rad, which is the largest error left in the 32-bit path's logits; the
    // table itself is float.
    const double pos = (double)positions[token];
    for (int i = threadIdx.x; i < half; i += 64) {
        const double inv_freq = pow((double)theta, -2.0 * (double)i / (double)rot);
        const double angle = pos * inv_freq;
        cs[(size_t)token * half + i] = make_float2((float)cos(angle), (float)sin(angle));
    }
}

// The same from a ladder of frequencies of the caller's own (inv_freq[rot / 2], double): cs[token][i] =
// magnitude * (cos, sin)(position * inv_freq[i]).  Scaled and interpolated ladders are such tables.
__global__ __launch_bounds__(64) void rope_table_ladder_kernel(const int* __restrict__ positions, int rot,
                                                               const double* __restrict__ inv_freq, float magnitude,
                                                               float2* __restrict__ cs) {
    const int token = blockIdx.x, half = rot >> 1;
    const double pos = (double)positions[token];
    for (int i = threadIdx.x; i < half; i += 64) {
        const double angle = pos * inv_freq[i];
        cs[(size_t)token * half + i] = make_float2((float)(magnitude * cos(angle)), (float)(magnitude * sin(angle)));
    }
}

extern "C" int fl_rope_table_ladder(const int* positions, int n, int rot, const double* inv_freq, float magnitude,
                                    float* cs, hipStream_t stream) {
    FL_CHECK(n >= 0 && rot > 0 && rot % 2 == 0 && inv_freq, "rope_table_ladder: %d rotated dims", rot);
    FL_CHECK((uintptr_t)cs % 8 == 0 && (uintptr_t)inv_freq % 8 == 0, "rope_table_ladder: the tables must be 8-byte aligned");
    if (n == 0) return 0;
    rope_table_ladder_kernel<<<n, 64, 0, stream>>>(positions, rot, inv_freq, magnitude, (float2*)cs);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_rope_table_ladder)

extern "C" int fl_rope_table(const int* positions, int n, int rot, float theta, float* cs, hipStream_t stream) {
    FL_CHECK(n >= 0 && rot > 0 && rot % 2 == 0, "rope_table: %d rotated dims", rot);
    FL_CHECK((uintptr_t)cs % 8 == 0, "rope_table: the table must be 8-byte aligned");
    if (n == 0) return 0;
    rope_table_kernel<<<n, 64, 0, stream>>>(positions, rot, theta, (float2*)cs);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_rope_table)

// One block per (token, head) over the fused projection row [q heads | k heads | v heads].
// Q heads: rotated, written to q_out.  K heads: rotated, written to the cache at the token's
// position.  V heads: written to the cache as they are.  rot = rotated dims (pairs (i, i+rot/2));
// rot = 0 means no rotation at all (another position encoding has run, or none).  cs: the step's
// table of cosines and sines, or null (then they are computed here).  paired: the rotated dims of
// a q or k head arrive in the order of fl_rotary_paired_rows (8 dims, their 8 partners, the next
// 8 dims, ...), as the projection's fused kernels want them.
template <typename TIn, typename T>
__global__ __launch_bounds__(64) void rope_kv_write_kernel(
    const TIn* __restrict__ qkv, int ld, const int* __restrict__ positions,
    const int* __restrict__ tok_seq, const int* __restrict__ block_table, int max_blocks,
    T* __restrict__ q_out, PagedCache cache, int nh, int hd, int rot, float theta, int write_cache,
    const float2* __restrict__ cs, int paired, int n_parts, size_t part_stride) {
    const int token = blockIdx.x;
    const int head = blockIdx.y;
    const int nkv = cache.n_kv_heads;
    const int pos = positions[token];
    const TIn* src = qkv + (size_t)token * ld + (size_t)head * hd;
    // the projection may arrive as n_parts partial sums (a product that split K): added here, in rising order
    auto value = [&](int i) {
        float v = to_f32(src[i]);
        for (int part = 1; part < n_parts; ++part) v += to_f32(src[(size_t)part * part_stride + i]);
        return v;
    };
    T* dst;
    size_t stride = 1;      // distance between consecutive head dims at the destination
    bool rotate;
    if (head < nh) {
        dst = q_out + ((size_t)token * nh + head) * hd;
        rotate = true;
    } else {
        if (!write_cache) return;
        const int kvh = (head - nh) % nkv;
        const int is_v = (head - nh) / nkv;
        const int page = block_table[(size_t)tok_seq[token] * max_blocks + pos / cache.page_size];
        if (page < 0 || page >= cache.n_pages) return;  // padding rows of a fixed-size batch
        const int row = pos % cache.page_size;
        if (is_v) {
            dst = (T*)cache.base + cache_v_offset(cache, page, kvh, row, 0);
            stride = cache.page_size;
        } else {
            dst = (T*)cache.base + cache_k_offset(cache, page, kvh, row, 0);
        }
        rotate = !is_v;
    }
    const int half = rot >> 1;
    if (rotate && rot > 0) {
        for (int i = threadIdx.x; i < half; i += 64) {
            float c, s;
            if (cs) {
                const float2 v = cs[(size_t)token * half + i];
                c = v.x; s = v.y;
            } else {
                // (in double, as in rope_table_kernel)
                const double angle = (double)pos * pow((double)theta, -2.0 * (double)i / (double)rot);
                c = (float)cos(angle); s = (float)sin(angle);
            }
            const int at = paired ? 16 * (i >> 3) + (i & 7) : i;
            const float x0 = value(at), x1 = value(paired ? at + 8 : i + half);
            dst[i] = from_f32<T>(x0 * c - x1 * s);
            dst[i + half] = from_f32<T>(x0 * s + x1 * c);
        }
        for (int i = rot + threadIdx.x; i < hd; i += 64) dst[i] = from_f32<T>(value(i));
    } else {
        for (int i = threadIdx.x; i < hd; i += 64) dst[(size_t)i * stride] = from_f32<T>(value(i));
    }
}

extern "C" int fl_rope_kv_write(const void* qkv, int in_dtype, int ld, const int* positions,
                                const int* tok_seq, const int* block_table, int max_blocks,
                                void* q_out, void* cache_base, int dtype, int n, int nh, int nkv,
                                int hd, int page_size, int n_pages, int rot, float theta,
                                int write_cache, const float* cs, int paired, int n_parts, long part_stride,
                                hipStream_t stream) {
    FL_CHECK(n >= 0 && nh > 0 && nkv > 0 && hd > 0 && page_size > 0, "rope_kv_write: bad sizes");
    FL_CHECK(n_parts >= 1 && (n_parts == 1 || part_stride >= (long)n * ld), "rope_kv_write: %d parts %ld values apart", n_parts, part_stride);
    FL_CHECK(rot >= 0 && rot <= hd && rot % 2 == 0, "rope_kv_write: rotated dims %d of head %d", rot, hd);
    FL_CHECK(ld >= (nh + 2 * nkv) * hd, "rope_kv_write: row stride %d too small", ld);
    FL_CHECK(!paired || (rot % 16 == 0 && hd % 16 == 0), "rope_kv_write: the paired order needs rotated dims and head size in steps of 16 (%d of %d)", rot, hd);
    if (n == 0) return 0;
    PagedCache c{cache_base, nkv, page_size, hd, n_pages};
    dim3 grid(n, nh + 2 * nkv);
#define FL_ROPE(TIN, TT)                                                                       \
    rope_kv_write_kernel<TIN, TT><<<grid, 64, 0, stream>>>((const TIN*)qkv, ld, positions, tok_seq, \
                                                           block_table, max_blocks, (TT*)q_out, c, \
                                                           nh, hd, rot, theta, write_cache, (const float2*)cs, paired, n_parts, (size_t)part_stride)
    if (in_dtype == FL_F32 && dtype == FL_F32) FL_ROPE(float, float);
    else if (in_dtype == FL_F32 && dtype == FL_BF16) FL_ROPE(float, bf16_t);
    else if (in_dtype == FL_BF16 && dtype == FL_BF16) FL_ROPE(bf16_t, bf16_t);
    else FL_CHECK(false, "rope_kv_write: unsupported dtypes in=%d store=%d", in_dtype, dtype);
#undef FL_ROPE
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_rope_kv_write)

// ------------------------------------------------------------------ plain attention over the cache
// One block per (token, query head).  The query at position p sees the keys
// t in [max(0, p - window + 1), p] of its own request (window 0: from 0), all read from the
// paged cache (this step's keys were written before).  Four waves take every fourth key with
// an online softmax each; lanes own the head dims; the four states are merged at the end.
#define FL_PLAIN_MAX_HD 256
template <typename T>
__global__ __launch_bounds__(256) void attn_plain_kernel(
    const T* __restrict__ q, T* __restrict__ out, PagedCache cache,
    const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks, int nh, float scale, int window) {
    __shared__ float s_m[4], s_l[4];
    __shared__ float s_acc[4][FL_PLAIN_MAX_HD];
    const int token = blockIdx.x, head = blockIdx.y;
    const int hd = cache.head_dim;
    const int kvh = head / (nh / cache.n_kv_heads);
    const int p = positions[token];
    const int* table = block_table + (size_t)tok_seq[token] * max_blocks;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const T* qr = q + ((size_t)token * nh + head) * hd;
    float qv[4], acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int d = lane + 64 * j;
        qv[j] = d < hd ? to_f32(qr[d]) : 0.f;
        acc[j] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    for (int t = lo + wave; t <= p; t += 4) {
        const int page = table[t / cache.page_size];
        if (page < 0 || page >= cache.n_pages) continue;
        const int row = t % cache.page_size;
        const T* kr = (const T*)cache.base + cache_k_offset(cache, page, kvh, row, 0);
        const T* vr = (const T*)cache.base + cache_v_offset(cache, page, kvh, row, 0);
        const int vs = cache.page_size;
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = lane + 64 * j;
            if (d < hd) part = fmaf(qv[j], to_f32(kr[d]), part);
        }
        const float s = wave_sum(part) * scale;
        const float m_new = fmaxf(m, s);
        const float corr = expf(m - m_new);
        const float pe = expf(s - m_new);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = lane + 64 * j;
            if (d < hd) acc[j] = acc[j] * corr + pe * to_f32(vr[(size_t)d * vs]);
        }
        l = l * corr + pe;
        m = m_new;
    }
    if (lane == 0) { s_m[wave] = m; s_l[wave] = l; }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int d = lane + 64 * j;
        if (d < hd) s_acc[wave][d] = acc[j];
    }
    __syncthreads();
    if (wave == 0) {
        float mm = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
        float f[4], ll = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            f[w] = (s_m[w] == -INFINITY) ? 0.f : expf(s_m[w] - mm);
            ll += s_l[w] * f[w];
        }
        T* orow = out + ((size_t)token * nh + head) * hd;
        const float inv = ll > 0.f ? 1.0f / ll : 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = lane + 64 * j;
            if (d < hd) {
                float o = 0.f;
#pragma unroll
                for (int w = 0; w < 4; ++w) o += s_acc[w][d] * f[w];
                orow[d] = from_f32<T>(o * inv);
            }
        }
    }
}

// The largest head size any attention kernel of the library takes (the plain kernel keeps a head in LDS).
extern "C" int fl_attn_max_head_dim(void) { return FL_PLAIN_MAX_HD; }

extern "C" int fl_attn_plain(const void* q, void* out, const void* cache_base, int dtype,
                             const int* positions, const int* tok_seq, const int* block_table,
                             int max_blocks, int n, int nh, int nkv, int hd, int page_size,
                             int n_pages, float scale, int window, hipStream_t stream) {
    FL_CHECK(n >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attn: bad head counts %d/%d", nh, nkv);
    FL_CHECK(hd > 0 && hd <= FL_PLAIN_MAX_HD, "attn: head size %d not in 1..%d", hd, FL_PLAIN_MAX_HD);
    FL_CHECK(window >= 0, "attn: negative window");
    if (n == 0) return 0;
    PagedCache c{(void*)cache_base, nkv, page_size, hd, n_pages};
    dim3 grid(n, nh);
    if (dtype == FL_F32)
        attn_plain_kernel<float><<<grid, 256, 0, stream>>>((const float*)q, (float*)out, c, positions, tok_seq, block_table, max_blocks, nh, scale, window);
    else if (dtype == FL_BF16)
        attn_plain_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, c, positions, tok_seq, block_table, max_blocks, nh, scale, window);
    else
        FL_CHECK(false, "attn: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_attn_plain)

// ------------------------------------------------------------------ SiLU gate
// out[r, i] = silu(gu[r, i]) * gu[r, I + i], silu(g) = g / (1 + exp(-g)), all in float.
template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void silu_mul_kernel(const TIn* __restrict__ gu, TOut* __restrict__ out,
                                                       int I, int ld) {
    const int r = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= I) return;
    const float g = to_f32(gu[(size_t)r * ld + i]);
    const float u = to_f32(gu[(size_t)r * ld + I + i]);
    out[(size_t)r * I + i] = from_f32<TOut>(g / (1.0f + expf(-g)) * u);
}

extern "C" int fl_silu_mul(const void* gu, int in_dtype, void* out, int out_dtype, int n, int I,
                           hipStream_t stream) {
    FL_CHECK(n >= 0 && I > 0, "silu_mul: bad sizes");
    if (n == 0) return 0;
    dim3 grid(ceil_div(I, 256), n);
    if (in_dtype == FL_F32 && out_dtype == FL_F32)
        silu_mul_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)gu, (float*)out, I, 2 * I);
    else if (in_dtype == FL_F32 && out_dtype == FL_BF16)
        silu_mul_kernel<float, bf16_t><<<grid, 256, 0, stream>>>((const float*)gu, (bf16_t*)out, I, 2 * I);
    else if (in_dtype == FL_BF16 && out_dtype == FL_BF16)
        silu_mul_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, 2 * I);
    else
        FL_CHECK(false, "silu_mul: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_silu_mul)

// ------------------------------------------------------------------ sampling
// The better of two (value, index) candidates: the larger value, the smaller index among equals.
__device__ __forceinline__ void take_better(float& v, int& i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

// Best candidate of a block of NW waves, in every thread.
template <int NW>
__device__ __forceinline__ void block_argmax(float& v, int& i, float* sv, int* si) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) take_better(v, i, __shfl_xor(v, off, 64), __shfl_xor(i, off, 64));
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { sv[wave] = v; si[wave] = i; }
    __syncthreads();
    v = sv[0]; i = si[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) take_better(v, i, sv[w], si[w]);
    __syncthreads();
}

// argmax per row; the first maximum wins (crates/runtime/src/sampling.rs:486-496).  One block of
// 1024 threads per row; a thread fetches eight values 1024 apart before it compares them, so a
// row of 32k values costs one round trip to memory, not a hundred.
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float* row = logits + (size_t)blockIdx.x * V;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int base = 0; base < V; base += 8 * 1024) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = base + u * 1024 + threadIdx.x;
            v[u] = i < V ? row[i] : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (v[u] > best) { best = v[u]; bi = base + u * 1024 + threadIdx.x; }      // rising index: the first maximum stays
    }
    block_argmax<16>(best, bi, sv, si);
    if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

// Temperature draw per row: p_i = exp((l_i - max) * inv_t); the token is the first index at
// which the running sum of p in index order reaches u * sum(p) (inverse CDF; the same walk as
// crates/runtime/src/sampling.rs:735-745 without filters).  inv_t <= 0 means argmax.
// Thread t owns the contiguous chunk [t*C, (t+1)*C) so that the walk keeps index order.
__global__ __launch_bounds__(256) void sample_kernel(const float* __restrict__ logits,
                                                     const float* __restrict__ inv_temp,
                                                     const float* __restrict__ uniform,
                                                     int* __restrict__ out, int V) {
    __shared__ float chunk_sum[256];
    __shared__ float sv[4];
    __shared__ int si[4];
    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * V;
    const float it = inv_temp[r];
    // the maximum (and its first index) with coalesced loads, eight in flight per thread
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int base = 0; base < V; base += 8 * 256) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = base + u * 256 + threadIdx.x;
            v[u] = i < V ? row[i] : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (v[u] > best) { best = v[u]; bi = base + u * 256 + threadIdx.x; }
    }
    block_argmax<4>(best, bi, sv, si);
    const float mx = best;
    const int amax = bi == 0x7fffffff ? 0 : bi;
    // for the walk in index order thread t owns the contiguous chunk [t C, (t + 1) C)
    const int C = (V + 255) / 256;
    const int lo = threadIdx.x * C, hi = min(V, lo + C);
    if (!(it > 0.f)) {
        if (threadIdx.x == 0) out[r] = amax;
        return;
    }
    float part = 0.f;
    {
        int i = lo;
        for (; i + 8 <= hi; i += 8) {                  // eight loads in flight; the sum keeps index order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = row[i + u];
#pragma unroll
            for (int u = 0; u < 8; ++u) part += expf((v[u] - mx) * it);
        }
        for (; i < hi; ++i) part += expf((row[i] - mx) * it);
    }
    chunk_sum[threadIdx.x] = part;
    __syncthreads();
    if (threadIdx.x == 0) {
        // the total is the chunks' sums added in index order, as the walk below takes them away again:
        // the target can never outlast the last chunk by rounding, and nothing depends on a tree's shape
        float total = 0.f;
        for (int c = 0; c < 256; ++c) total += chunk_sum[c];
        float target = uniform[r] * total;
        int chosen = -1;
        int c = 0;
        for (; c < 256; ++c) {
            if (target <= chunk_sum[c] && chunk_sum[c] > 0.f) break;
            target -= chunk_sum[c];
        }
        if (c < 256) {
            const int clo = c * C, chi = min(V, clo + C);
            for (int i = clo; i < chi; ++i) {
                target -= expf((row[i] - mx) * it);
                if (target <= 0.f) { chosen = i; break; }
            }
            if (chosen < 0) chosen = chi - 1;
        } else {
            chosen = amax;
        }
        out[r] = chosen;
    }
}

// Token ids that are still on the device: tokens[i] = ids[src[i]] where src[i] >= 0 (the token a
// request drew in the step before, fed back without a round trip through the host).
__global__ __launch_bounds__(256) void feed_tokens_kernel(int* __restrict__ tokens, const int* __restrict__ ids,
                                                          const int* __restrict__ src, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n && src[i] >= 0) tokens[i] = ids[src[i]];
}

extern "C" int fl_feed_tokens(int* tokens, const int* ids, const int* src, int n, hipStream_t stream) {
    FL_CHECK(n >= 0, "feed_tokens: bad size");
    if (n == 0) return 0;
    feed_tokens_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(tokens, ids, src, n);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_feed_tokens)

extern "C" int fl_argmax(const float* logits, int* out, int rows, int V, hipStream_t stream) {
    FL_CHECK(rows >= 0 && V > 0, "argmax: bad sizes");
    if (rows == 0) return 0;
    argmax_kernel<<<rows, 1024, 0, stream>>>(logits, out, V);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_argmax)

extern "C" int fl_sample(const float* logits, const float* inv_temp, const float* uniform, int* out,
                         int rows, int V, hipStream_t stream) {
    FL_CHECK(rows >= 0 && V > 0, "sample: bad sizes");
    if (rows == 0) return 0;
    sample_kernel<<<rows, 256, 0, stream>>>(logits, inv_temp, uniform, out, V);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_sample)

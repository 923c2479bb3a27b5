// Tiled bf16 matrix product for prompt portions: out[m, n] = sum_k x[m, k] w[n, k] with many
// rows m, on the matrix cores (v_mfma_f32_16x16x32_bf16, float accumulation).
//
//  * w arrives packed (kernels/packing.py): a tile of 16 features x 32 k is 1 KB in lane order,
//    so the block's slice of w is copied to LDS as it lies in memory, and a wave reads an
//    operand tile from LDS with one ds_read_b128 per lane at consecutive addresses (no bank
//    conflicts, no transposition);
//  * x is row-major; on its way into LDS every 16-byte chunk is put where the same tile layout
//    wants it, so the x operand is read the same way;
//  * a block of four waves (2 x 2) computes BM x BN = 128 x 128 outputs, each wave 64 x 64
//    (16 accumulator tiles); K is walked in slices of 64 with two LDS buffers: the next slice
//    is fetched from memory into registers while the current one is multiplied;
//  * the w tile is the A operand and the x tile the B operand: C[feature][token] leaves each
//    lane with four consecutive features of one token, one 16-byte store;
//  * with few rows and a narrow matrix the grid would not fill the chip: K is then split over
//    blockIdx.z, the parts are written as float partial sums and a second kernel adds them in
//    a fixed order.
//
// The reference's nearest kernel multiplies a 64 x 8 tile per 64-thread block without matrix
// cores (crates/kernels-hip/src/kernels/mmq_f16_tile.cu:33-107).
#include "common.h"
#include "api.h"

#define TG_BM 128
#define TG_BN 128
#define TG_BK 64
#define TG_TILE 512                      // values in a 16 x 32 tile

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

template <typename TOut>
__device__ __forceinline__ void tg_store4(TOut* p, f32x4 v);
template <> __device__ __forceinline__ void tg_store4<float>(float* p, f32x4 v) { *(f32x4*)p = v; }
template <> __device__ __forceinline__ void tg_store4<bf16_t>(bf16_t* p, f32x4 v) {
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *(bf16x4*)p = o;
}

// SWIGLU: w holds gate and up rows interleaved in fours; the block writes silu(gate) * up,
// out_cols <= N / 2 values per token (never together with a split of K).
template <typename TOut, bool SWIGLU>
__global__ __launch_bounds__(256, 2) void gemm_tiled_kernel(const bf16_t* __restrict__ x,
                                                            const bf16_t* __restrict__ wp,
                                                            TOut* __restrict__ out, int M, int N, int K,
                                                            int n_steps, int steps_per_split, int out_cols) {
    // [buffer][operand tile row (8)][k-step in slice (2)][512 values]
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][TG_BM / 16][2][TG_TILE];
    __shared__ __attribute__((aligned(16))) bf16_t ws[2][TG_BN / 16][2][TG_TILE];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;          // wave's place in the 2 x 2 arrangement
    const int m0 = blockIdx.y * TG_BM, n0 = blockIdx.x * TG_BN;
    const int n_groups = (N + 15) >> 4;               // row groups of the packed matrix
    const int s_begin = blockIdx.z * steps_per_split;
    const int s_end = min(n_steps, s_begin + steps_per_split);
    const u32x4 zero4 = {0u, 0u, 0u, 0u};

    f32x4 acc[4][4];                                  // [feature tile][token tile]
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // ---- what this thread fetches for one K slice (64 values of k = two steps)
    // x: 128 rows x 8 chunks of 16 bytes; thread t takes chunks t, t+256, t+512, t+768
    //    chunk c -> row c / 8, k-chunk c % 8 -> LDS tile (row / 16, kc / 4), lane 16 (kc % 4) + row % 16
    // w: 8 row groups x 2 steps x 64 lanes of 16 bytes, copied as they lie
    u32x4 xr[4], wr[4];
    auto fetch = [&](int s) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = tid + 256 * u;
            const int row = c >> 3, kc = c & 7;
            const int gm = m0 + row;
            const int k = s * 32 + kc * 8;
            xr[u] = (gm < M && k + 8 <= K && s + (kc >> 2) < s_end) ? *(const u32x4*)(x + (size_t)gm * K + k) : zero4;
            const int grp = c >> 7, st = (c >> 6) & 1, ln = c & 63;
            const int gg = (n0 >> 4) + grp;
            wr[u] = (gg < n_groups && s + st < s_end)
                        ? *(const u32x4*)(wp + (((size_t)gg * n_steps + s + st) * 64 + ln) * 8) : zero4;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = tid + 256 * u;
            const int row = c >> 3, kc = c & 7;
            *(u32x4*)&xs[buf][row >> 4][kc >> 2][(16 * (kc & 3) + (row & 15)) * 8] = xr[u];
            const int grp = c >> 7, st = (c >> 6) & 1, ln = c & 63;
            *(u32x4*)&ws[buf][grp][st][ln * 8] = wr[u];
        }
    };

    int buf = 0;
    if (s_begin < s_end) {
        fetch(s_begin);
        stash(0);
    }
    __syncthreads();
    for (int s = s_begin; s < s_end; s += 2) {
        const bool more = s + 2 < s_end;
        if (more) fetch(s + 2);
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            bf16x8 a[4], b[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                a[t] = *(const bf16x8*)&ws[buf][wn * 4 + t][st][lane * 8];
                b[t] = *(const bf16x8*)&xs[buf][wm * 4 + t][st][lane * 8];
            }
#pragma unroll
            for (int ta = 0; ta < 4; ++ta)
#pragma unroll
                for (int tb = 0; tb < 4; ++tb)
                    acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ta], b[tb], acc[ta][tb], 0, 0, 0);
        }
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    // ---- store: lane (token j = lane % 16, g) holds rows 4 g .. 4 g + 3 of tile (ta, tb)
    const int j = lane & 15, g = lane >> 4;
    if (SWIGLU) {
#pragma unroll
        for (int tb = 0; tb < 4; ++tb) {
            const int tok = m0 + (wm * 4 + tb) * 16 + j;
#pragma unroll
            for (int ta = 0; ta < 4; ++ta) {
                f32x4 up;
#pragma unroll
                for (int r = 0; r < 4; ++r) up[r] = __shfl_down(acc[ta][tb][r], 16, 64);
                const int f0 = (n0 >> 1) + (wn * 4 + ta) * 8 + 2 * g;
                if ((g & 1) == 0 && tok < M && f0 < out_cols) {
                    f32x4 act;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float gv = acc[ta][tb][r];
                        act[r] = gv / (1.0f + expf(-gv)) * up[r];
                    }
                    TOut* p = out + (size_t)tok * out_cols + f0;
                    if (out_cols % 4 == 0 && f0 + 4 <= out_cols) {
                        tg_store4<TOut>(p, act);
                    } else {
                        for (int r = 0; r < 4 && f0 + r < out_cols; ++r) p[r] = from_f32<TOut>(act[r]);
                    }
                }
            }
        }
        return;
    }
    TOut* obase = out + (size_t)blockIdx.z * M * N;
    const int vec_out = (N % 4 == 0) ? 1 : 0;
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
        const int tok = m0 + (wm * 4 + tb) * 16 + j;
        if (tok >= M) continue;
#pragma unroll
        for (int ta = 0; ta < 4; ++ta) {
            const int f0 = n0 + (wn * 4 + ta) * 16 + 4 * g;
            if (f0 >= N) continue;
            TOut* p = obase + (size_t)tok * N + f0;
            if (vec_out && f0 + 4 <= N) {
                tg_store4<TOut>(p, acc[ta][tb]);
            } else {
                for (int r = 0; r < 4 && f0 + r < N; ++r) p[r] = from_f32<TOut>(acc[ta][tb][r]);
            }
        }
    }
}

template <typename TOut>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ part,
                                                                 TOut* __restrict__ out, size_t total,
                                                                 int splits) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float s = part[i];
    for (int z = 1; z < splits; ++z) s += part[(size_t)z * total + i];
    out[i] = from_f32<TOut>(s);
}

// How many ways K is split for a product of this shape: 1 if the grid fills the chip.
extern "C" int fl_gemm_tiled_splits(int M, int N, int K) {
    const int blocks = ceil_div(M, TG_BM) * ceil_div(N, TG_BN);
    const int steps = ceil_div(K, 32);
    int splits = 1;
    while (blocks * splits < 384 && splits < 16 && steps / (splits * 2) >= 8) splits *= 2;
    return splits;
}

// epilogue 0: out[M, N] = x w^T.  epilogue 1 (SwiGLU): out[M, out_cols] = silu(gate) * up from the
// N interleaved gate/up rows of w (K is not split then).
extern "C" int fl_gemm_tiled(const void* x, const void* w_packed, void* out, float* workspace,
                             int out_dtype, int M, int N, int K, int epilogue, int out_cols,
                             hipStream_t stream) {
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
    FL_CHECK(K % 8 == 0, "gemm_tiled: K=%d is no multiple of 8 (16-byte loads)", K);
    FL_CHECK(out_dtype == FL_F32 || out_dtype == FL_BF16, "gemm_tiled: unknown output dtype %d", out_dtype);
    FL_CHECK(epilogue == 0 || epilogue == 1, "gemm_tiled: unknown epilogue %d", epilogue);
    FL_CHECK(epilogue == 0 ? out_cols == N : (N % 16 == 0 && out_cols > 0 && out_cols <= N / 2),
             "gemm_tiled: %d output columns do not fit %d rows of w", out_cols, N);
    FL_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w_packed % 16 == 0) && ((uintptr_t)out % 16 == 0),
             "gemm_tiled: operands must be 16-byte aligned");
    if (M == 0) return 0;
    const int n_steps = ceil_div(K, 32);
    const int splits = epilogue ? 1 : fl_gemm_tiled_splits(M, N, K);
    FL_CHECK(splits == 1 || workspace, "gemm_tiled: this shape splits K %d ways and needs a workspace", splits);
    int per = ceil_div(n_steps, splits);
    per += per & 1;                                    // whole slices of two steps
    dim3 grid(ceil_div(N, TG_BN), ceil_div(M, TG_BM), splits);
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w_packed;
    if (epilogue) {
        if (out_dtype == FL_F32)
            gemm_tiled_kernel<float, true><<<grid, 256, 0, stream>>>(xb, wb, (float*)out, M, N, K, n_steps, per, out_cols);
        else
            gemm_tiled_kernel<bf16_t, true><<<grid, 256, 0, stream>>>(xb, wb, (bf16_t*)out, M, N, K, n_steps, per, out_cols);
    } else if (splits > 1) {
        gemm_tiled_kernel<float, false><<<grid, 256, 0, stream>>>(xb, wb, workspace, M, N, K, n_steps, per, N);
        FL_LAUNCH_CHECK();
        const size_t total = (size_t)M * N;
        const unsigned rb = (unsigned)((total + 255) / 256);
        if (out_dtype == FL_F32)
            gemm_splitk_reduce_kernel<float><<<rb, 256, 0, stream>>>(workspace, (float*)out, total, splits);
        else
            gemm_splitk_reduce_kernel<bf16_t><<<rb, 256, 0, stream>>>(workspace, (bf16_t*)out, total, splits);
    } else if (out_dtype == FL_F32) {
        gemm_tiled_kernel<float, false><<<grid, 256, 0, stream>>>(xb, wb, (float*)out, M, N, K, n_steps, per, N);
    } else {
        gemm_tiled_kernel<bf16_t, false><<<grid, 256, 0, stream>>>(xb, wb, (bf16_t*)out, M, N, K, n_steps, per, N);
    }
    FL_LAUNCH_CHECK();
    return 0;
}

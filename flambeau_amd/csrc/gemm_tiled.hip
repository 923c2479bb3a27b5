// Tiled bf16 matrix product for prompt portions: out[m, n] = sum_k x[m, k] w[n, k] with many
// rows m, on the matrix cores (v_mfma_f32_16x16x32_bf16, float accumulation).
//
//  * w arrives packed (kernels/packing.py): a tile of 16 features x 32 k is 1 KB in lane order.
//    Operand tiles of both matrices go from memory straight into LDS with
//    global_load_lds_dwordx4 (no staging registers, no ds_write): for w a wave copies the tile as
//    it lies; for the row-major x every lane reads the 16 bytes that the tile layout wants at its
//    place.  A wave then reads an operand from LDS with one ds_read_b128 per lane at consecutive
//    addresses (no bank conflicts, no transposition);
//  * LDS is a ring of NS stages of one k-step (32 values of k); one bare s_barrier per stage;
//  * the w tile is the A operand and the x tile the B operand: C[feature][token] leaves each
//    lane with four consecutive features of one token, one 16-byte store;
//  * two shapes: 256 features x 128 tokens per block (a wave computes 8 x 4 tiles: 12 operand
//    reads feed 32 products) when that grid fills the chip, else 128 x 128 (4 x 4 tiles, deeper
//    ring);
//  * with few rows and a narrow matrix even that grid is small: K is then split over
//    blockIdx.z, the parts are written as float partial sums and a second kernel adds them in
//    a fixed order;
//  * optional SwiGLU epilogue over gate/up rows interleaved in fours.
//
// Measured on the 7B shapes at 2,048 rows: 0.73 to 0.88 PFLOP/s.  What bounds it is the delivery
// of operand tiles into LDS (the same kernel without loads runs at 1.2 to 1.6 PFLOP/s).
//
// The reference's nearest kernel multiplies a 64 x 8 tile per 64-thread block without matrix
// cores (crates/kernels-hip/src/kernels/mmq_f16_tile.cu:33-107).
#include "common.h"
#include "api.h"

#define TG_BM 128                        // block tile the split-K rule counts with
#define TG_BN 128


template <typename TOut>
__device__ __forceinline__ void tg_store4(TOut* p, f32x4 v);
template <> __device__ __forceinline__ void tg_store4<float>(float* p, f32x4 v) { *(f32x4*)p = v; }
template <> __device__ __forceinline__ void tg_store4<bf16_t>(bf16_t* p, f32x4 v) {
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *(bf16x4*)p = o;
}

// ---- the asynchronous variant: operand tiles go from memory straight into LDS
// (global_load_lds_dwordx4: every lane gives its own global address, the 64 x 16 bytes of a wave
// land side by side in LDS, which is exactly the tile layout), through a ring of NS stages of one
// k-step (32 values of k) each.  No staging registers, no ds_write, one barrier per stage:
//     wait for my loads of stage i; barrier; issue the loads of stage i + NS - 1 into the slot that
//     stage i - 1 just left; read the operands of stage i from LDS; FT * TT products.
// Nothing is zero-filled: rows beyond M and feature groups beyond N are clamped to valid ones (their
// results are never stored), and k beyond K meets the zero padding of the packed w.
template <int FT, int TT, int NS, int OCC, typename TOut, bool SWIGLU>
__global__ __launch_bounds__(256, OCC) void gemm_async_kernel(const bf16_t* __restrict__ x,
                                                            const bf16_t* __restrict__ wp,
                                                            TOut* __restrict__ out, int M, int N, int K,
                                                            int n_steps, int steps_per_split, int out_cols) {
    constexpr int NTF = 2 * FT, NTT = 2 * TT;         // operand tiles of the block: features, tokens
    constexpr int TILES = NTF + NTT;                  // 1 KB tiles per stage
    constexpr int LPS = TILES / 4;                    // load instructions per wave and stage
    static_assert(TILES % 4 == 0, "tiles must divide among four waves");
    extern __shared__ __attribute__((aligned(16))) bf16_t ring[];      // [NS][TILES][512]

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wf = wave & 1, wt = wave >> 1;
    const int m0 = blockIdx.y * (NTT * 16), n0 = blockIdx.x * (NTF * 16);
    const int n_groups = (N + 15) >> 4;
    const int s_begin = blockIdx.z * steps_per_split;
    const int s_end = min(n_steps, s_begin + steps_per_split);
    const int n_iter = max(0, s_end - s_begin);

    f32x4 acc[FT][TT];
#pragma unroll
    for (int a = 0; a < FT; ++a)
#pragma unroll
        for (int b = 0; b < TT; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // per-lane source addresses of this wave's tiles at k-step 0 (tile t = wave + 4 u)
    const bf16_t* src[LPS];
    int kstride[LPS];                                 // values to advance per k-step
#pragma unroll
    for (int u = 0; u < LPS; ++u) {
        const int t = wave + 4 * u;
        if (t < NTF) {
            const int gg = min((n0 >> 4) + t, n_groups - 1);
            src[u] = wp + (((size_t)gg * n_steps) * 64 + lane) * 8;
            kstride[u] = 512;
        } else {
            const int row = min(m0 + (t - NTF) * 16 + (lane & 15), M - 1);
            src[u] = x + (size_t)row * K + 8 * (lane >> 4);
            kstride[u] = 32;
        }
    }
    const int x_kmax = K - 8;                         // last whole 16-byte chunk of a row of x
    auto issue = [&](int i) {                         // loads of stage i (k-step s_begin + i) into slot i % NS
        const int s = s_begin + i;
        bf16_t* slot = ring + (size_t)(i % NS) * TILES * 512;
#pragma unroll
        for (int u = 0; u < LPS; ++u) {
            const int t = wave + 4 * u;
            const bf16_t* g = src[u] + (size_t)s * kstride[u];
            if (t >= NTF) {                           // x: keep the chunk inside the row
                const int k = s * 32 + 8 * (lane >> 4);
                if (k > x_kmax) g -= (k - x_kmax);
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                             (__attribute__((address_space(3))) void*)(slot + t * 512), 16, 0, 0);
        }
    };

#pragma unroll
    for (int i = 0; i < NS - 1; ++i)
        if (i < n_iter) issue(i);
    for (int i = 0; i < n_iter; ++i) {
        // my loads of stage i have landed when at most the later stages' are still in flight
        if (i + NS - 2 < n_iter) {
            __builtin_amdgcn_s_waitcnt(0xF70 | ((LPS * (NS - 2)) & 0xF) | ((((LPS * (NS - 2)) >> 4) & 3) << 14));
        } else {
            __builtin_amdgcn_s_waitcnt(0xF70);        // vmcnt(0)
        }
        // a bare barrier: __syncthreads() would add a fence that waits for ALL loads in flight,
        // also those of the later stages, and the ring would be one stage deep
        asm volatile("s_barrier" ::: "memory");
        if (i + NS - 1 < n_iter) issue(i + NS - 1);
        const bf16_t* slot = ring + (size_t)(i % NS) * TILES * 512;
        bf16x8 a[FT], b[TT];
#pragma unroll
        for (int t = 0; t < FT; ++t) a[t] = *(const bf16x8*)(slot + (wf * FT + t) * 512 + lane * 8);
#pragma unroll
        for (int t = 0; t < TT; ++t) b[t] = *(const bf16x8*)(slot + (NTF + wt * TT + t) * 512 + lane * 8);
#pragma unroll
        for (int ta = 0; ta < FT; ++ta)
#pragma unroll
            for (int tb = 0; tb < TT; ++tb)
                acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ta], b[tb], acc[ta][tb], 0, 0, 0);
        // all operand reads first, then the products (the scheduler would otherwise wait for LDS
        // once per pair of feature tiles)
        __builtin_amdgcn_sched_group_barrier(0x100, FT + TT, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, FT * TT, 0);
    }
    // the loads are done (the last stage waited for vmcnt(0)); LDS is not touched again

    const int j = lane & 15, g = lane >> 4;
    if (SWIGLU) {
#pragma unroll
        for (int tb = 0; tb < TT; ++tb) {
            const int tok = m0 + (wt * TT + tb) * 16 + j;
#pragma unroll
            for (int ta = 0; ta < FT; ++ta) {
                f32x4 up;
#pragma unroll
                for (int r = 0; r < 4; ++r) up[r] = __shfl_down(acc[ta][tb][r], 16, 64);
                const int f0 = (n0 >> 1) + (wf * FT + ta) * 8 + 2 * g;
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
    for (int tb = 0; tb < TT; ++tb) {
        const int tok = m0 + (wt * TT + tb) * 16 + j;
        if (tok >= M) continue;
#pragma unroll
        for (int ta = 0; ta < FT; ++ta) {
            const int f0 = n0 + (wf * FT + ta) * 16 + 4 * g;
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

template <int FT, int TT, int NS, int OCC, typename TOut, bool SWIGLU>
static void launch_async(int splits, hipStream_t stream, const bf16_t* x, const bf16_t* wp, TOut* out, int M, int N,
                         int K, int n_steps, int per, int out_cols) {
    constexpr int LDS = NS * (2 * FT + 2 * TT) * 1024;
    static bool configured = false;
    auto kern = gemm_async_kernel<FT, TT, NS, OCC, TOut, SWIGLU>;
    if (!configured) {
        (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        configured = true;
    }
    dim3 grid(ceil_div(N, 2 * FT * 16), ceil_div(M, 2 * TT * 16), splits);
    kern<<<grid, 256, LDS, stream>>>(x, wp, out, M, N, K, n_steps, per, out_cols);
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

// Shape of the block tile: 0 = chosen from the sizes, 1 = 128 x 128, 2 = 256 x 128 (for experiments).
static int g_tiled_variant = 0;
extern "C" int fl_gemm_tiled_set_variant(int v) { g_tiled_variant = v; return 0; }

template <typename TOut, bool SWIGLU>
static void launch_tiled(int variant, int splits, hipStream_t stream, const bf16_t* x, const bf16_t* wp, TOut* out,
                         int M, int N, int K, int n_steps, int per, int out_cols) {
    if (variant == 0) variant = (ceil_div(N, 256) * ceil_div(M, 128) * splits >= 320) ? 2 : 1;
    if (variant == 2)
        launch_async<8, 4, 2, 2, TOut, SWIGLU>(splits, stream, x, wp, out, M, N, K, n_steps, per, out_cols);
    else
        launch_async<4, 4, 4, 2, TOut, SWIGLU>(splits, stream, x, wp, out, M, N, K, n_steps, per, out_cols);
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
    const int per = ceil_div(n_steps, splits);
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w_packed;
    const int v = g_tiled_variant;
    if (epilogue) {
        if (out_dtype == FL_F32)
            launch_tiled<float, true>(v, 1, stream, xb, wb, (float*)out, M, N, K, n_steps, per, out_cols);
        else
            launch_tiled<bf16_t, true>(v, 1, stream, xb, wb, (bf16_t*)out, M, N, K, n_steps, per, out_cols);
    } else if (splits > 1) {
        launch_tiled<float, false>(v, splits, stream, xb, wb, workspace, M, N, K, n_steps, per, N);
        FL_LAUNCH_CHECK();
        const size_t total = (size_t)M * N;
        const unsigned rb = (unsigned)((total + 255) / 256);
        if (out_dtype == FL_F32)
            gemm_splitk_reduce_kernel<float><<<rb, 256, 0, stream>>>(workspace, (float*)out, total, splits);
        else
            gemm_splitk_reduce_kernel<bf16_t><<<rb, 256, 0, stream>>>(workspace, (bf16_t*)out, total, splits);
    } else if (out_dtype == FL_F32) {
        launch_tiled<float, false>(v, 1, stream, xb, wb, (float*)out, M, N, K, n_steps, per, N);
    } else {
        launch_tiled<bf16_t, false>(v, 1, stream, xb, wb, (bf16_t*)out, M, N, K, n_steps, per, N);
    }
    FL_LAUNCH_CHECK();
    return 0;
}

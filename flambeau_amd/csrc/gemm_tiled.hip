// Tiled bf16 matrix product for prompt portions: out[m, n] = sum_k x[m, k] w[n, k] with many
// rows m, on the matrix cores (v_mfma_f32_16x16x32_bf16, float accumulation).
//
//  * w arrives packed (kernels/packing.py): a tile of 16 features x 32 k is 1 KB in lane order.
//    Operand tiles of both matrices go from memory straight into LDS with
//    global_load_lds_dwordx4 (no staging registers, no ds_write): for w a wave copies the tile as
//    it lies; of the row-major x a wave copies 16 rows of 64 bytes, four lanes per row.  A wave
//    then reads an operand from LDS with one ds_read_b128 per lane (w at consecutive addresses, x
//    through an exchange of pieces that keeps the banks apart);
//  * LDS is a ring of NS stages of one k-step (32 values of k); one bare s_barrier per stage;
//  * the w tile is the A operand and the x tile the B operand: C[feature][token] leaves each
//    lane with four consecutive features of one token, one 16-byte store;
//  * two shapes: 256 features x 128 tokens per block (four waves, a wave computes 8 x 4 tiles: 12
//    operand reads feed 32 products; ring of 3; two blocks per compute unit) when that grid fills
//    the chip, else 128 x 256 (eight waves of 4 x 4 tiles, ring of 4, one block per unit); blocks
//    are handed to the eight dies in turn, each die working on a compact patch of tiles;
//  * with few rows and a narrow matrix even that grid is small: K is then split over
//    blockIdx.z, the parts are written as float partial sums and a second kernel adds them in
//    a fixed order;
//  * epilogues: plain; SwiGLU over gate/up rows interleaved in fours; rotate and store q and the
//    cache rows (rope_store.h); add to the residual stream and leave the next norm in factors.
//    Every one can scale a token's results by the factor of a norm left that way (TiledFusion).
//
// Measured on the 7B shapes: 0.78 to 1.09 PFLOP/s at 2,048 rows, 1.1 to 1.2 at 4,096.  What bounds
// it is the delivery of operand tiles into LDS: for 28672 x 4096 x 4096 the matrix cores alone take
// 555 us, with the operand reads 583, with the barrier 637, the whole kernel 871, and the stream
// of copies alone 700 (about 14 TB/s out of the L2s, whatever the tile shape, ring depth, order of
// issue or row stride).
//
// The reference's nearest kernel multiplies a 64 x 8 tile per 64-thread block without matrix
// cores (crates/kernels-hip/src/kernels/mmq_f16_tile.cu:33-107).
#include <type_traits>
#include "common.h"
#include "api.h"
#include "recordable.h"
#include "rope_store.h"

#define TG_PLAIN 0                       // epilogues
#define TG_SWIGLU 1
#define TG_ROPE 2
#define TG_RESIDUAL 3

// Fusion with the norms around a product (as in gemm_skinny.hip).  in_ssq: x is bf16(r * g) and every
// token's results are multiplied by rsqrt(sum_p in_ssq[m][p] / K + eps).  TG_RESIDUAL: nothing is
// stored in out; resid[M, N] += the product, xg = bf16(resid * g), out_ssq[m][tile of features] =
// the block's sum of resid^2.
struct TiledFusion {
    const float* in_ssq;
    int in_parts;
    float eps;
    float* resid;
    const float* g;
    bf16_t* xg;
    float* out_ssq;
};


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
template <int FT, int TT, int WT, int NS, int OCC, typename TOut, int EPI, bool KWHOLE>
__global__ __launch_bounds__(128 * WT, OCC) void gemm_async_kernel(const bf16_t* __restrict__ x,
                                                            const bf16_t* __restrict__ wp,
                                                            TOut* __restrict__ out, int M, int N, int K,
                                                            int n_steps, int steps_per_split, int out_cols,
                                                            RopeStore rs, TiledFusion fu) {
    constexpr int NW = 2 * WT;                        // waves: 2 along the features, WT along the tokens
    constexpr int NTF = 2 * FT, NTT = WT * TT;        // operand tiles of the block: features, tokens
    constexpr int TILES = NTF + NTT;                  // 1 KB tiles per stage
    constexpr int LPS = TILES / NW;                   // load instructions per wave and stage
    static_assert(TILES % NW == 0, "tiles must divide among the waves");
    extern __shared__ __attribute__((aligned(16))) bf16_t ring[];      // [NS][TILES][512]
    __shared__ float s_scale[NTT * 16];                               // row scale of the block's tokens

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // the same for the whole wave: LDS addresses of its copies are scalars
    const int wf = wave & 1, wt = wave >> 1;
    // Which tile: blocks go to the eight dies of the chip in turn (block b to die b % 8), each die
    // with an L2 of its own.  A die gets one contiguous eighth of the tiles, ordered in groups of 8
    // feature tiles by all token tiles, so that the blocks it runs at one time share rows of w and x.
    const int n_ft = (N + NTF * 16 - 1) / (NTF * 16), n_tt = (M + NTT * 16 - 1) / (NTT * 16);
    const int total = n_ft * n_tt, per_die = (total + 7) >> 3;
    const int lin = (blockIdx.x & 7) * per_die + (blockIdx.x >> 3);
    if (lin >= total) return;
    const int grp = lin / (8 * n_tt), within = lin - grp * (8 * n_tt);
    const int gf = min(8, n_ft - grp * 8);
    const int tile_f = grp * 8 + within % gf, tile_t = within / gf;
    const int m0 = tile_t * (NTT * 16), n0 = tile_f * (NTF * 16);
    const int n_groups = (N + 15) >> 4;
    const int s_begin = blockIdx.z * steps_per_split;
    const int s_end = min(n_steps, s_begin + steps_per_split);
    const int n_iter = max(0, s_end - s_begin);

    f32x4 acc[FT][TT];
#pragma unroll
    for (int a = 0; a < FT; ++a)
#pragma unroll
        for (int b = 0; b < TT; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // per-lane source addresses of this wave's tiles at the next stage to load; a wave copies LW
    // tiles of w and LX tiles of x per stage
    constexpr int LW = NTF / NW, LX = NTT / NW;
    static_assert(NTF % NW == 0 && NTT % NW == 0, "tiles must divide among the waves");
    const bf16_t* wsrc[LW];
    const bf16_t* xsrc[LX];
#pragma unroll
    for (int u = 0; u < LW; ++u) {
        const int gg = min((n0 >> 4) + wave * LW + u, n_groups - 1);
        wsrc[u] = wp + (((size_t)gg * n_steps + s_begin) * 64 + lane) * 8;
    }
    // x: the four lanes of a quad read 64 consecutive bytes of one row (a quad that spreads over four
    // rows costs four cache lookups instead of one: measured 15 against 37 bytes per clock and CU).
    // The tile then lies row by row in LDS; the 16-byte pieces of a row are exchanged by
    // (row / 2) % 4, with which the operand reads below meet no bank twice (measured: 4.3 clocks per
    // read instruction against 8.2 without or with other exchanges).
    const int x_piece = 8 * ((lane & 3) ^ ((lane >> 3) & 3));
#pragma unroll
    for (int u = 0; u < LX; ++u) {
        const int row = min(m0 + (wave * LX + u) * 16 + (lane >> 2), M - 1);
        xsrc[u] = x + (size_t)row * K + (size_t)s_begin * 32 + x_piece;
    }
    const int x_kmax = K - 8;                         // last whole 16-byte chunk of a row of x
    // operand lane (token i = lane % 16, k-piece g = lane / 16) finds its 16 bytes of an x tile here
    const int x_read = 32 * (lane & 15) + 8 * ((lane >> 4) ^ (((lane & 15) >> 1) & 3));
    // load c of this wave's LPS loads of stage i (k-step s_begin + i) into slot i % NS: its LW tiles of
    // w first, then its LX tiles of x
    auto issue_one = [&](int i, auto c_) {
        constexpr int c = decltype(c_)::value;
        bf16_t* slot = ring + (size_t)(i % NS) * TILES * 512;
        if constexpr (c < LW) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)wsrc[c],
                                             (__attribute__((address_space(3))) void*)(slot + (wave * LW + c) * 512), 16, 0, 0);
            wsrc[c] += 512;
        } else {
            constexpr int u = c - LW;
            const bf16_t* g = xsrc[u];
            if (!KWHOLE) {                            // K is no multiple of 32: keep the last pieces inside the row
                const int k = (s_begin + i) * 32 + x_piece;
                if (k > x_kmax) g -= (k - x_kmax);
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                             (__attribute__((address_space(3))) void*)(slot + (NTF + wave * LX + u) * 512), 16, 0, 0);
            xsrc[u] += 32;
        }
    };
    auto issue = [&](int i) {                         // all loads of stage i
        static_for<LPS>([&](auto c) { issue_one(i, c); });
    };

    // One block per CU has nothing that runs beside its epilogue, so the residual epilogue's reads
    // are issued here, ahead of all other loads, and wait in registers (where there is room: with 4 x 4
    // tiles per wave, not with 8 x 4).
    constexpr bool PREFETCH = EPI == TG_RESIDUAL && OCC == 1 && FT * TT <= 16;
    const int j = lane & 15, g = lane >> 4;
    f32x4 pre[PREFETCH ? FT : 1][PREFETCH ? TT : 1];
    if (PREFETCH) {
#pragma unroll
        for (int tb = 0; tb < TT; ++tb)
#pragma unroll
            for (int ta = 0; ta < FT; ++ta) {
                const int tok = min(m0 + (wt * TT + tb) * 16 + j, M - 1);
                const int f0 = min(n0 + (wf * FT + ta) * 16 + 4 * g, N - 4);
                pre[PREFETCH ? ta : 0][PREFETCH ? tb : 0] = *(const f32x4*)(fu.resid + (size_t)tok * N + f0);
            }
    }

#pragma unroll
    for (int i = 0; i < NS - 1; ++i)
        if (i < n_iter) issue(i);
    if (fu.in_ssq) {
        // Every token's factor rsqrt(mean r^2 + eps) while the first stages are on their way: eight
        // lanes add a token's parts (lane l parts l, l + 8, ...), then each other's sums.
        const int lp = tid & 7;
#pragma unroll
        for (int t = tid >> 3; t < NTT * 16; t += NW * 8) {
            const float* parts = fu.in_ssq + (size_t)min(m0 + t, M - 1) * fu.in_parts;
            const int last = fu.in_parts - 1;
            float sum = 0.f;
            for (int p = lp; p <= last; p += 32) {
                const float v0 = parts[p], v1 = parts[min(p + 8, last)], v2 = parts[min(p + 16, last)],
                            v3 = parts[min(p + 24, last)];
                sum += (v0 + (p + 8 <= last ? v1 : 0.f)) + ((p + 16 <= last ? v2 : 0.f) + (p + 24 <= last ? v3 : 0.f));
            }
            sum += __shfl_xor(sum, 1, 64);
            sum += __shfl_xor(sum, 2, 64);
            sum += __shfl_xor(sum, 4, 64);
            if (lp == 0) s_scale[t] = rsqrtf(sum / (float)K + fu.eps);
        }
    }
    auto read_operands = [&](bf16x8 (&a)[FT], bf16x8 (&b)[TT], int i) {
        const bf16_t* slot = ring + (size_t)(i % NS) * TILES * 512;
#pragma unroll
        for (int t = 0; t < TT; ++t) b[t] = *(const bf16x8*)(slot + (NTF + wt * TT + t) * 512 + x_read);
#pragma unroll
        for (int t = 0; t < FT; ++t) a[t] = *(const bf16x8*)(slot + (wf * FT + t) * 512 + lane * 8);
    };
    auto products = [&](const bf16x8 (&a)[FT], const bf16x8 (&b)[TT]) {
#pragma unroll
        for (int ta = 0; ta < FT; ++ta)
#pragma unroll
            for (int tb = 0; tb < TT; ++tb)
                acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ta], b[tb], acc[ta][tb], 0, 0, 0);
    };
    // my loads of stage j have landed when at most BEHIND later stages' are still in flight
    auto wait_stage = [&](int j, auto behind) {
        constexpr int N_LATER = LPS * decltype(behind)::value;
        if (j + decltype(behind)::value < n_iter) {
            __builtin_amdgcn_s_waitcnt(0xF70 | (N_LATER & 0xF) | (((N_LATER >> 4) & 3) << 14));
        } else {
            __builtin_amdgcn_s_waitcnt(0xF70);        // vmcnt(0)
        }
        // a bare barrier: __syncthreads() would add a fence that waits for ALL loads in flight,
        // also those of the later stages, and the ring would be one stage deep
        asm volatile("s_barrier" ::: "memory");
    };
    using Behind1 = std::integral_constant<int, NS - 2>;       // reads follow the loads NS - 1 stages behind
    {
        for (int i = 0; i < n_iter; ++i) {
            wait_stage(i, Behind1{});
            // the operand reads of this stage go first (x, then w in the order the products want
            // them); the loads of a later stage are issued while they are on their way (spreading
            // them among the products instead gained nothing)
            bf16x8 a[FT], b[TT];
            read_operands(a, b, i);
            __builtin_amdgcn_sched_barrier(0);
            if (i + NS - 1 < n_iter) issue(i + NS - 1);
            __builtin_amdgcn_sched_barrier(0);
            products(a, b);
        }
    }
    // the loads are done (the last stage waited for vmcnt(0)); LDS is not touched again

    if (fu.in_ssq) {
        __syncthreads();                                              // s_scale is written
#pragma unroll
        for (int tb = 0; tb < TT; ++tb) {
            const float scale = s_scale[(wt * TT + tb) * 16 + j];
#pragma unroll
            for (int ta = 0; ta < FT; ++ta)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[ta][tb][r] *= scale;
        }
    }
    if (EPI == TG_RESIDUAL) {
        // resid += product; xg = bf16(resid * g); the block's sum of resid^2 per token: this wave's
        // features, then the four lanes of a token, then the two waves that share the tokens
        float* s_part = (float*)ring;                                 // [2][NTT * 16]
        f32x4 gain[FT];                                               // the norm's weights of this lane's features
#pragma unroll
        for (int ta = 0; ta < FT; ++ta) gain[ta] = *(const f32x4*)(fu.g + min(n0 + (wf * FT + ta) * 16 + 4 * g, N - 4));
        __syncthreads();                                              // the ring is no longer read
#pragma unroll
        for (int tb = 0; tb < TT; ++tb) {
            const int tok = m0 + (wt * TT + tb) * 16 + j;
            float sq = 0.f;
            f32x4 old[FT];                                            // the token's residual values, read together
#pragma unroll
            for (int ta = 0; ta < FT; ++ta) {
                const int f0 = min(n0 + (wf * FT + ta) * 16 + 4 * g, N - 4);
                old[ta] = PREFETCH ? pre[PREFETCH ? ta : 0][PREFETCH ? tb : 0]
                                   : *(const f32x4*)(fu.resid + (size_t)min(tok, M - 1) * N + f0);
            }
#pragma unroll
            for (int ta = 0; ta < FT; ++ta) {
                const int f0 = n0 + (wf * FT + ta) * 16 + 4 * g;
                if (tok < M && f0 < N) {
                    const f32x4 nr = old[ta] + acc[ta][tb];
                    const f32x4 gv = gain[ta];
                    *(f32x4*)(fu.resid + (size_t)tok * N + f0) = nr;
                    const bf16x4 o = {(bf16_t)(nr[0] * gv[0]), (bf16_t)(nr[1] * gv[1]), (bf16_t)(nr[2] * gv[2]), (bf16_t)(nr[3] * gv[3])};
                    *(bf16x4*)(fu.xg + (size_t)tok * N + f0) = o;
                    sq += (nr[0] * nr[0] + nr[1] * nr[1]) + (nr[2] * nr[2] + nr[3] * nr[3]);
                }
            }
            sq += __shfl_xor(sq, 16, 64);
            sq += __shfl_xor(sq, 32, 64);
            if (g == 0) s_part[wf * (NTT * 16) + (wt * TT + tb) * 16 + j] = sq;
        }
        __syncthreads();
        for (int t = tid; t < NTT * 16; t += NW * 64)
            if (m0 + t < M) fu.out_ssq[(size_t)(m0 + t) * n_ft + tile_f] = s_part[t] + s_part[NTT * 16 + t];
        return;
    }
    if (EPI == TG_ROPE) {
        // the joined q/k/v projection: rotate, store q and the cache rows (rope_store.h).  What the
        // epilogue looks up (places, angles) is loaded in batches, each with one wait.
        int toks[TT];
        TokenPlace places[TT];
#pragma unroll
        for (int tb = 0; tb < TT; ++tb) toks[tb] = m0 + (wt * TT + tb) * 16 + j;
        rope_token_places<TT>(rs, toks, M, places);
#pragma unroll
        for (int tb = 0; tb < TT; ++tb) {
            const int tok = toks[tb];
            RopeAngles an[FT];
            if (rs.rot) {                                             // (no table without rotated dims)
#pragma unroll
                for (int ta = 0; ta < FT; ++ta)
                    an[ta] = rope_angles(rs, min(tok, M - 1), n0 + (wf * FT + ta) * 16 + 4 * g, g);
            }
#pragma unroll
            for (int ta = 0; ta < FT; ++ta) {
                const int f0 = n0 + (wf * FT + ta) * 16 + 4 * g;
                rope_store4<true>(rs, tok, places[tb], f0, g, acc[ta][tb], tok < M && f0 < N, an[ta]);
            }
        }
        return;
    }
    if (EPI == TG_SWIGLU) {
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

template <int FT, int TT, int WT, int NS, int OCC, typename TOut, int EPI>
static void launch_async(int splits, hipStream_t stream, const bf16_t* x, const bf16_t* wp, TOut* out, int M, int N,
                         int K, int n_steps, int per, int out_cols, const RopeStore& rs, const TiledFusion& fu) {
    constexpr int LDS = NS * (2 * FT + WT * TT) * 1024;
    static bool configured = false;
    auto whole = gemm_async_kernel<FT, TT, WT, NS, OCC, TOut, EPI, true>;
    auto ragged = gemm_async_kernel<FT, TT, WT, NS, OCC, TOut, EPI, false>;
    if (!configured) {
        (void)hipFuncSetAttribute((const void*)whole, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        (void)hipFuncSetAttribute((const void*)ragged, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        configured = true;
    }
    auto kern = (K % 32 == 0) ? whole : ragged;
    const int tiles = ceil_div(N, 2 * FT * 16) * ceil_div(M, WT * TT * 16);
    dim3 grid(ceil_div(tiles, 8) * 8, 1, splits);
    kern<<<grid, 128 * WT, LDS, stream>>>(x, wp, out, M, N, K, n_steps, per, out_cols, rs, fu);
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

// Shape of the block: 3 = 256 features x 128 tokens (4 waves, ring of 3, two blocks per compute unit),
// 7 = 192 x 128 and 8 = 128 x 128 (the same with fewer features), 10 = 256 x 256 (8 waves, ring of 4, one
// block per compute unit), 6 = 128 x 256 (the same with fewer features); 0 = chosen here, together
// with the number of K-splits.  The entry points whose names end in _ex take either from the caller, for
// tests and measurements.
//
// What a shape costs follows from what bounds the kernel, the copies into LDS: a compute unit takes
// about 0.1 us per k-step and round of resident blocks plus 17.5 ns per KB that its blocks copy
// (57 GB/s per unit, whatever the shape and however many blocks share the unit).  So the time of a
// product is that of the units' load, taken half from the mean and half from the unit with the
// most blocks; splitting K adds the parts' way to memory and back and the kernel that sums them.
// A 256 x 256 block copies a third less per product and is bound by the matrix cores as much as by
// the copies: 0.80 us per k-step, and 8 us per block that nothing overlaps (0.73 and 2 where K is
// split and the grid gives no unit a second block: such blocks store plain partial sums; with K whole
// the epilogue is a rotation, an addition to the residual stream or an activation, and the same
// price for it made the joined q/k/v product of 2,048 rows 130 us instead of 118).  It wins where its few blocks still load the units evenly (large
// products: 10 to 20 % at the 24B feed-forward, 12 to 15 % at 7B o/down and 4,096 rows, the 7B down
// product at 300 to 2,048 rows with K in parts).
// Against every shape and number of parts measured (7B and 24B q/k/v, o, gate/up and down at 14 row
// counts from 128 to 4,096, cold weights, parts of K 1 to 6 and 8) the formula's picks take 1.1 % more time
// than the best in total, 2.4 % per product on average and 38 % at worst (o at 384, 768 and 1,536 rows, where
// a split or a smaller block would do better than it predicts).
struct TileShape { int variant, features, tokens, per_unit; };
static const TileShape g_shapes[] = {{3, 256, 128, 2}, {7, 192, 128, 2}, {8, 128, 128, 2}, {10, 256, 256, 1}, {6, 128, 256, 1}};
static const TileShape& tile_shape(int variant) {
    for (const TileShape& t : g_shapes)
        if (t.variant == variant) return t;
    return g_shapes[0];
}
static bool tiled_known(int variant) { return variant == 0 || tile_shape(variant).variant == variant; }

static float tiled_cost(const TileShape& t, int splits, int M, int N, int K) {
    const int units = fl_units();
    const int steps = ceil_div(ceil_div(K, 32), splits);
    const long blocks = (long)ceil_div(N, t.features) * ceil_div(M, t.tokens) * splits;
    const long most = (blocks + units - 1) / units;                    // blocks of the unit with the most
    const long rounds = (most + t.per_unit - 1) / t.per_unit;
    const float mean = blocks > units ? (float)blocks / units : 1.f;
    const float kb = (t.features + t.tokens) * 64 / 1024.f;            // copied per block and k-step
    float us;
    // eight waves, a unit to itself, one block after the other; a grid of parts of K that gives no
    // unit a second block measures shorter (the long K of a down product at 300 to 1,500 rows)
    if (t.variant == 10) us = most == 1 && splits > 1 ? steps * 0.73f + 2.f + 3.f : most * (steps * 0.80f + 8.f) + 3.f;
    else us = steps * (0.10f * rounds + 0.0175f * kb * 0.5f * (mean + most)) + 3.f;
    if (splits > 1) us += 3.f + (float)M * N * 4.f * (2 * splits + 1) / 4.5e6f;
    return us;
}

struct TilePlan { int variant, splits; };
// forced_variant / forced_splits: 0 = free; may_split: the epilogue allows parts of K.  The number of
// splits never depends on a forced shape (a caller sizes the workspace from the sizes alone).
static TilePlan tiled_plan(int M, int N, int K, bool may_split, int forced_variant, int forced_splits) {
    const int steps = ceil_div(K, 32);
    int splits = 1;
    if (forced_splits > 0) {
        splits = max(1, min(forced_splits, steps / 8));
    } else if (may_split) {
        float best_us = 0.f;
        for (const TileShape& t : g_shapes) {
            if (t.variant == 6) continue;                              // (128 x 256 only on request)
            // (any number of parts up to 6, or 8: three fill two rounds where four start a third; 7 and more
            // than 8 measured worse than the formula says, their partial sums no longer stay in the caches)
            for (int s = 1; s <= 8 && (s == 1 || steps / s >= 8); s += (s == 6 ? 2 : 1)) {
                const float us = tiled_cost(t, s, M, N, K);
                if (best_us == 0.f || us < best_us * 0.999f) { best_us = us; splits = s; }
            }
        }
    }
    if (forced_variant) return {forced_variant, splits};
    TilePlan best = {3, splits};
    float best_us = 0.f;
    for (const TileShape& t : g_shapes) {
        if (t.variant == 6) continue;
        const float us = tiled_cost(t, splits, M, N, K);
        if (best_us == 0.f || us < best_us * 0.999f) { best_us = us; best.variant = t.variant; }
    }
    return best;
}

// Parts in which the residual epilogue leaves a token's sum of squares: one per tile of features.
extern "C" int fl_gemm_tiled_parts_ex(int M, int N, int K, int variant) {
    return ceil_div(N, tile_shape(tiled_plan(M, N, K, false, variant, 0).variant).features);
}
extern "C" int fl_gemm_tiled_parts(int M, int N, int K) { return fl_gemm_tiled_parts_ex(M, N, K, 0); }

template <typename TOut, int EPI>
static void launch_tiled(int variant, int splits, hipStream_t stream, const bf16_t* x, const bf16_t* wp, TOut* out,
                         int M, int N, int K, int n_steps, int per, int out_cols, const RopeStore& rs,
                         const TiledFusion& fu = TiledFusion{}) {
    switch (variant) {                                 // (decided by tiled_plan)
        case 6: launch_async<4, 4, 4, 4, 1, TOut, EPI>(splits, stream, x, wp, out, M, N, K, n_steps, per, out_cols, rs, fu); break;
        case 7: launch_async<6, 4, 2, 3, 2, TOut, EPI>(splits, stream, x, wp, out, M, N, K, n_steps, per, out_cols, rs, fu); break;
        case 8: launch_async<4, 4, 2, 3, 2, TOut, EPI>(splits, stream, x, wp, out, M, N, K, n_steps, per, out_cols, rs, fu); break;
        case 10: launch_async<8, 4, 4, 4, 1, TOut, EPI>(splits, stream, x, wp, out, M, N, K, n_steps, per, out_cols, rs, fu); break;
        default: launch_async<8, 4, 2, 3, 2, TOut, EPI>(splits, stream, x, wp, out, M, N, K, n_steps, per, out_cols, rs, fu); break;
    }
}

// How many ways K is split for a product of this shape (forced > 0: that many, as far as K allows).
extern "C" int fl_gemm_tiled_splits_ex(int M, int N, int K, int forced) {
    return tiled_plan(M, N, K, true, 0, forced).splits;
}
extern "C" int fl_gemm_tiled_splits(int M, int N, int K) { return fl_gemm_tiled_splits_ex(M, N, K, 0); }
// The block shape chosen for a product of this shape (may_split = 0: an epilogue that takes whole sums only).
extern "C" int fl_gemm_tiled_shape(int M, int N, int K, int may_split) { return tiled_plan(M, N, K, may_split != 0, 0, 0).variant; }

// epilogue 0: out[M, N] = x w^T.  epilogue 1 (SwiGLU): out[M, out_cols] = silu(gate) * up from the
// N interleaved gate/up rows of w (K is not split then).  in_ssq (or null): [M, in_parts] partial sums of
// squares of the rows that x was made from; every token's results are multiplied by rsqrt(sum / K + eps).
extern "C" int fl_gemm_tiled_ex(const void* x, const void* w_packed, void* out, float* workspace,
                                int out_dtype, int M, int N, int K, int epilogue, int out_cols,
                                const float* in_ssq, int in_parts, float eps, int variant, int forced_splits,
                                hipStream_t stream) {
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
    FL_CHECK(K % 8 == 0, "gemm_tiled: K=%d is no multiple of 8 (16-byte loads)", K);
    FL_CHECK(out_dtype == FL_F32 || out_dtype == FL_BF16, "gemm_tiled: unknown output dtype %d", out_dtype);
    FL_CHECK(epilogue == 0 || epilogue == 1, "gemm_tiled: unknown epilogue %d", epilogue);
    FL_CHECK(epilogue == 0 ? out_cols == N : (N % 16 == 0 && out_cols > 0 && out_cols <= N / 2),
             "gemm_tiled: %d output columns do not fit %d rows of w", out_cols, N);
    FL_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w_packed % 16 == 0) && ((uintptr_t)out % 16 == 0),
             "gemm_tiled: operands must be 16-byte aligned");
    FL_CHECK(!in_ssq || in_parts > 0, "gemm_tiled: a row scale over %d parts", in_parts);
    if (M == 0) return 0;
    const int n_steps = ceil_div(K, 32);
    FL_CHECK(tiled_known(variant), "gemm_tiled: block shape %d (0, 3, 6, 7, 8 or 10)", variant);
    const TilePlan plan = tiled_plan(M, N, K, !epilogue, variant, epilogue ? 1 : forced_splits);
    const int splits = plan.splits, v = plan.variant;
    FL_CHECK(splits == 1 || workspace, "gemm_tiled: this shape splits K %d ways and needs a workspace", splits);
    const int per = ceil_div(n_steps, splits);
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w_packed;
    const RopeStore none{};
    const TiledFusion fu = {in_ssq, in_parts, eps, nullptr, nullptr, nullptr, nullptr};
    if (epilogue) {
        if (out_dtype == FL_F32)
            launch_tiled<float, TG_SWIGLU>(v, 1, stream, xb, wb, (float*)out, M, N, K, n_steps, per, out_cols, none, fu);
        else
            launch_tiled<bf16_t, TG_SWIGLU>(v, 1, stream, xb, wb, (bf16_t*)out, M, N, K, n_steps, per, out_cols, none, fu);
    } else if (splits > 1) {
        launch_tiled<float, TG_PLAIN>(v, splits, stream, xb, wb, workspace, M, N, K, n_steps, per, N, none, fu);
        FL_LAUNCH_CHECK();
        const size_t total = (size_t)M * N;
        const unsigned rb = (unsigned)((total + 255) / 256);
        if (out_dtype == FL_F32)
            gemm_splitk_reduce_kernel<float><<<rb, 256, 0, stream>>>(workspace, (float*)out, total, splits);
        else
            gemm_splitk_reduce_kernel<bf16_t><<<rb, 256, 0, stream>>>(workspace, (bf16_t*)out, total, splits);
    } else if (out_dtype == FL_F32) {
        launch_tiled<float, TG_PLAIN>(v, 1, stream, xb, wb, (float*)out, M, N, K, n_steps, per, N, none, fu);
    } else {
        launch_tiled<bf16_t, TG_PLAIN>(v, 1, stream, xb, wb, (bf16_t*)out, M, N, K, n_steps, per, N, none, fu);
    }
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_tiled_ex)

extern "C" int fl_gemm_tiled_scaled(const void* x, const void* w_packed, void* out, float* workspace,
                                    int out_dtype, int M, int N, int K, int epilogue, int out_cols,
                                    const float* in_ssq, int in_parts, float eps, hipStream_t stream) {
    return fl_gemm_tiled_ex(x, w_packed, out, workspace, out_dtype, M, N, K, epilogue, out_cols, in_ssq, in_parts, eps, 0, 0, stream);
}
FL_RECORDABLE(fl_gemm_tiled_scaled)

extern "C" int fl_gemm_tiled(const void* x, const void* w_packed, void* out, float* workspace,
                             int out_dtype, int M, int N, int K, int epilogue, int out_cols,
                             hipStream_t stream) {
    return fl_gemm_tiled_ex(x, w_packed, out, workspace, out_dtype, M, N, K, epilogue, out_cols, nullptr, 0, 0.f, 0, 0, stream);
}
FL_RECORDABLE(fl_gemm_tiled)

// resid[M, N] += x w^T (float, in place), xg[M, N] = bf16(resid * g), out_ssq[M, fl_gemm_tiled_residual_parts(M, N, K)]
// = the sums of resid^2 in parts: the factors of the norm that follows.  Where K is not split the
// product's epilogue does it (one part per tile of features); where it is, the partial sums go to
// the workspace (fl_gemm_tiled_splits(M, N, K) * M * N floats) and the kernel that adds them does it
// (one part per 4096 features, fl_reduce_residual).
extern "C" int fl_gemm_tiled_residual_ex(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                                         float* resid, const float* g, void* xg, float* out_ssq, int variant,
                                         hipStream_t stream) {
    FL_CHECK(tiled_known(variant), "gemm_tiled_residual: block shape %d (0, 3, 6, 7, 8 or 10)", variant);
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled_residual: bad sizes M=%d N=%d K=%d", M, N, K);
    FL_CHECK(K % 8 == 0, "gemm_tiled_residual: K=%d is no multiple of 8 (16-byte loads)", K);
    FL_CHECK(N % 4 == 0, "gemm_tiled_residual: N=%d is no multiple of 4 (16-byte accesses to the residual rows)", N);
    FL_CHECK(resid && g && xg && out_ssq, "gemm_tiled_residual: needs resid, g, xg and out_ssq");
    FL_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w_packed % 16 == 0) && ((uintptr_t)resid % 16 == 0) &&
             ((uintptr_t)g % 16 == 0) && ((uintptr_t)xg % 8 == 0), "gemm_tiled_residual: operands must be aligned (16 bytes, xg 8)");
    if (M == 0) return 0;
    const int n_steps = ceil_div(K, 32);
    const TilePlan plan = tiled_plan(M, N, K, true, variant, 0);
    const int splits = plan.splits;
    if (splits > 1) {
        FL_CHECK(workspace && (uintptr_t)workspace % 16 == 0, "gemm_tiled_residual: this shape splits K %d ways and needs a workspace", splits);
        launch_tiled<float, TG_PLAIN>(plan.variant, splits, stream, (const bf16_t*)x, (const bf16_t*)w_packed, workspace, M, N, K,
                                      n_steps, ceil_div(n_steps, splits), N, RopeStore{});
        FL_LAUNCH_CHECK();
        return fl_reduce_residual(workspace, resid, g, xg, out_ssq, M, N, splits, stream);
    }
    const TiledFusion fu = {nullptr, 0, 0.f, resid, g, (bf16_t*)xg, out_ssq};
    launch_tiled<float, TG_RESIDUAL>(plan.variant, 1, stream, (const bf16_t*)x, (const bf16_t*)w_packed, resid, M, N, K,
                                     n_steps, n_steps, N, RopeStore{}, fu);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_tiled_residual_ex)

extern "C" int fl_gemm_tiled_residual(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                                      float* resid, const float* g, void* xg, float* out_ssq, hipStream_t stream) {
    return fl_gemm_tiled_residual_ex(x, w_packed, workspace, M, N, K, resid, g, xg, out_ssq, 0, stream);
}
FL_RECORDABLE(fl_gemm_tiled_residual)

// Parts in which fl_gemm_tiled_residual leaves a token's sum of squares.
extern "C" int fl_gemm_tiled_residual_parts(int M, int N, int K) {
    return fl_gemm_tiled_splits(M, N, K) > 1 ? fl_gemm_mid_parts(N) : fl_gemm_tiled_parts(M, N, K);
}

// The K-splits of x w^T left apart: workspace[splits][M][N] (splits = fl_gemm_tiled_splits(M, N, K), at
// least one) for a kernel that adds them with work of its own (the rotation kernel does).  in_ssq as
// in fl_gemm_tiled_scaled: every part is scaled, so that their sum is.
extern "C" int fl_gemm_tiled_partials(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                                      const float* in_ssq, int in_parts, float eps, hipStream_t stream) {
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled_partials: bad sizes M=%d N=%d K=%d", M, N, K);
    FL_CHECK(K % 8 == 0, "gemm_tiled_partials: K=%d is no multiple of 8 (16-byte loads)", K);
    FL_CHECK(workspace && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w_packed % 16 == 0) && ((uintptr_t)workspace % 16 == 0),
             "gemm_tiled_partials: operands must be 16-byte aligned");
    FL_CHECK(!in_ssq || in_parts > 0, "gemm_tiled_partials: a row scale over %d parts", in_parts);
    if (M == 0) return 0;
    const int n_steps = ceil_div(K, 32);
    const TilePlan plan = tiled_plan(M, N, K, true, 0, 0);
    const TiledFusion fu = {in_ssq, in_parts, eps, nullptr, nullptr, nullptr, nullptr};
    launch_tiled<float, TG_PLAIN>(plan.variant, plan.splits, stream, (const bf16_t*)x, (const bf16_t*)w_packed, workspace, M, N, K,
                                  n_steps, ceil_div(n_steps, plan.splits), N, RopeStore{}, fu);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_tiled_partials)

// The joined q/k/v projection of many rows with its rows in paired order: q is rotated and written to
// q_out[M, nh * hd], k rotated and v as it is into the cache pages at the tokens' positions; cs[M,
// rot / 2, 2] are the step's cosines and sines.  K is never split here (for shapes whose K the plain
// product would split, that product followed by the rotation kernel is the faster way).  in_ssq as in
// fl_gemm_tiled_scaled.
extern "C" int fl_gemm_tiled_rope_ex(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                                     int in_parts, float eps, const int* positions, const int* tok_seq,
                                     const int* block_table, int max_blocks, const float* cs, void* q_out,
                                     void* cache_base, int nh, int nkv, int hd, int page_size, int n_pages, int rot,
                                     int write_cache, int variant, hipStream_t stream) {
    FL_CHECK(tiled_known(variant), "gemm_tiled_rope: block shape %d (0, 3, 6, 7, 8 or 10)", variant);
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled_rope: bad sizes M=%d N=%d K=%d", M, N, K);
    FL_CHECK(K % 8 == 0, "gemm_tiled_rope: K=%d is no multiple of 8 (16-byte loads)", K);
    FL_CHECK(positions && tok_seq && block_table && cs && q_out && cache_base,
             "gemm_tiled_rope: needs positions, requests, block table, angles, q and the cache");
    FL_CHECK(hd % 16 == 0 && rot % 16 == 0 && rot <= hd && N == (nh + 2 * nkv) * hd,
             "gemm_tiled_rope: %d features with heads of %d (%d rotated), %d + 2 x %d heads", N, hd, rot, nh, nkv);
    FL_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w_packed % 16 == 0), "gemm_tiled_rope: operands must be 16-byte aligned");
    FL_CHECK(!in_ssq || in_parts > 0, "gemm_tiled_rope: a row scale over %d parts", in_parts);
    if (M == 0) return 0;
    const RopeStore rs = {positions, tok_seq, block_table, max_blocks, (const float2*)cs, (bf16_t*)q_out,
                          PagedCache{cache_base, nkv, page_size, hd, n_pages}, nh, rot, write_cache};
    const TiledFusion fu = {in_ssq, in_parts, eps, nullptr, nullptr, nullptr, nullptr};
    const int n_steps = ceil_div(K, 32);
    launch_tiled<bf16_t, TG_ROPE>(tiled_plan(M, N, K, false, variant, 0).variant, 1, stream, (const bf16_t*)x, (const bf16_t*)w_packed, (bf16_t*)q_out,
                                  M, N, K, n_steps, n_steps, N, rs, fu);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_tiled_rope_ex)

extern "C" int fl_gemm_tiled_rope(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                                  int in_parts, float eps, const int* positions, const int* tok_seq,
                                  const int* block_table, int max_blocks, const float* cs, void* q_out,
                                  void* cache_base, int nh, int nkv, int hd, int page_size, int n_pages, int rot,
                                  int write_cache, hipStream_t stream) {
    return fl_gemm_tiled_rope_ex(x, w_packed, M, N, K, in_ssq, in_parts, eps, positions, tok_seq, block_table, max_blocks, cs,
                                 q_out, cache_base, nh, nkv, hd, page_size, n_pages, rot, write_cache, 0, stream);
}
FL_RECORDABLE(fl_gemm_tiled_rope)

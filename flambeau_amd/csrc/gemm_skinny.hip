// Skinny bf16 matrix product for decode: out[m, n] = sum_k x[m, k] w[n, k] with few rows m
// (up to 64) and a large weight matrix that is read exactly once.  The product is bound by the
// stream of w out of HBM, so the kernel is built around that stream:
//
//  * w is stored packed (see pack_weight in kernels/packing.py): the 16 rows x 32 k that one
//    matrix-core instruction takes as its A operand are 1 KB of contiguous memory in lane
//    order, tiles of one row group following each other along k.  A wave's load instruction
//    then reads one whole kilobyte, and its 8 loads per iteration 8 KB in a row (measured:
//    6.2 TB/s against 5.3 TB/s for 16 row pieces of 64 B per instruction);
//  * a block owns 16 consecutive output features (a row group), or two such groups where that
//    spreads the blocks better over the units (skinny_tiles); its NW waves split K between
//    them and add their partial sums through LDS in a fixed order (no atomics: the result
//    does not depend on timing);
//  * a wave keeps 8 16-byte loads of w in flight per lane before it consumes them; w is loaded
//    with the non-temporal hint so that it does not push x out of the caches;
//  * the arithmetic is v_mfma_f32_16x16x32_bf16 with w as the A operand (16 features x 32 k)
//    and x as the B operand (32 k x 16 tokens): C[feature][token] leaves each lane with four
//    consecutive features of one token, i.e. one 16-byte store.  Rows of x beyond M are not
//    loaded.  With MT > 1 the same w registers feed MT token tiles.  Every block reads all of x:
//    from 5 rows on that is worth fetching by whole rows (skinny_x_staged);
//
// Two fusions with the norm around a product save a kernel each in a decode step:
//  * epilogue 2 (residual): instead of storing the product the block adds it to the residual
//    stream r (float, in place), stores bf16(r * g) for the next product (g = the weight of the
//    norm that follows) and the sum of r^2 over its 16 features, one value per token and block;
//  * row scale: a product whose x is such a bf16(r * g) multiplies every token's results by
//    rsqrt(sum r^2 / K + eps), the sums of the producing blocks added in a fixed order.  The
//    scale commutes with the product, so together the two are norm(r) W^T without a norm kernel
//    (the reference fuses the add into its norm kernel instead,
//    crates/kernels-hip/src/kernels/rmsnorm_f16_add_residual.cu).
//
// The reference's nearest kernels are its float GEMV, one block per output row
// (crates/kernels-hip/src/kernels/dense_gemv_f16_f16.cu:27-71, ..._batched.cu:17-63).
#include "common.h"
#include "api.h"
#include "recordable.h"
#include "rope_store.h"

__device__ __forceinline__ void store4(float* p, f32x4 v) { *(f32x4*)p = v; }
__device__ __forceinline__ void store4(bf16_t* p, f32x4 v) {
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *(bf16x4*)p = o;
}

// SWIGLU: the rows of w are gate and up rows interleaved in fours ([g0-3 | u0-3 | g4-7 | u4-7] per
// group of 16, see interleave_gate_up in kernels/packing.py); the kernel then writes
// silu(gate) * up, N / 2 values per token, instead of the N products.
struct SkinnyFusion {
    const float* in_ssq;      // [M][in_parts] sums of squares of the rows of x before the norm's weight, or null
    int in_parts;
    float eps;
    float* resid;             // epilogue 2: [M][N], read and written
    const float* g;           // epilogue 2: [N] weight of the following norm
    bf16_t* xg;               // epilogue 2: [M][N] bf16(resid * g)
    float* out_ssq;           // epilogue 2: [M][blocks] sum of resid^2 over the block's features
};

#define SKINNY_SCALE_LOADS 4     // loads of partial sums per thread for the row scale
#define SKINNY_LDS_MAX (160 * 1024)
#define EPI_PLAIN 0
#define EPI_SWIGLU 1
#define EPI_RESIDUAL 2
#define EPI_ROPE 3               // rotate q and k, store q and the cache rows (rope_store.h)

// x of eight steps of K for a wave's product, fetched by whole rows: load i brings rows 2 i and 2 i + 1
// (512 bytes each, the lanes end to end, so that every cache line is asked for once and whole; a
// 16-byte piece per row and lane touches every line of the rows in each of the eight loads), parked in
// the wave's own piece of LDS and read back as the matrix instruction's operand.  Piece p (16 bytes) of
// row 2 i + r lies in slot 32 r + (p + r + 2 i) % 32 of load i's kilobyte: the 16 lanes that read
// together (one piece each of rows 0 .. 15) then hit 16 different groups of banks, and so do the 16
// that write together.  XS = loads, rows 2 XS and beyond do not exist (rows from M on repeat row M - 1;
// their columns of the product are never stored).
template <int XS>
__device__ __forceinline__ void skinny_x_staged(const bf16_t* __restrict__ x, int M, int K, int s, int lane, char* stage,
                                                bf16x8 (&b)[8]) {
    const int r = lane >> 5, p = lane & 31;
    bf16x8 v[XS];
#pragma unroll
    for (int i = 0; i < XS; ++i)
        v[i] = *(const bf16x8*)(x + (size_t)min(2 * i + r, M - 1) * K + (size_t)s * 32 + p * 8);
#pragma unroll
    for (int i = 0; i < XS; ++i)
        *(bf16x8*)(stage + i * 1024 + (32 * r + ((p + r + 2 * i) & 31)) * 16) = v[i];
    const int li = lane & 15, g = lane >> 4;
    const int i = min(li >> 1, XS - 1), rr = li & 1;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        b[j] = *(const bf16x8*)(stage + i * 1024 + (32 * rr + ((4 * j + g + rr + 2 * i) & 31)) * 16);
}

template <int MT, typename TOut, int EPI, int T, int XS>
__global__ __launch_bounds__(T == 1 ? 1024 : 512) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                           const bf16_t* __restrict__ wp,
                                                           TOut* __restrict__ out, int M, int N, int K,
                                                           int n_steps, int out_cols, SkinnyFusion fu, RopeStore rs) {
    constexpr bool SWIGLU = EPI == EPI_SWIGLU;
    static_assert(T == 1 || MT == 1, "several row groups per block only with one tile of tokens");
    static_assert(XS == 0 || MT == 1, "x through LDS only with one tile of tokens");
    extern __shared__ float red[];               // [NW][MT * T][64][4], then [NW * 4][16] for the row scale
    const int nw = blockDim.x >> 6;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);      // the same for the whole wave: what depends on it is scalar
    const int li = lane & 15, g = lane >> 4;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    // the block's T row groups (the last block may hold fewer: it reads its last one again and drops the
    // results); tiles of a row group: [n_steps][64 lanes][8 values]
    const int groups = (N + 15) >> 4;
    const int grp0 = blockIdx.x * T;
    const int nt = min(T, groups - grp0);
    const bf16_t* wt[T];
#pragma unroll
    for (int t = 0; t < T; ++t) wt[t] = wp + ((size_t)(grp0 + min(t, nt - 1)) * n_steps * 64 + lane) * 8;
    // wave t < nt finishes row group grp0 + t after the loop
    const bool owner = wave < nt;
    const int my_grp = grp0 + wave;

    // K in steps of 32; this wave's steps [s0, s1)
    const int per = (n_steps + nw - 1) / nw;
    const int s0 = wave * per, s1 = min(n_steps, s0 + per);

    const bf16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int tok = mt * 16 + li;
        xok[mt] = tok < M;
        xrow[mt] = x + (size_t)min(tok, M - 1) * K + 8 * g;
    }
    f32x4 acc[MT * T];
#pragma unroll
    for (int i = 0; i < MT * T; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // row scale (one tile of tokens only): thread t fetches its share of the parts of token t % 16
    // (in fours where the number of parts allows 16-byte loads); the loads are in flight during
    // the loop and are added after it
    constexpr int SSV = SKINNY_SCALE_LOADS;
    f32x4 sv[SSV];
#pragma unroll
    for (int j = 0; j < SSV; ++j) sv[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (MT == 1 && fu.in_ssq) {
        const int n_slices = blockDim.x >> 4;
        const int tok = threadIdx.x & 15;
        if (tok < M) {
            const float* row = fu.in_ssq + (size_t)tok * fu.in_parts;
            if ((fu.in_parts & 3) == 0) {
#pragma unroll
                for (int j = 0; j < SSV; ++j) {
                    const int p = ((threadIdx.x >> 4) + j * n_slices) * 4;
                    if (p < fu.in_parts) sv[j] = *(const f32x4*)(row + p);
                }
            } else {
#pragma unroll
                for (int j = 0; j < SSV; ++j) {
                    const int p = (threadIdx.x >> 4) + j * n_slices;
                    if (p < fu.in_parts) sv[j][0] = row[p];
                }
            }
        }
    }
    // epilogue 2: the wave that finishes a row group fetches its part of the residual stream and of g before the loop
    f32x4 r_in[MT], g_in = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) r_in[mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (EPI == EPI_RESIDUAL && MT == 1 && owner) {
        const int f0 = my_grp * 16 + 4 * g;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (f0 + r < N) g_in[r] = fu.g[f0 + r];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int tok = mt * 16 + li;
            if (tok < M) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (f0 + r < N) r_in[mt][r] = fu.resid[(size_t)tok * N + f0 + r];
            }
        }
    }

    // epilogue 3: where this token's key and value go (two dependent loads) and the angles of this
    // lane's pairs, all asked for now
    TokenPlace place = {-1, 0};
    RopeAngles angles = {};
    const bool angles_early = EPI == EPI_ROPE && MT == 1 && rs.rot >= 8;
    if (EPI == EPI_ROPE && MT == 1 && owner && li < M) {
        place = rope_token_place(rs, li);
        if (angles_early) angles = rope_angles(rs, li, my_grp * 16 + 4 * g, g);
    }

    // the wave's piece of LDS for x (behind the partial sums and the row scale's)
    char* stage = (char*)(red + (size_t)nw * MT * T * 256 + (size_t)nw * 64) + (size_t)wave * XS * 1024;
    int s = s0;
    // iterations of U steps: every load of the iteration is issued before the first product needs
    // its data.  x beyond K does not exist (w is zero there): such chunks count as zero.
#define FL_SKINNY_ITER(U)                                                                              \
    for (; s + U <= s1; s += U) {                                                                      \
        if constexpr (T == 1) {                                                                        \
            bf16x8 a[U];                                                                               \
            _Pragma("unroll") for (int j = 0; j < U; ++j)                                              \
                a[j] = __builtin_nontemporal_load((const bf16x8*)(wt[0] + (size_t)(s + j) * 512));     \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                        \
                bf16x8 b[U];                                                                           \
                if constexpr (XS > 0 && U == 8) {                                                      \
                    skinny_x_staged<XS>(x, M, K, s, lane, stage, b);                                   \
                } else {                                                                               \
                    _Pragma("unroll") for (int j = 0; j < U; ++j)                                      \
                        b[j] = (xok[mt] && (s + j) * 32 + 8 * g + 8 <= K)                              \
                                   ? *(const bf16x8*)(xrow[mt] + (s + j) * 32) : zero;                 \
                }                                                                                      \
                _Pragma("unroll") for (int j = 0; j < U; ++j)                                          \
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], b[j], acc[mt], 0, 0, 0);   \
            }                                                                                          \
        } else {                                                                                       \
            /* the same U steps of every row group in turn (U KB in a row each), x loaded once; the loads   \
               of the next row group are issued before the products of this one (the scheduler is told to   \
               leave that order alone: it would otherwise trade loads in flight for registers) */          \
            bf16x8 b[U];                                                                               \
            bf16x8 a[2][U];                                                                            \
            _Pragma("unroll") for (int j = 0; j < U; ++j)                                              \
                a[0][j] = __builtin_nontemporal_load((const bf16x8*)(wt[0] + (size_t)(s + j) * 512));  \
            if constexpr (XS > 0 && U == 8) {                                                          \
                skinny_x_staged<XS>(x, M, K, s, lane, stage, b);                                       \
            } else {                                                                                   \
                _Pragma("unroll") for (int j = 0; j < U; ++j)                                          \
                    b[j] = (xok[0] && (s + j) * 32 + 8 * g + 8 <= K)                                   \
                               ? *(const bf16x8*)(xrow[0] + (s + j) * 32) : zero;                      \
            }                                                                                          \
            _Pragma("unroll") for (int t = 0; t < T; ++t) {                                            \
                if (t + 1 < T) {                                                                       \
                    _Pragma("unroll") for (int j = 0; j < U; ++j)                                      \
                        a[(t + 1) & 1][j] = __builtin_nontemporal_load(                                \
                            (const bf16x8*)(wt[t + 1 < T ? t + 1 : 0] + (size_t)(s + j) * 512));       \
                }                                                                                      \
                __builtin_amdgcn_sched_barrier(0);                                                     \
                _Pragma("unroll") for (int j = 0; j < U; ++j)                                          \
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t & 1][j], b[j], acc[t], 0, 0, 0); \
                __builtin_amdgcn_sched_barrier(0);                                                     \
            }                                                                                          \
        }                                                                                              \
    }
    FL_SKINNY_ITER(8)
    FL_SKINNY_ITER(4)
    FL_SKINNY_ITER(2)
    FL_SKINNY_ITER(1)
#undef FL_SKINNY_ITER

    // add the waves' partial sums in wave order
#pragma unroll
    for (int i = 0; i < MT * T; ++i) *(f32x4*)(red + (((size_t)wave * MT * T + i) * 64 + lane) * 4) = acc[i];
    float* ssred = red + (size_t)nw * MT * T * 256;              // [slices][16]
    if (MT == 1 && fu.in_ssq) {
        float t = 0.f;
#pragma unroll
        for (int j = 0; j < SSV; ++j) t += (sv[j][0] + sv[j][1]) + (sv[j][2] + sv[j][3]);
        ssred[(threadIdx.x >> 4) * 16 + (threadIdx.x & 15)] = t;
    }
    __syncthreads();
    if (owner) {
        // (with T = 1 this is wave 0 and every tile of tokens; with T > 1 there is one tile of tokens and wave t takes row group t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int mine = T == 1 ? mt : wave;
            f32x4 sum = *(f32x4*)(red + ((size_t)mine * 64 + lane) * 4);
            for (int ww = 1; ww < nw; ++ww) {
                const f32x4 v = *(f32x4*)(red + (((size_t)ww * MT * T + mine) * 64 + lane) * 4);
                sum += v;
            }
            // lane (token li, group g) holds rows 16*block + 4g .. 4g+3 of token mt*16 + li
            const int tok = mt * 16 + li;
            if (MT == 1 && fu.in_ssq) {
                // the token's sum of squares: slices g, g + 4, ... by this lane, then the four lanes of the token
                const int n_slices = blockDim.x >> 4;
                float t = 0.f;
                for (int sl = g; sl < n_slices; sl += 4) t += ssred[sl * 16 + li];
                t += __shfl_xor(t, 16, 64);
                t += __shfl_xor(t, 32, 64);
                const float scale = rsqrtf(t / (float)K + fu.eps);
#pragma unroll
                for (int r = 0; r < 4; ++r) sum[r] *= scale;
            }
            if (EPI == EPI_ROPE) {
                const int f0 = my_grp * 16 + 4 * g;
                if (angles_early) rope_store4<true>(rs, tok, place, f0, g, sum, MT == 1 && tok < M && f0 < N, angles);
                else rope_store4(rs, tok, place, f0, g, sum, MT == 1 && tok < M && f0 < N);
            } else if (EPI == EPI_RESIDUAL) {
                const int f0 = my_grp * 16 + 4 * g;
                f32x4 nr;
                float sq = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    nr[r] = r_in[mt][r] + sum[r];
                    if (f0 + r < N) sq += nr[r] * nr[r];
                }
                sq += __shfl_xor(sq, 16, 64);
                sq += __shfl_xor(sq, 32, 64);
                if (tok < M) {
                    if (g == 0) fu.out_ssq[(size_t)tok * groups + my_grp] = sq;
                    if (f0 < N) {
                        float* pr = fu.resid + (size_t)tok * N + f0;
                        bf16_t* px = fu.xg + (size_t)tok * N + f0;
                        if (N % 4 == 0 && f0 + 4 <= N) {
                            store4(pr, nr);
                            store4(px, (f32x4){nr[0] * g_in[0], nr[1] * g_in[1], nr[2] * g_in[2], nr[3] * g_in[3]});
                        } else {
                            for (int r = 0; r < 4 && f0 + r < N; ++r) {
                                pr[r] = nr[r];
                                px[r] = from_f32<bf16_t>(nr[r] * g_in[r]);
                            }
                        }
                    }
                }
            } else if (SWIGLU) {
                f32x4 up;
#pragma unroll
                for (int r = 0; r < 4; ++r) up[r] = __shfl_down(sum[r], 16, 64);      // lane g+1 holds the up rows
                const int f0 = my_grp * 8 + 2 * g;                                     // g even: features 8 b + 4 (g / 2)
                if ((g & 1) == 0 && tok < M && f0 < out_cols) {
                    f32x4 act;
#pragma unroll
                    for (int r = 0; r < 4; ++r) act[r] = sum[r] / (1.0f + expf(-sum[r])) * up[r];
                    TOut* p = out + (size_t)tok * out_cols + f0;
                    if (out_cols % 4 == 0 && f0 + 4 <= out_cols) {
                        store4(p, act);
                    } else {
                        for (int r = 0; r < 4 && f0 + r < out_cols; ++r) p[r] = from_f32<TOut>(act[r]);
                    }
                }
            } else {
                const int f0 = my_grp * 16 + 4 * g;
                if (tok < M && f0 < N) {
                    TOut* p = out + (size_t)tok * N + f0;
                    if (N % 4 == 0 && f0 + 4 <= N) {
                        store4(p, sum);
                    } else {
                        for (int r = 0; r < 4 && f0 + r < N; ++r) p[r] = from_f32<TOut>(sum[r]);
                    }
                }
            }
        }
    }
}

// Row groups per block.  Every block reads all of x, so with two row groups per block x crosses the chip
// half as often; against that, fewer and larger blocks spread less evenly over the units.  Measured at 7B
// sizes (microseconds at 1 / 8 / 16 rows, x by rows through LDS from 5 rows on): 384 row groups (q/k/v)
// one per block 11.3 / 11.7 / 13.4, two 10.3 / 11.1 / 11.9 (192 blocks: one per unit instead of one or
// two); 1,792 row groups (gate/up) one per block 37.7 / 38.3 / 41.8, two 39.7 / 40.8 / 41.1, four
// 41.4 / 43.0 / 43.5.  The results do not depend on the choice (K is split over the waves as before).
static int skinny_tiles(int M, int N, int tiles_hint) {
    if (M > 16) return 1;
    if (tiles_hint > 0) return tiles_hint;
    const int groups = ceil_div(N, 16);
    if (groups > fl_units() && groups <= 2 * fl_units()) return 2;        // (between one and two row groups per compute unit)
    // from 9 rows on x is fetched by eight loads of two rows where eight rows take four: wide matrices, which
    // have blocks to spare, then share it between two row groups (at 16 rows: 28672 x 4096 43 -> 42 us,
    // 65536 x 5120 120 -> 103, 131072 x 5120 246 -> 209, 32768 x 4096 50 -> 46; at 8 rows no gain)
    return M > 8 && groups >= 2 * fl_units() ? 2 : 1;
}

static int skinny_waves(int N, int K, int nw_hint, int T) {
    const int blocks = ceil_div(ceil_div(N, 16), T);
    const int n_steps = ceil_div(K, 32);
    // enough waves in flight to cover the memory latency: about eight per compute unit and more
    int nw = 4;
    while (nw < 16 && blocks * nw < 8 * fl_units()) nw *= 2;
    if (nw_hint > 0) nw = nw_hint;
    // two row groups per block: a wave holds two sets of w registers, twice the bytes in flight (blocks of
    // 512 threads at most), and with a long K four waves do better than eight (5120 x 32768 at 1 and 8 rows:
    // 53 to 57 us against 60 to 63; with K of 4096 or 5120 the plain product is the same with either and
    // the one that rotates and stores 2 us slower with four)
    if (T > 1 && nw > 8) nw = 8;
    if (T > 1 && n_steps >= 512 && nw > 4) nw = 4;
    while (nw > 1 && n_steps < nw * 2) nw /= 2;
    return nw < T ? T : nw;                   // wave t finishes row group t
}

// How many partial sums per token the row scale of a product of this shape can add.
extern "C" int fl_gemm_skinny_scale_parts(int N, int K, int in_parts) {
    int slices = 64;
    for (int T = 1; T <= 2; T *= 2) slices = min(slices, 4 * skinny_waves(N, K, 0, T));
    return SKINNY_SCALE_LOADS * slices * ((in_parts & 3) == 0 ? 4 : 1);
}

template <int MT, typename TOut, int T, int XS>
static int launch_skinny_t(const bf16_t* x, const bf16_t* wp, TOut* out, int M, int N, int K, int nw_hint,
                           int epilogue, int out_cols, const SkinnyFusion& fu, const RopeStore& rs, hipStream_t stream) {
    const int blocks = ceil_div(ceil_div(N, 16), T);
    const int n_steps = ceil_div(K, 32);
    const int nw = skinny_waves(N, K, nw_hint, T);
    const size_t lds = (size_t)nw * MT * T * 64 * 4 * sizeof(float) + (size_t)nw * 4 * 16 * sizeof(float) + (size_t)nw * XS * 1024;
    // (a launch may ask for more than 64 KB of LDS once the kernel has been told so)
#define FL_SK_LAUNCH(EPI_)                                                                                         \
    {                                                                                                              \
        auto* kernel = gemm_skinny_kernel<MT, TOut, EPI_, T, XS>;                                                  \
        static bool raised = false;                                                                                \
        if (lds > 64 * 1024 && !raised) {                                                                          \
            const hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                                     SKINNY_LDS_MAX);                                              \
            FL_CHECK(e == hipSuccess, "gemm_skinny: hipFuncSetAttribute failed: %s", hipGetErrorString(e));         \
            raised = true;                                                                                         \
        }                                                                                                          \
        kernel<<<blocks, nw * 64, lds, stream>>>(x, wp, out, M, N, K, n_steps, out_cols, fu, rs);                  \
    }
    if (epilogue == EPI_SWIGLU) FL_SK_LAUNCH(EPI_SWIGLU)
    else if (epilogue == EPI_RESIDUAL) FL_SK_LAUNCH(EPI_RESIDUAL)
    else if (epilogue == EPI_ROPE) FL_SK_LAUNCH(EPI_ROPE)
    else FL_SK_LAUNCH(EPI_PLAIN)
#undef FL_SK_LAUNCH
    return 0;
}

// hint: waves per block (0: chosen here) + 256 x row groups per block (0: chosen here, 1 or 2) + 65536 if x is not to go through LDS
template <int MT, typename TOut>
static int launch_skinny(const bf16_t* x, const bf16_t* wp, TOut* out, int M, int N, int K, int hint,
                         int epilogue, int out_cols, const SkinnyFusion& fu, const RopeStore& rs, hipStream_t stream) {
    const int nw_hint = hint & 255;
    if constexpr (MT == 1) {
        const int T = skinny_tiles(M, N, (hint >> 8) & 255);
        // x through LDS from five rows on (four loads of two rows each, or eight), whole steps of K only; with
        // fewer rows the pieces of a load lie in so few cache lines that the detour gains nothing
        int xs = (M <= 4 || K % 32 != 0 || (hint >> 16)) ? 0 : M <= 8 ? 4 : 8;
        if ((size_t)skinny_waves(N, K, nw_hint, T) * (T * 1024 + 256 + xs * 1024) > SKINNY_LDS_MAX) xs = 0;
#define FL_SK_T(T_)                                                                                                     \
        switch (xs) {                                                                                                   \
            case 4: return launch_skinny_t<1, TOut, T_, 4>(x, wp, out, M, N, K, nw_hint, epilogue, out_cols, fu, rs, stream); \
            case 8: return launch_skinny_t<1, TOut, T_, 8>(x, wp, out, M, N, K, nw_hint, epilogue, out_cols, fu, rs, stream); \
            default: return launch_skinny_t<1, TOut, T_, 0>(x, wp, out, M, N, K, nw_hint, epilogue, out_cols, fu, rs, stream); \
        }
        if (T == 2) { FL_SK_T(2) }
        FL_SK_T(1)
#undef FL_SK_T
    }
    return launch_skinny_t<MT, TOut, 1, 0>(x, wp, out, M, N, K, nw_hint, epilogue, out_cols, fu, rs, stream);
}

static int skinny_entry(const void* x, const void* w_packed, void* out, int out_dtype, int M, int N, int K,
                        int nw_hint, int epilogue, int out_cols, const SkinnyFusion& fu, const RopeStore& rs,
                        hipStream_t stream) {
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
    FL_CHECK(M <= 64, "gemm_skinny: %d rows, at most 64", M);
    {
        const int tiles_hint = (nw_hint >> 8) & 255;
        FL_CHECK(nw_hint >= 0 && (nw_hint & 255) <= 16 && tiles_hint <= 2 && (nw_hint >> 17) == 0,
                 "gemm_skinny: hint %d: at most 16 waves per block, and 1 or 2 row groups", nw_hint);
    }
    FL_CHECK(K % 8 == 0, "gemm_skinny: K=%d is no multiple of 8 (16-byte loads)", K);
    FL_CHECK(epilogue >= 0 && epilogue <= 3, "gemm_skinny: unknown epilogue %d", epilogue);
    FL_CHECK(epilogue != EPI_SWIGLU ? out_cols == N : (N % 16 == 0 && out_cols > 0 && out_cols <= N / 2),
             "gemm_skinny: %d output columns do not fit %d rows of w", out_cols, N);
    FL_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w_packed % 16 == 0) && ((uintptr_t)out % 16 == 0),
             "gemm_skinny: operands must be 16-byte aligned");
    if (epilogue == EPI_RESIDUAL) {
        FL_CHECK(fu.resid && fu.g && fu.xg && fu.out_ssq, "gemm_skinny: the residual epilogue needs resid, g, xg and out_ssq");
        FL_CHECK(((uintptr_t)fu.resid % 16 == 0) && ((uintptr_t)fu.xg % 8 == 0), "gemm_skinny: resid and xg must be aligned to 16 and 8 bytes");
    }
    if (epilogue == EPI_ROPE) {
        const int hd = rs.cache.head_dim;
        FL_CHECK(rs.positions && rs.tok_seq && rs.block_table && rs.cs && rs.q_out && rs.cache.base,
                 "gemm_skinny: the rotate-and-store epilogue needs positions, requests, block table, angles, q and the cache");
        FL_CHECK(hd % 16 == 0 && rs.rot % 16 == 0 && rs.rot <= hd && N == (rs.nh + 2 * rs.cache.n_kv_heads) * hd,
                 "gemm_skinny: rotate-and-store over %d features with heads of %d (%d rotated), %d + 2 x %d heads", N, hd,
                 rs.rot, rs.nh, rs.cache.n_kv_heads);
    }
    if (fu.in_ssq || epilogue == EPI_RESIDUAL || epilogue == EPI_ROPE)
        FL_CHECK(M <= 16, "gemm_skinny: the fusions with the norm take at most 16 rows, not %d", M);
    if (fu.in_ssq) {
        const int cap = fl_gemm_skinny_scale_parts(N, K, fu.in_parts);
        FL_CHECK(fu.in_parts > 0 && fu.in_parts <= cap, "gemm_skinny: a row scale over %d parts (at most %d for this shape)",
                 fu.in_parts, cap);
        FL_CHECK((uintptr_t)fu.in_ssq % 16 == 0, "gemm_skinny: the partial sums must be 16-byte aligned");
    }
    if (M == 0) return 0;
    const int mt = ceil_div(M, 16);
#define FL_SK(MT_)                                                                                         \
    if (out_dtype == FL_F32) launch_skinny<MT_, float>((const bf16_t*)x, (const bf16_t*)w_packed, (float*)out, M, N, K, nw_hint, epilogue, out_cols, fu, rs, stream); \
    else launch_skinny<MT_, bf16_t>((const bf16_t*)x, (const bf16_t*)w_packed, (bf16_t*)out, M, N, K, nw_hint, epilogue, out_cols, fu, rs, stream)
    FL_CHECK(out_dtype == FL_F32 || out_dtype == FL_BF16, "gemm_skinny: unknown output dtype %d", out_dtype);
    switch (mt) {
        case 1: FL_SK(1); break;
        case 2: FL_SK(2); break;
        case 3: FL_SK(3); break;
        default: FL_SK(4); break;
    }
#undef FL_SK
    FL_LAUNCH_CHECK();
    return 0;
}

// epilogue 0: out[M, N] = x w^T.  epilogue 1 (SwiGLU): w holds N interleaved gate/up rows and
// out[M, out_cols] = silu(gate) * up with out_cols <= N / 2.
extern "C" int fl_gemm_skinny(const void* x, const void* w_packed, void* out, int out_dtype, int M, int N,
                              int K, int nw_hint, int epilogue, int out_cols, hipStream_t stream) {
    FL_CHECK(epilogue == 0 || epilogue == 1, "gemm_skinny: unknown epilogue %d", epilogue);
    const SkinnyFusion none = {nullptr, 0, 0.f, nullptr, nullptr, nullptr, nullptr};
    return skinny_entry(x, w_packed, out, out_dtype, M, N, K, nw_hint, epilogue, out_cols, none, RopeStore{}, stream);
}
FL_RECORDABLE(fl_gemm_skinny)

// The same product fused with the norms around it.  in_ssq (or null): [M, in_parts] partial sums of
// squares of the rows that x was made from; every token's results are multiplied by
// rsqrt(sum / K + eps).  epilogue 2: nothing is stored in out (it may be null); resid[M, N] += the
// product, xg[M, N] = bf16(resid * g), out_ssq[M, blocks] = the blocks' sums of resid^2, blocks =
// fl_gemm_skinny_blocks(N).
extern "C" int fl_gemm_skinny_fused(const void* x, const void* w_packed, void* out, int out_dtype, int M, int N,
                                    int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                                    float eps, float* resid, const float* g, void* xg, float* out_ssq,
                                    hipStream_t stream) {
    FL_CHECK(epilogue != EPI_ROPE, "gemm_skinny_fused: the rotate-and-store epilogue has its own entry point");
    const SkinnyFusion fu = {in_ssq, in_parts, eps, resid, g, (bf16_t*)xg, out_ssq};
    if (epilogue == EPI_RESIDUAL && !out) out = resid;
    return skinny_entry(x, w_packed, out, epilogue == EPI_RESIDUAL ? FL_F32 : out_dtype, M, N, K, 0, epilogue,
                        out_cols, fu, RopeStore{}, stream);
}
FL_RECORDABLE(fl_gemm_skinny_fused)

// The joined q/k/v projection of at most 16 rows with its rows in paired order: q is rotated and
// written to q_out[M, nh * hd], k rotated and v as it is into the cache pages at the tokens'
// positions; cs[M, rot / 2, 2] are the step's cosines and sines.  in_ssq as in fl_gemm_skinny_fused.
extern "C" int fl_gemm_skinny_rope(const void* x, const void* w_packed, int M, int N, int K, const float* in_ssq,
                                   int in_parts, float eps, const int* positions, const int* tok_seq,
                                   const int* block_table, int max_blocks, const float* cs, void* q_out,
                                   void* cache_base, int nh, int nkv, int hd, int page_size, int n_pages, int rot,
                                   int write_cache, hipStream_t stream) {
    const SkinnyFusion fu = {in_ssq, in_parts, eps, nullptr, nullptr, nullptr, nullptr};
    const RopeStore rs = {positions, tok_seq, block_table, max_blocks, (const float2*)cs, (bf16_t*)q_out,
                          PagedCache{cache_base, nkv, page_size, hd, n_pages}, nh, rot, write_cache};
    return skinny_entry(x, w_packed, q_out, FL_BF16, M, N, K, 0, EPI_ROPE, N, fu, rs, stream);
}
FL_RECORDABLE(fl_gemm_skinny_rope)

extern "C" int fl_gemm_skinny_blocks(int N) { return ceil_div(N, 16); }

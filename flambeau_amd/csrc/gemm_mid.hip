// bf16 matrix product for 17 to 64 rows: out[m, n] = sum_k x[m, k] w[n, k], a decode batch of
// that many requests.  Like the skinny kernel it is bound by the stream of w out of HBM, which a
// wave reads tile by tile (1 KB of packed w per load instruction) straight into registers.  With
// more than one tile of tokens the second operand becomes the problem: each 1 KB of w wants up
// to 4 KB of x, and when every wave fetches those from the caches itself the loop waits for the
// cache four times per iteration.  So here the eight waves of a block walk the SAME range of k,
// each with a row group of its own, and share x through LDS:
//
//  * x is read in chunks of GM_CH k-steps; the waves of the block share the loads of a chunk
//    (every lane reads the 16 bytes that the operand layout wants at its place, so that a tile
//    is 1 KB in lane order in LDS too) and keep them in registers for one chunk's time before
//    they write them into one of two LDS slots;
//  * per chunk: issue the loads of x for the chunk after the next and of w for the next; read
//    the operands of this chunk from its LDS slot, GM_CH * MT products; write the x registers of
//    the next chunk into the other slot; one bare s_barrier.  All loads go to registers, so the
//    compiler counts them and every wait lets the younger loads stay in flight;
//  * K is split over blockIdx.y when the row groups alone do not fill the chip; the parts are
//    float partial sums that a second kernel adds in a fixed order;
//  * nothing is zero-filled: token rows beyond M are clamped to the last row (their columns are
//    never stored), K is a multiple of 32 (other shapes stay with the skinny kernel), and k-steps
//    beyond the matrix take a zero tile of w.
//
// Like the skinny kernel it fuses with the norms around it: a product whose x is bf16(r * g) (g =
// the norm's weight) multiplies every token's results by rsqrt(sum r^2 / K + eps) (the sums come
// in parts), and the kernel that adds the K-splits can add them to the residual stream instead and
// leave bf16(r * g) and the sums of r^2 for the next product: no norm kernel runs between them.
//
// The reference's nearest kernel is its batched float GEMV, one block per output row
// (crates/kernels-hip/src/kernels/dense_gemv_f16_f16_batched.cu:17-63).
#include "common.h"
#include "api.h"
#include "recordable.h"


template <typename TOut>
__device__ __forceinline__ void gm_store4(TOut* p, f32x4 v);
template <> __device__ __forceinline__ void gm_store4<float>(float* p, f32x4 v) { *(f32x4*)p = v; }
template <> __device__ __forceinline__ void gm_store4<bf16_t>(bf16_t* p, f32x4 v) {
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *(bf16x4*)p = o;
}

#define GM_SCALE_PARTS 4          // parts of a token's sum of squares the row scale keeps in registers
#define GM_SCALE_MAX_PARTS 4096   // more parts than that (a producer with a part per 16 features) are added before the loop

// GM_NW waves (row groups) per block, GM_CH k-steps per chunk
template <int MT, int GM_NW, int GM_CH, typename TOut, bool SWIGLU>
__global__ __launch_bounds__(GM_NW * 64) void gemm_mid_kernel(const bf16_t* x, const bf16_t* wp, TOut* out, int M, int N, int K,
                                                              int n_steps, int chunks_per_split, int out_cols,
                                                              const float* in_ssq, int in_parts, float eps) {
    constexpr int FR = GM_CH * MT;                    // 1 KB operand tiles of x per chunk
    constexpr int XL = (FR + GM_NW - 1) / GM_NW;      // x loads per wave and chunk
    __shared__ __attribute__((aligned(16))) bf16_t slots[2][FR * 512];

    // wave-uniform values live in scalar registers, so that a load's address is a scalar base plus
    // a per-lane offset that never changes: no vector arithmetic per load
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int li = lane & 15, g = lane >> 4;
    const int n_groups = (N + 15) >> 4;
    const int group = blockIdx.x * GM_NW + wave;
    const int gg = min(group, n_groups - 1);          // waves beyond the matrix repeat the last group, store nothing
    const bf16_t* wt = wp + (size_t)gg * n_steps * 512;
    const unsigned w_lane = lane * 8;

    const int n_chunks = (n_steps + GM_CH - 1) / GM_CH;
    const int c_begin = blockIdx.y * chunks_per_split;
    const int n_iter = max(0, min(n_chunks, c_begin + chunks_per_split) - c_begin);
    if (n_iter == 0 && !(!SWIGLU && gridDim.y > 1)) return;       // an empty part still writes its zeros

    // This wave's share of a chunk's x: the chunk is MT * 16 rows of GM_CH * 64 bytes, which FR loads of
    // 1 KB take row by row (a load covers 16 / GM_CH whole rows, so that every cache line it touches is
    // used whole; a load that followed the operand tiles would touch 16 rows for 64 bytes each).  Lane
    // (row r, 16-byte piece p) holds k-step j = p / 4, quarter q = p % 4 of its row, which belongs in
    // tile (j, r / 16) at the place of operand lane (q, r % 16).  Inside a tile the 16 tokens of a quarter
    // are exchanged by 4 j + q, so that the sixteen lanes that write one row, and the sixteen that read
    // one quarter of a tile, meet every bank once.
    static_assert(16 % GM_CH == 0, "a load takes whole rows of a chunk");
    constexpr int RPL = 16 / GM_CH, LPR = 64 / RPL;   // rows per load, lanes per row
    unsigned x_lane[XL];
    int xj[XL], xdst[XL];
#pragma unroll
    for (int u = 0; u < XL; ++u) {
        const int f = min(wave + GM_NW * u, FR - 1);  // a surplus load repeats the last one
        const int r = f * RPL + lane / LPR, p = lane % LPR;
        const int j = p >> 2, q = p & 3;
        xj[u] = j;
        xdst[u] = (j * MT + (r >> 4)) * 512 + (q * 16 + ((r & 15) ^ ((4 * j + q) & 15))) * 8;
        x_lane[u] = (unsigned)min(r, M - 1) * (unsigned)K + 8 * q;
    }
    // where operand lane (quarter g, token li) finds its 16 bytes in a tile of k-step j
    int rd_off[GM_CH];
#pragma unroll
    for (int j = 0; j < GM_CH; ++j) rd_off[j] = (g * 16 + (li ^ ((4 * j + g) & 15))) * 8;
    const int last = max(n_iter - 1, 0);
    // chunks beyond the part are clamped to its last chunk and k-steps beyond the matrix to its last
    // step: loads without branches, whose results nobody uses
    auto load_x = [&](bf16x8 (&xr)[XL], int i) {
        const int c = c_begin + min(i, last);
#pragma unroll
        for (int u = 0; u < XL; ++u) {
            const unsigned k = (unsigned)min(c * GM_CH + xj[u], n_steps - 1) * 32u;
            xr[u] = *(const bf16x8*)(x + (x_lane[u] + k));
        }
    };
    auto store_x = [&](const bf16x8 (&xr)[XL], int slot) {
#pragma unroll
        for (int u = 0; u < XL; ++u) *(bf16x8*)(&slots[slot][xdst[u]]) = xr[u];
    };
    auto load_w = [&](bf16x8 (&a)[GM_CH], int i) {
        const int c = c_begin + min(i, last);
#pragma unroll
        for (int j = 0; j < GM_CH; ++j) {
            const bf16_t* base = wt + (size_t)min(c * GM_CH + j, n_steps - 1) * 512;
            a[j] = __builtin_nontemporal_load((const bf16x8*)(base + w_lane));
        }
    };

    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

    bf16x8 a_even[GM_CH], a_odd[GM_CH], x_even[XL], x_odd[XL];
    load_x(x_even, 0);
    load_w(a_even, 0);
    load_x(x_odd, 1);
    // row scale: x was bf16(r * g); every token's sums are multiplied by rsqrt(mean r^2 + eps) at the
    // end (a partial sum of a K-split scales the same way).  The parts of the sums of squares are
    // fetched here, behind the first loads of the operands, and not touched before the loop is over.
    float ssq_part[MT][GM_SCALE_PARTS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int p = 0; p < GM_SCALE_PARTS; ++p) ssq_part[mt][p] = 0.f;
    if (in_ssq && in_parts <= GM_SCALE_PARTS) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int tok = min(mt * 16 + li, M - 1);
#pragma unroll
            for (int p = 0; p < GM_SCALE_PARTS; ++p)
                if (p < in_parts) ssq_part[mt][p] = in_ssq[(size_t)tok * in_parts + p];
        }
    } else if (in_ssq) {
        // many parts (the skinny product leaves one per 16 features): the four lanes of a token add every
        // fourth piece each, four loads at a time, and then each other's sums, in a fixed order
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float* row = in_ssq + (size_t)min(mt * 16 + li, M - 1) * in_parts;
            float t = 0.f;
            if ((in_parts & 3) == 0) {
                const int quads = in_parts >> 2;
                for (int q = g; q < quads; q += 16) {
                    f32x4 v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = *(const f32x4*)(row + 4 * min(q + 4 * e, quads - 1));
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (q + 4 * e < quads) t += (v[e][0] + v[e][1]) + (v[e][2] + v[e][3]);
                }
            } else {
                for (int q = g; q < in_parts; q += 4) t += row[q];
            }
            t += __shfl_xor(t, 16, 64);
            t += __shfl_xor(t, 32, 64);
            ssq_part[mt][0] = t;
        }
    }
    store_x(x_even, 0);
    __builtin_amdgcn_s_waitcnt(0xC07F);               // lgkmcnt(0): my part of the slot is written
    asm volatile("s_barrier" ::: "memory");

    // chunk i: a_cur holds its w, x_nxt the x of chunk i + 1; a_nxt and x_nn receive the loads of
    // chunks i + 1 and i + 2 (the register sets swap roles from chunk to chunk, no copies)
    auto chunk = [&](int i, bf16x8 (&a_cur)[GM_CH], bf16x8 (&a_nxt)[GM_CH], bf16x8 (&x_nxt)[XL], bf16x8 (&x_nn)[XL]) {
        load_x(x_nn, i + 2);
        load_w(a_nxt, i + 1);
        __builtin_amdgcn_sched_barrier(0);            // ... and before the products, not after them
        const bf16_t* slot = &slots[i & 1][0];
        bf16x8 b[GM_CH][MT];
#pragma unroll
        for (int j = 0; j < GM_CH; ++j)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) b[j][mt] = *(const bf16x8*)(slot + (j * MT + mt) * 512 + rd_off[j]);
#pragma unroll
        for (int j = 0; j < GM_CH; ++j) {
            const bf16x8 a = ((c_begin + i) * GM_CH + j < n_steps) ? a_cur[j] : zero;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[j][mt], acc[mt], 0, 0, 0);
        }
        store_x(x_nxt, (i + 1) & 1);
        // a bare barrier: __syncthreads() would wait for every load in flight
        __builtin_amdgcn_s_waitcnt(0xC07F);           // lgkmcnt(0)
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);            // the next chunk's loads are issued after the barrier, in this order
    };
    int i = 0;
    for (; i + 1 < n_iter; i += 2) {                  // no branch inside: the compiler's count of the loads in flight stays exact
        chunk(i, a_even, a_odd, x_odd, x_even);
        chunk(i + 1, a_odd, a_even, x_even, x_odd);
    }
    if (i < n_iter) chunk(i, a_even, a_odd, x_odd, x_even);

    if (group >= n_groups) return;
    if (in_ssq) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            float t = ssq_part[mt][0];
#pragma unroll
            for (int p = 1; p < GM_SCALE_PARTS; ++p) t += ssq_part[mt][p];
            const float scale = rsqrtf(t / (float)K + eps);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[mt][r] *= scale;
        }
    }
    // lane (token li, quarter g) holds features 16 * group + 4 g .. + 3 of token mt * 16 + li
    if (SWIGLU) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int tok = mt * 16 + li;
            f32x4 up;
#pragma unroll
            for (int r = 0; r < 4; ++r) up[r] = __shfl_down(acc[mt][r], 16, 64);      // quarter g + 1 holds the up rows
            const int f0 = group * 8 + 2 * g;
            if ((g & 1) == 0 && tok < M && f0 < out_cols) {
                f32x4 act;
#pragma unroll
                for (int r = 0; r < 4; ++r) act[r] = acc[mt][r] / (1.0f + expf(-acc[mt][r])) * up[r];
                TOut* p = out + (size_t)tok * out_cols + f0;
                if (out_cols % 4 == 0 && f0 + 4 <= out_cols) {
                    gm_store4<TOut>(p, act);
                } else {
                    for (int r = 0; r < 4 && f0 + r < out_cols; ++r) p[r] = from_f32<TOut>(act[r]);
                }
            }
        }
        return;
    }
    TOut* obase = out + (size_t)blockIdx.y * M * N;
    const int f0 = group * 16 + 4 * g;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int tok = mt * 16 + li;
        if (tok < M && f0 < N) {
            TOut* p = obase + (size_t)tok * N + f0;
            if (N % 4 == 0 && f0 + 4 <= N) {
                gm_store4<TOut>(p, acc[mt]);
            } else {
                for (int r = 0; r < 4 && f0 + r < N; ++r) p[r] = from_f32<TOut>(acc[mt][r]);
            }
        }
    }
}

template <typename TOut>
__global__ __launch_bounds__(256) void gemm_mid_reduce_kernel(const float* __restrict__ part, TOut* __restrict__ out,
                                                              size_t total, int splits) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float s = part[i];
    for (int z = 1; z < splits; ++z) s += part[(size_t)z * total + i];
    out[i] = from_f32<TOut>(s);
}

// The K-splits added to the residual stream: resid[m, c] += sum_s part[s][m][c] (rising s); xg[m, c] =
// bf16(resid * g[c]); out_ssq[m, b] = sum of resid^2 over the 4096 columns of block b.  One block
// per (4096 columns, row).
#define GM_RED_COLS 4096
__global__ __launch_bounds__(1024) void gemm_mid_reduce_residual_kernel(const float* __restrict__ part,
                                                                       float* __restrict__ resid,
                                                                       const float* __restrict__ g,
                                                                       bf16_t* __restrict__ xg,
                                                                       float* __restrict__ out_ssq, int M, int N,
                                                                       int splits) {
    __shared__ float red[16];
    const int row = blockIdx.y, c0 = blockIdx.x * GM_RED_COLS + 4 * threadIdx.x;
    const size_t total = (size_t)M * N;
    float sq = 0.f;
    if (c0 < N) {
        const size_t at = (size_t)row * N + c0;
        if (N % 4 == 0) {
            f32x4 s = *(const f32x4*)(part + at);
            for (int z = 1; z < splits; ++z) s += *(const f32x4*)(part + (size_t)z * total + at);
            const f32x4 r = *(const f32x4*)(resid + at) + s;
            const f32x4 gv = *(const f32x4*)(g + c0);
            *(f32x4*)(resid + at) = r;
            const bf16x4 o = {(bf16_t)(r[0] * gv[0]), (bf16_t)(r[1] * gv[1]), (bf16_t)(r[2] * gv[2]), (bf16_t)(r[3] * gv[3])};
            *(bf16x4*)(xg + at) = o;
            sq = (r[0] * r[0] + r[1] * r[1]) + (r[2] * r[2] + r[3] * r[3]);
        } else {
            for (int u = 0; u < 4 && c0 + u < N; ++u) {
                float s = part[at + u];
                for (int z = 1; z < splits; ++z) s += part[(size_t)z * total + at + u];
                const float r = resid[at + u] + s;
                resid[at + u] = r;
                xg[at + u] = from_f32<bf16_t>(r * g[c0 + u]);
                sq += r * r;
            }
        }
    }
    sq = block_sum<16>(sq, red);
    if (threadIdx.x == 0) out_ssq[(size_t)row * gridDim.x + blockIdx.x] = sq;
}

#define GM_STEPS 4                       // k-steps per chunk

// Waves per block: eight row groups share x where the matrix has row groups enough to fill the
// chip with such blocks, four otherwise.
static int mid_waves(int N, int forced = 0) {
    if (forced == 4 || forced == 8) return forced;
    return ceil_div(N, 16) >= 4 * fl_units() ? 8 : 4;
}

// Waves per block and parts of K for a product whose K may be split.  These products are short (tens of
// microseconds) and a block has its compute unit to itself, so they run best as one round of blocks that
// fills the chip as far as it goes: parts = units / blocks, rounded down, whatever number that is (a part is
// at least 4 chunks long, 8 for blocks of eight waves).  Measured at 64 rows: 5120 x 4096 in 80 blocks x 3
// parts 15.4 us, x 2 18.0, x 4 20.0; 5120 x 32768 in 40 blocks of eight waves x 6 parts 59 us, in 80 of four
// x 3 74, x 8 (more than two rounds) 80.  Eight waves stream about 30 GB/s per unit against 22 for four
// and are taken where that outweighs their longer blocks, by 15 % if a block streams less than half a megabyte
// (in effect for the long K of a wide feed-forward's down product); the chip as a whole gives 6.3 TB/s; parts cost a kernel that adds them and their way to memory
// and back.
// (The entry points whose names end in _ex take waves per block and K-splits from the caller, for
// tests and measurements: 0 = chosen here.)
struct MidPlan { int waves, splits; };
static MidPlan mid_plan(int N, int K, int forced_waves, int forced_splits) {
    const int groups = ceil_div(N, 16);
    const int n_chunks = ceil_div(ceil_div(K, 32), GM_STEPS);
    const int units = fl_units();
    MidPlan best = {4, 1};
    float best_us = 0.f;
    for (int w = 4; w <= 8; w *= 2) {
        if (forced_waves ? w != forced_waves : (w == 4 && groups >= 4 * units)) continue;      // (many row groups: eight share x)
        const int blocks = ceil_div(groups, w);
        const int s = forced_splits > 0 ? min(forced_splits, n_chunks)
                                        : max(1, min(min(units / blocks, n_chunks / (w == 8 ? 8 : 4)), 32));
        const long total = (long)blocks * s;
        const float bytes = (float)groups * 32.f * K / total;                                   // of w per block
        const float rate = fminf(w == 8 ? 30e3f : 22e3f, 6.3e6f / (float)min(total, (long)units));   // bytes per us
        float us = (float)ceil_div((int)total, units) * bytes / rate + (s > 1 ? 4.5f + s * 64.f * N * 8.f / 5e6f : 0.f);
        if (w == 8 && bytes < 5e5f) us *= 1.15f;      // (their higher rate shows in long streams only: 6 % at 611 KB per block, none at 458, a loss at 262)
        if (best_us == 0.f || us < best_us) { best = {w, s}; best_us = us; }
    }
    return best;
}

extern "C" int fl_gemm_mid_splits_ex(int M, int N, int K, int waves, int forced) {
    (void)M;
    return mid_plan(N, K, waves, forced).splits;
}
extern "C" int fl_gemm_mid_splits(int M, int N, int K) { return fl_gemm_mid_splits_ex(M, N, K, 0, 0); }

struct MidScale {              // the row scale of a product whose x is a norm in factors (or none)
    const float* in_ssq;
    int in_parts;
    float eps;
};

template <int MT, int NW, int CH, typename TOut, bool SWIGLU>
static void launch_mid_shape(const bf16_t* x, const bf16_t* wp, TOut* out, int M, int N, int K, int splits, int out_cols,
                             const MidScale& sc, hipStream_t stream) {
    const int n_steps = ceil_div(K, 32);
    const int n_chunks = ceil_div(n_steps, CH);
    const int per = ceil_div(n_chunks, splits);
    dim3 grid(ceil_div(ceil_div(N, 16), NW), splits);
    gemm_mid_kernel<MT, NW, CH, TOut, SWIGLU><<<grid, NW * 64, 0, stream>>>(x, wp, out, M, N, K, n_steps, per, out_cols,
                                                                            sc.in_ssq, sc.in_parts, sc.eps);
}

template <int MT, typename TOut, bool SWIGLU>
static void launch_mid(const bf16_t* x, const bf16_t* wp, TOut* out, int M, int N, int K, int splits, int out_cols,
                       const MidScale& sc, hipStream_t stream, int waves) {
    if (mid_waves(N, waves) == 8) launch_mid_shape<MT, 8, GM_STEPS, TOut, SWIGLU>(x, wp, out, M, N, K, splits, out_cols, sc, stream);
    else launch_mid_shape<MT, 4, GM_STEPS, TOut, SWIGLU>(x, wp, out, M, N, K, splits, out_cols, sc, stream);
}

template <typename TOut, bool SWIGLU>
static void launch_mid_mt(int mt, const bf16_t* x, const bf16_t* wp, TOut* out, int M, int N, int K, int splits,
                          int out_cols, const MidScale& sc, hipStream_t stream, int waves = 0) {
    switch (mt) {
        case 1: launch_mid<1, TOut, SWIGLU>(x, wp, out, M, N, K, splits, out_cols, sc, stream, waves); break;
        case 2: launch_mid<2, TOut, SWIGLU>(x, wp, out, M, N, K, splits, out_cols, sc, stream, waves); break;
        case 3: launch_mid<3, TOut, SWIGLU>(x, wp, out, M, N, K, splits, out_cols, sc, stream, waves); break;
        default: launch_mid<4, TOut, SWIGLU>(x, wp, out, M, N, K, splits, out_cols, sc, stream, waves); break;
    }
}

static int mid_checks(const void* x, const void* w_packed, int M, int N, int K) {
    FL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_mid: bad sizes M=%d N=%d K=%d", M, N, K);
    FL_CHECK(M <= 64, "gemm_mid: %d rows, at most 64", M);
    FL_CHECK(K % 32 == 0, "gemm_mid: K=%d is no multiple of 32 (whole k-steps of x)", K);
    FL_CHECK((size_t)M * K < ((size_t)1 << 31), "gemm_mid: x of %d x %d values is beyond 32-bit offsets", M, K);
    FL_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w_packed % 16 == 0), "gemm_mid: operands must be 16-byte aligned");
    return 0;
}

// epilogue 0: out[M, N] = x w^T; a shape that splits K (fl_gemm_mid_splits > 1) needs a float
// workspace of splits * M * N values.  epilogue 1 (SwiGLU): out[M, out_cols] = silu(gate) * up
// from the N interleaved gate/up rows of w; K is not split then.  in_ssq (or null): [M, in_parts]
// partial sums of squares of the rows that x was made from; every token's results are multiplied
// by rsqrt(sum / K + eps).
extern "C" int fl_gemm_mid_ex(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                              int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                              float eps, int waves, int forced_splits, hipStream_t stream) {
    FL_CHECK(waves == 0 || waves == 4 || waves == 8, "gemm_mid: %d waves per block (0, 4 or 8)", waves);
    if (mid_checks(x, w_packed, M, N, K)) return -1;
    FL_CHECK(out_dtype == FL_F32 || out_dtype == FL_BF16, "gemm_mid: unknown output dtype %d", out_dtype);
    FL_CHECK(epilogue == 0 || epilogue == 1, "gemm_mid: unknown epilogue %d", epilogue);
    FL_CHECK(epilogue == 0 ? out_cols == N : (N % 16 == 0 && out_cols > 0 && out_cols <= N / 2),
             "gemm_mid: %d output columns do not fit %d rows of w", out_cols, N);
    FL_CHECK((uintptr_t)out % 16 == 0, "gemm_mid: operands must be 16-byte aligned");
    FL_CHECK(!in_ssq || (in_parts > 0 && in_parts <= GM_SCALE_MAX_PARTS &&
                         (in_parts <= GM_SCALE_PARTS || (in_parts & 3) || (uintptr_t)in_ssq % 16 == 0)),
             "gemm_mid: a row scale over %d parts (at most %d; in fours they must be 16-byte aligned)", in_parts, GM_SCALE_MAX_PARTS);
    if (M == 0) return 0;
    const int mt = ceil_div(M, 16);
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w_packed;
    const MidScale sc = {in_ssq, in_parts, eps};
    const MidPlan plan = epilogue ? MidPlan{mid_waves(N, waves), 1} : mid_plan(N, K, waves, forced_splits);
    const int splits = plan.splits;
    waves = plan.waves;
    FL_CHECK(splits == 1 || workspace, "gemm_mid: this shape splits K %d ways and needs a workspace", splits);
    if (epilogue) {
        if (out_dtype == FL_F32) launch_mid_mt<float, true>(mt, xb, wb, (float*)out, M, N, K, 1, out_cols, sc, stream, waves);
        else launch_mid_mt<bf16_t, true>(mt, xb, wb, (bf16_t*)out, M, N, K, 1, out_cols, sc, stream, waves);
    } else if (splits > 1) {
        launch_mid_mt<float, false>(mt, xb, wb, workspace, M, N, K, splits, N, sc, stream, waves);
        FL_LAUNCH_CHECK();
        const size_t total = (size_t)M * N;
        const unsigned rb = (unsigned)((total + 255) / 256);
        if (out_dtype == FL_F32)
            gemm_mid_reduce_kernel<float><<<rb, 256, 0, stream>>>(workspace, (float*)out, total, splits);
        else
            gemm_mid_reduce_kernel<bf16_t><<<rb, 256, 0, stream>>>(workspace, (bf16_t*)out, total, splits);
    } else if (out_dtype == FL_F32) {
        launch_mid_mt<float, false>(mt, xb, wb, (float*)out, M, N, K, 1, N, sc, stream, waves);
    } else {
        launch_mid_mt<bf16_t, false>(mt, xb, wb, (bf16_t*)out, M, N, K, 1, N, sc, stream, waves);
    }
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_mid_ex)

extern "C" int fl_gemm_mid_scaled(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                                  int M, int N, int K, int epilogue, int out_cols, const float* in_ssq, int in_parts,
                                  float eps, hipStream_t stream) {
    return fl_gemm_mid_ex(x, w_packed, out, workspace, out_dtype, M, N, K, epilogue, out_cols, in_ssq, in_parts, eps, 0, 0, stream);
}
FL_RECORDABLE(fl_gemm_mid_scaled)

extern "C" int fl_gemm_mid(const void* x, const void* w_packed, void* out, float* workspace, int out_dtype,
                           int M, int N, int K, int epilogue, int out_cols, hipStream_t stream) {
    return fl_gemm_mid_scaled(x, w_packed, out, workspace, out_dtype, M, N, K, epilogue, out_cols, nullptr, 0, 0.f, stream);
}
FL_RECORDABLE(fl_gemm_mid)

// The K-splits of x w^T left apart: workspace[s][M][N] for s < fl_gemm_mid_splits(M, N, K) (one "split"
// if K is not split), for a kernel that adds them itself (fl_rope_kv_write).  in_ssq as in
// fl_gemm_mid_scaled: every part is scaled, so their sum is.
extern "C" int fl_gemm_mid_partials(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                                    const float* in_ssq, int in_parts, float eps, hipStream_t stream) {
    if (mid_checks(x, w_packed, M, N, K)) return -1;
    FL_CHECK(workspace && (uintptr_t)workspace % 16 == 0, "gemm_mid_partials: needs a 16-byte aligned workspace");
    FL_CHECK(!in_ssq || (in_parts > 0 && in_parts <= GM_SCALE_MAX_PARTS &&
                         (in_parts <= GM_SCALE_PARTS || (in_parts & 3) || (uintptr_t)in_ssq % 16 == 0)),
             "gemm_mid: a row scale over %d parts (at most %d; in fours they must be 16-byte aligned)", in_parts, GM_SCALE_MAX_PARTS);
    if (M == 0) return 0;
    const MidScale sc = {in_ssq, in_parts, eps};
    const MidPlan plan = mid_plan(N, K, 0, 0);
    launch_mid_mt<float, false>(ceil_div(M, 16), (const bf16_t*)x, (const bf16_t*)w_packed, workspace, M, N, K,
                                plan.splits, N, sc, stream, plan.waves);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_mid_partials)

// resid[M, N] += x w^T (float, in place), xg[M, N] = bf16(resid * g), out_ssq[M, fl_gemm_mid_parts(N)] =
// sums of resid^2 over 4096 columns each: the factors of the norm that follows.  The workspace holds
// fl_gemm_mid_splits(M, N, K) * M * N floats (also when K is not split).
extern "C" int fl_gemm_mid_residual(const void* x, const void* w_packed, float* workspace, int M, int N, int K,
                                    float* resid, const float* g, void* xg, float* out_ssq, hipStream_t stream) {
    if (mid_checks(x, w_packed, M, N, K)) return -1;
    FL_CHECK(workspace && resid && g && xg && out_ssq, "gemm_mid_residual: needs workspace, resid, g, xg and out_ssq");
    FL_CHECK(((uintptr_t)workspace % 16 == 0) && ((uintptr_t)resid % 16 == 0) && ((uintptr_t)g % 16 == 0) &&
             ((uintptr_t)xg % 8 == 0), "gemm_mid_residual: workspace, resid and g must be 16-byte aligned, xg 8-byte");
    if (M == 0) return 0;
    const MidPlan plan = mid_plan(N, K, 0, 0);
    const int splits = plan.splits;
    const MidScale none = {nullptr, 0, 0.f};
    launch_mid_mt<float, false>(ceil_div(M, 16), (const bf16_t*)x, (const bf16_t*)w_packed, workspace, M, N, K, splits, N,
                                none, stream, plan.waves);
    FL_LAUNCH_CHECK();
    dim3 grid(ceil_div(N, GM_RED_COLS), M);
    gemm_mid_reduce_residual_kernel<<<grid, 1024, 0, stream>>>(workspace, resid, g, (bf16_t*)xg, out_ssq, M, N, splits);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_gemm_mid_residual)

extern "C" int fl_gemm_mid_parts(int N) { return ceil_div(N, GM_RED_COLS); }

// The second half of fl_gemm_mid_residual on its own, for any number of rows: part[splits][M][N] are
// partial sums of a product; resid += their sum, xg = bf16(resid * g), out_ssq[M, fl_gemm_mid_parts(N)].
extern "C" int fl_reduce_residual(const float* part, float* resid, const float* g, void* xg, float* out_ssq, int M,
                                  int N, int splits, hipStream_t stream) {
    FL_CHECK(M >= 0 && N > 0 && splits >= 1, "reduce_residual: bad sizes M=%d N=%d splits=%d", M, N, splits);
    FL_CHECK(part && resid && g && xg && out_ssq, "reduce_residual: needs part, resid, g, xg and out_ssq");
    FL_CHECK(((uintptr_t)part % 16 == 0) && ((uintptr_t)resid % 16 == 0) && ((uintptr_t)g % 16 == 0) &&
             ((uintptr_t)xg % 8 == 0), "reduce_residual: part, resid and g must be 16-byte aligned, xg 8-byte");
    FL_CHECK(M <= 65535, "reduce_residual: %d rows, at most 65535", M);
    if (M == 0) return 0;
    dim3 grid(ceil_div(N, GM_RED_COLS), M);
    gemm_mid_reduce_residual_kernel<<<grid, 1024, 0, stream>>>(part, resid, g, (bf16_t*)xg, out_ssq, M, N, splits);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_reduce_residual)

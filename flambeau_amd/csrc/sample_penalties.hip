// Penalties and logit bias on the device, so that requests that ask for them are sampled without
// their logits travelling to the host (the engine then stays a step ahead of the host for them too).
//
// Rules and order are the reference's (crates/runtime/src/sampling.rs:575-606 penalties over the
// tokens generated so far, :168-176 bias after them):
//   a token seen c > 0 times:  l = l > 0 ? l / rp : l * rp;  l -= pp;  l -= fp * c
//   then                       l[token] += bias
// The history lives on the device as one row of counts per state slot (16-bit: a token is not
// generated 65,536 times in one request): zeroed or rebuilt when a request takes the slot, bumped
// by the token drawn in every step.
#include "common.h"
#include "api.h"
#include "recordable.h"

// grid (blocks over the vocabulary, rows); rows whose slot is negative or whose penalties are neutral are skipped
__global__ __launch_bounds__(256) void sample_penalise_kernel(float* __restrict__ logits, int V,
                                                              const unsigned short* __restrict__ counts,
                                                              const float* __restrict__ slot,
                                                              const float* __restrict__ repetition,
                                                              const float* __restrict__ presence,
                                                              const float* __restrict__ frequency) {
    const int r = blockIdx.y;
    const int s = (int)slot[r];
    const float rp = repetition[r], pp = presence[r], fp = frequency[r];
    if (s < 0 || (rp == 1.f && pp == 0.f && fp == 0.f)) return;
    const unsigned short* seen = counts + (size_t)s * V;
    float* row = logits + (size_t)r * V;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < V; i += gridDim.x * 256) {
        const unsigned c = seen[i];
        if (c == 0u) continue;
        float l = row[i];
        if (rp != 1.f) l = l > 0.f ? l / rp : __fmul_rn(l, rp);
        if (pp != 0.f) l = __fsub_rn(l, pp);
        if (fp != 0.f) l = __fsub_rn(l, __fmul_rn(fp, (float)c));
        row[i] = l;
    }
}

// logits[row[j]][token[j]] += value[j]; a (row, token) pair occurs once
__global__ __launch_bounds__(256) void sample_bias_kernel(float* __restrict__ logits, int V, int n,
                                                          const float* __restrict__ row, const float* __restrict__ token,
                                                          const float* __restrict__ value) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    const int t = (int)token[j];
    if (t < 0 || t >= V) return;
    float* p = logits + (size_t)(int)row[j] * V + t;
    *p = __fadd_rn(*p, value[j]);
}

// counts[slot[r]][ids[r]] += 1 for rows with a slot (one row per slot in a step)
__global__ __launch_bounds__(256) void sample_count_kernel(unsigned short* __restrict__ counts, int V, int rows,
                                                           const float* __restrict__ slot, const int* __restrict__ ids) {
    const int r = blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    const int s = (int)slot[r], t = ids[r];
    if (s < 0 || t < 0 || t >= V) return;
    unsigned short* p = counts + (size_t)s * V + t;
    *p = (unsigned short)min(65535u, (unsigned)*p + 1u);
}

// One slot's row is counted anew in two kernels: the row is zeroed by a grid over the vocabulary, then
// every token adds one to its count.  16-bit counts have no atomics of their own: a thread adds 1 or
// 65536 to the aligned 32-bit word that holds the count (rows start at even counts only if V is even, so
// the word is found from the count's own address).  Fewer than 65,536 tokens cannot carry from one count
// into its neighbour; longer lists are counted by one thread, saturating.
__global__ __launch_bounds__(256) void sample_history_zero_kernel(unsigned short* __restrict__ counts, int V, int slot) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < V) counts[(size_t)slot * V + i] = 0;
}

__global__ __launch_bounds__(256) void sample_history_count_kernel(unsigned short* __restrict__ counts, int V, int slot,
                                                                   const int* __restrict__ tokens, int n, int serial) {
    unsigned short* row = counts + (size_t)slot * V;
    if (serial) {
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            for (int j = 0; j < n; ++j) {
                const int t = tokens[j];
                if (t >= 0 && t < V) row[t] = (unsigned short)min(65535u, (unsigned)row[t] + 1u);
            }
        }
        return;
    }
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    const int t = tokens[j];
    if (t < 0 || t >= V) return;
    const uintptr_t at = (uintptr_t)(row + t);
    atomicAdd((unsigned*)(at & ~(uintptr_t)3), (at & 2) ? 65536u : 1u);
}

// Penalties of the rows that have a history slot (slot[r] >= 0, as a float), in place on logits [rows, V].
extern "C" int fl_sample_penalise(float* logits, int rows, int V, const unsigned short* counts, const float* slot,
                                  const float* repetition, const float* presence, const float* frequency,
                                  hipStream_t stream) {
    FL_CHECK(rows >= 0 && V > 0 && logits && counts && slot && repetition && presence && frequency, "sample_penalise: bad arguments");
    if (rows == 0) return 0;
    FL_CHECK(rows <= 65535, "sample_penalise: %d rows, at most 65535", rows);
    dim3 grid(min(ceil_div(V, 256 * 8), 64), rows);
    sample_penalise_kernel<<<grid, 256, 0, stream>>>(logits, V, counts, slot, repetition, presence, frequency);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_sample_penalise)

extern "C" int fl_sample_bias(float* logits, int V, int n, const float* row, const float* token, const float* value,
                              hipStream_t stream) {
    FL_CHECK(n >= 0 && V > 0 && logits && (n == 0 || (row && token && value)), "sample_bias: bad arguments");
    if (n == 0) return 0;
    sample_bias_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(logits, V, n, row, token, value);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_sample_bias)

// The drawn tokens join their requests' histories.
extern "C" int fl_sample_count(unsigned short* counts, int V, int rows, const float* slot, const int* ids, hipStream_t stream) {
    FL_CHECK(rows >= 0 && V > 0 && counts && slot && ids, "sample_count: bad arguments");
    if (rows == 0) return 0;
    sample_count_kernel<<<ceil_div(rows, 256), 256, 0, stream>>>(counts, V, rows, slot, ids);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_sample_count)

// A request takes a slot: its row is zeroed and the n tokens it has generated so far are counted.
extern "C" int fl_sample_history(unsigned short* counts, int V, int slot, const int* tokens, int n, hipStream_t stream) {
    FL_CHECK(V > 0 && slot >= 0 && n >= 0 && counts && (n == 0 || tokens), "sample_history: bad arguments");
    FL_CHECK((uintptr_t)counts % 4 == 0, "sample_history: the counts must be 4-byte aligned");
    sample_history_zero_kernel<<<ceil_div(V, 256), 256, 0, stream>>>(counts, V, slot);
    FL_LAUNCH_CHECK();
    if (n > 0) {
        const int serial = n >= 65536 ? 1 : 0;
        sample_history_count_kernel<<<serial ? 1 : ceil_div(n, 256), 256, 0, stream>>>(counts, V, slot, tokens, n, serial);
        FL_LAUNCH_CHECK();
    }
    return 0;
}
FL_RECORDABLE(fl_sample_history)

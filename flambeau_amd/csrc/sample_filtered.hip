// The filtered temperature draw on the device: top-k, top-p and min-p.
//
// Per row, in the order of the reference's host sampler (crates/runtime/src/sampling.rs:610-746):
//   p_i = exp(l_i / T - max), normalised by the sum over the whole vocabulary;
//   candidates in the order of falling probability, equal ones by rising index;
//   top-k keeps the first k (2048 stand in when only top-p or min-p is given);
//   top-p keeps the shortest prefix whose probability reaches p; min-p cuts where a probability
//   falls below min_p times the largest (at least one candidate stays);
//   the draw is the first candidate at which the running sum reaches u * sum(kept).
// The reference's device sampler (crates/kernels-hip/src/kernels/sampler_topk_softmax_f32.cu) is a
// single block over one row that selects the top k and leaves the walk to the host; here the walk
// runs on the device too, so that no logits travel and the engine stays a step ahead of the host.
//
// One block of 1,024 threads per row:
//   1. maximum and sum of the exponentials (coalesced);
//   2. the k-th largest probability by a radix selection over the bits of p (p >= 0, so the bits
//      order like the values): eight passes of 4 bits, counted in registers (vocabularies up to
//      32,768 keep their probabilities in registers between the passes);
//   3. the candidates above it, and of those equal to it the first by index, go to LDS as 64-bit
//      keys (bits of p, then the complement of the index) and are sorted by a bitonic network;
//   4. the walk: running sums over the sorted candidates, two per thread, and the first at which
//      top-p, min-p and the drawn number are met.
// Rows without a filter (and greedy rows) are left alone: fl_sample draws them.
#include "common.h"
#include "api.h"
#include "recordable.h"

#define SF_MAX_K 2048
#define SF_THREADS 1024
#define SF_WAVES (SF_THREADS / 64)
#define SF_KEEP 32                      // probabilities a thread keeps in registers (vocabularies up to 32,768)

// exp(l / T - max) with the product and the difference rounded one after the other, as the host forms them
__device__ __forceinline__ float sf_prob(float logit, float inv_t, float scaled_max) {
    return expf(__fsub_rn(__fmul_rn(logit, inv_t), scaled_max));
}

// KEEP: every thread holds the bits of its probabilities in registers (element tid + e * SF_THREADS in
// place e); otherwise they are written to the row's part of `stash` once and read back by every pass
// (or, without a stash, formed again in every pass).
template <bool KEEP>
__global__ __launch_bounds__(SF_THREADS) void sample_filtered_kernel(const float* __restrict__ logits,
                                                                    const float* __restrict__ inv_temp,
                                                                    const float* __restrict__ uniform,
                                                                    const float* __restrict__ top_k,
                                                                    const float* __restrict__ top_p,
                                                                    const float* __restrict__ min_p,
                                                                    int* __restrict__ out, int V,
                                                                    unsigned* __restrict__ stash) {
    __shared__ unsigned long long cand[SF_MAX_K];
    __shared__ unsigned bins[SF_WAVES][16];
    __shared__ int per_thread[SF_THREADS];
    __shared__ float sums[SF_THREADS];
    __shared__ float red[SF_WAVES];
    __shared__ float s_max[SF_WAVES];
    __shared__ unsigned s_prefix, s_remaining, s_count;
    __shared__ int s_end, s_pick;
    __shared__ float s_kept;
    const int r = blockIdx.x, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const float it = inv_temp[r];
    const int k_req = (int)top_k[r];
    const float tp = top_p[r], mp = min_p[r];
    const bool has_tp = tp > 0.f && tp < 1.f, has_mp = mp > 0.f;
    if (!(it > 0.f) || !(k_req > 0 || has_tp || has_mp)) return;          // greedy, or no filter: not this kernel's row
    const float* row = logits + (size_t)r * V;
    const int k = min(min(k_req > 0 ? k_req : SF_MAX_K, SF_MAX_K), V);

    // ---- 1. maximum, then the sum of the exponentials
    float best = -INFINITY;
    for (int i = tid; i < V; i += SF_THREADS) best = fmaxf(best, __fmul_rn(row[i], it));
    best = wave_max(best);
    if (lane == 0) s_max[wave] = best;
    __syncthreads();
    float smax = s_max[0];
#pragma unroll
    for (int w = 1; w < SF_WAVES; ++w) smax = fmaxf(smax, s_max[w]);
    unsigned kept_bits[KEEP ? SF_KEEP : 1];
    float part = 0.f;
    if (KEEP) {
#pragma unroll
        for (int e = 0; e < SF_KEEP; ++e) {
            const int i = tid + e * SF_THREADS;
            const float p = i < V ? sf_prob(row[i], it, smax) : 0.f;
            kept_bits[KEEP ? e : 0] = i < V ? __float_as_uint(p) : 0xFFFFFFFFu;          // (no probability has these bits)
            part += p;
        }
    } else {
        unsigned* mine = stash ? stash + (size_t)r * V : nullptr;
        for (int i = tid; i < V; i += SF_THREADS) {
            const float p = sf_prob(row[i], it, smax);
            if (mine) mine[i] = __float_as_uint(p);
            part += p;
        }
    }
    const float total = block_sum<SF_WAVES>(part, red);               // (its barriers also order the stash's writes before the reads below: every thread reads what it wrote)
    const unsigned* stashed = (!KEEP && stash) ? stash + (size_t)r * V : nullptr;
    auto bits_at = [&](int e, int i) -> unsigned {
        if (KEEP) return kept_bits[KEEP ? e : 0];
        return stashed ? stashed[i] : __float_as_uint(sf_prob(row[i], it, smax));
    };

    // ---- 2. the bits of the k-th largest probability: eight passes of four bits.  Every lane counts its
    // elements of each of sixteen values in registers (most probabilities share their leading bits: a
    // histogram in LDS would serialise on a few bins); the counts are added over the wave, then over
    // the waves by one thread.
    if (tid == 0) { s_prefix = 0u; s_remaining = (unsigned)k; }
    __syncthreads();
    unsigned known = 0u;                                                   // mask of the bits fixed so far
    const int n_elems = (V + SF_THREADS - 1) / SF_THREADS;
    for (int shift = 28; shift >= 0; shift -= 4) {
        const unsigned prefix = s_prefix;
        // sixteen counters of eight bits in two 64-bit words per lane (a lane sees at most 255 elements
        // in a pass), unpacked and added over the wave at the end of the pass
        unsigned long long c_lo = 0ull, c_hi = 0ull;
        auto count = [&](unsigned bits, bool valid) {
            const bool hit = valid && (bits & known) == prefix;
            const unsigned d = (bits >> shift) & 15u;
            const unsigned long long inc = 1ull << ((d & 7u) * 8u);
            c_lo += (hit && d < 8u) ? inc : 0ull;
            c_hi += (hit && d >= 8u) ? inc : 0ull;
        };
        if (KEEP) {
#pragma unroll
            for (int e = 0; e < SF_KEEP; ++e)
                if (e < n_elems) count(kept_bits[KEEP ? e : 0], tid + e * SF_THREADS < V);
        } else {
            int e = 0;
            for (; e + 4 <= n_elems; e += 4) {                              // four loads in flight
                unsigned v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int i = tid + (e + u) * SF_THREADS;
                    v[u] = i < V ? bits_at(e + u, i) : 0u;
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) count(v[u], tid + (e + u) * SF_THREADS < V);
            }
            for (; e < n_elems; ++e) {
                const int i = tid + e * SF_THREADS;
                count(i < V ? bits_at(e, i) : 0u, i < V);
            }
        }
#pragma unroll
        for (int b = 0; b < 16; ++b) {
            unsigned c = (unsigned)(((b < 8 ? c_lo : c_hi) >> ((b & 7) * 8)) & 255ull);
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
            if (lane == 0) bins[wave][b] = c;
        }
        __syncthreads();
        if (tid == 0) {
            unsigned above = 0u, remaining = s_remaining;
            int b = 15;
            for (; b > 0; --b) {
                unsigned h = 0u;
                for (int w = 0; w < SF_WAVES; ++w) h += bins[w][b];
                if (above + h >= remaining) break;
                above += h;
            }
            s_prefix = prefix | ((unsigned)b << shift);
            s_remaining = remaining - above;                               // how many of this bin are still wanted
        }
        known |= 15u << shift;
        __syncthreads();
    }
    const unsigned kth = s_prefix;
    const int n_equal = (int)s_remaining;                                  // candidates equal to the k-th: the first by index
    const int n_greater = k - n_equal;

    // ---- 3. the candidates: keys of (bits of p, complement of the index), larger first.  Those equal to
    // the k-th are taken in index order: element i = tid + e * SF_THREADS, so place e by place e the
    // threads' counts are scanned (few elements are equal: the scan runs over the places that have any).
    if (tid == 0) s_count = 0u;
    int n_mine = 0;                                                        // my elements equal to the k-th
    for (int e = 0; e < n_elems; ++e) {
        const int i = tid + e * SF_THREADS;
        n_mine += i < V && (KEEP ? kept_bits[KEEP ? min(e, SF_KEEP - 1) : 0] : bits_at(e, i)) == kth;
    }
    per_thread[tid] = n_mine;
    __syncthreads();
    // (usually all elements equal to the k-th are wanted: then their order does not matter)
    int all_equal = 0;
    for (int t = lane; t < SF_THREADS; t += 64) all_equal += per_thread[t];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) all_equal += __shfl_xor(all_equal, o, 64);
    const bool take_all = all_equal == n_equal;
    __syncthreads();
    int base_rank = 0;
    for (int e = 0; e < n_elems; ++e) {
        const int i = tid + e * SF_THREADS;
        const unsigned bits = i < V ? (KEEP ? kept_bits[KEEP ? min(e, SF_KEEP - 1) : 0] : bits_at(e, i)) : 0u;
        if (i < V && (bits > kth || (take_all && bits == kth))) {
            const unsigned at = atomicAdd(&s_count, 1u);
            if (at < SF_MAX_K) cand[at] = ((unsigned long long)bits << 32) | (unsigned long long)(0xFFFFFFFFu - (unsigned)i);
        }
        if (take_all) continue;
        // more elements equal the k-th than are wanted: the first by index, place by place
        const bool eq = i < V && bits == kth;
        if (__syncthreads_or(eq) && base_rank < n_equal) {
            // ranks of this place's equal elements, in the order of the threads (which is index order)
            const unsigned long long m = __ballot(eq);
            const int in_wave = __popcll(m & ((1ull << lane) - 1ull));
            if (lane == 0) per_thread[wave] = __popcll(m);
            __syncthreads();
            int before = 0, all = 0;
            for (int w = 0; w < SF_WAVES; ++w) { const int c = per_thread[w]; before += w < wave ? c : 0; all += c; }
            const int rank = base_rank + before + in_wave;
            if (eq && rank < n_equal)
                cand[n_greater + rank] = ((unsigned long long)kth << 32) | (unsigned long long)(0xFFFFFFFFu - (unsigned)i);
            base_rank += all;
            __syncthreads();
        }
    }
    int P = 1;
    while (P < k) P <<= 1;
    for (int i = k + tid; i < P; i += SF_THREADS) cand[i] = 0ull;          // padding sorts to the end
    __syncthreads();
    for (int size = 2; size <= P; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int t = tid; t < (P >> 1); t += SF_THREADS) {
                const int i = 2 * t - (t & (stride - 1));                  // lower index of the pair
                const int j = i + stride;
                const bool descending = (i & size) == 0;
                const unsigned long long a = cand[i], b = cand[j];
                if ((a < b) == descending) { cand[i] = b; cand[j] = a; }
            }
            __syncthreads();
        }
    }

    // ---- 4. the walk over the sorted candidates.  Thread t owns candidates [2 t, 2 t + 2) and adds them
    // in order; the threads' sums are added in order by one thread (a probability is p / total, as the
    // host forms it; the host adds one by one, so a draw on a boundary may fall to a neighbour).
    constexpr int PER = SF_MAX_K / SF_THREADS;
    float q[PER];
    float local = 0.f;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const int i = tid * PER + e;
        q[e] = i < k ? __uint_as_float((unsigned)(cand[i] >> 32)) / total : 0.f;
        local += q[e];
    }
    sums[tid] = local;
    if (tid == 0) { s_end = k; s_pick = k - 1; }
    __syncthreads();
    if (tid == 0) {
        float run = 0.f;
        const int used = (k + PER - 1) / PER;
        for (int t = 0; t < used; ++t) { const float c = sums[t]; sums[t] = run; run += c; }
    }
    __syncthreads();
    const float before = sums[tid];                                        // sum of the candidates before mine (threads that hold any)
    if (has_tp) {
        float cum = before;
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            cum += q[e];
            if (tid * PER + e < k && cum >= tp) { atomicMin(&s_end, tid * PER + e + 1); break; }
        }
        __syncthreads();
    }
    if (has_mp) {
        const float thr = __uint_as_float((unsigned)(cand[0] >> 32)) / total * mp;
        const int end = s_end;
        __syncthreads();
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int i = tid * PER + e;
            if (i < end && q[e] < thr) { atomicMin(&s_end, max(i, 1)); break; }
        }
        __syncthreads();
    }
    const int end = s_end;
    {   // the sum of the kept ones is the running sum behind the last of them
        float cum = before;
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            cum += q[e];
            if (tid * PER + e == end - 1) s_kept = cum;
        }
    }
    if (tid == 0) s_pick = end - 1;
    __syncthreads();
    const float target = uniform[r] * s_kept;
    {
        float cum = before;
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            cum += q[e];
            if (tid * PER + e < end && cum >= target) { atomicMin(&s_pick, tid * PER + e); break; }
        }
    }
    __syncthreads();
    if (tid == 0) out[r] = (int)(0xFFFFFFFFu - (unsigned)(cand[s_pick] & 0xFFFFFFFFull));
}

// Rows with a filter (top_k[r] >= 1, 0 < top_p[r] < 1 or min_p[r] > 0) and inv_temp[r] > 0 are drawn
// here; the others are not touched (fl_sample draws them).  top_k travels as a float (exact below 2^24);
// more than 2048 candidates are not kept: the caller sends such rows to the host sampler.  A vocabulary
// beyond 32,768 is read ten times: with `stash` (rows * V values, or null) the probabilities are formed
// once and kept there.
extern "C" int fl_sample_filtered(const float* logits, const float* inv_temp, const float* uniform,
                                  const float* top_k, const float* top_p, const float* min_p, int* out,
                                  int rows, int V, unsigned* stash, hipStream_t stream) {
    FL_CHECK(rows >= 0 && V > 0, "sample_filtered: bad sizes");
    FL_CHECK(V <= 255 * SF_THREADS, "sample_filtered: a vocabulary of %d, at most %d", V, 255 * SF_THREADS);
    FL_CHECK(logits && inv_temp && uniform && top_k && top_p && min_p && out, "sample_filtered: needs all its arrays");
    if (rows == 0) return 0;
    if (V <= SF_KEEP * SF_THREADS)
        sample_filtered_kernel<true><<<rows, SF_THREADS, 0, stream>>>(logits, inv_temp, uniform, top_k, top_p, min_p, out, V, nullptr);
    else
        sample_filtered_kernel<false><<<rows, SF_THREADS, 0, stream>>>(logits, inv_temp, uniform, top_k, top_p, min_p, out, V, stash);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_sample_filtered)

extern "C" int fl_sample_filtered_max_k(void) { return SF_MAX_K; }
extern "C" int fl_sample_filtered_max_vocab(void) { return 255 * SF_THREADS; }

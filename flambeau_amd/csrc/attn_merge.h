// Merge of attention computed over splits of the keys: every split s of a (query row, head) left
// its unnormalised output part_o[base + s][hdp] (relative to its own maximum), that maximum and its
// sum of exponentials in part_ml[base + s] = (m_s, l_s) (natural-log units; m_s = -inf for a split
// without keys).  out[d] = sum_s part_o[s][d] e^(m_s - m) / sum_s l_s e^(m_s - m), m = max m_s.  One
// block of 256 threads per (row, head): the pairs are read by one thread each, then every thread
// owns head dims and adds the splits' outputs, loads issued eight at a time.  The order of the sums
// is fixed (rising split).
#pragma once
#include "common.h"

// Split s lies in slot base + s * stride.
__device__ __forceinline__ void attn_merge_splits(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                  bf16_t* __restrict__ out_row, size_t base, int hd, int hdp, int n_split,
                                                  size_t stride = 1) {
    __shared__ float s_f[256];       // exp(m_s - m_max) per split (n_split <= 256)
    __shared__ float s_l[256];
    __shared__ float s_inv;
    const int t = threadIdx.x;
    float ms = -INFINITY, ls = 0.f;
    if (t < n_split) {
        ms = part_ml[(base + t * stride) * 2];
        ls = part_ml[(base + t * stride) * 2 + 1];
    }
    s_f[t] = ms;
    __syncthreads();
    float mm = -INFINITY;
    for (int s = 0; s < n_split; ++s) mm = fmaxf(mm, s_f[s]);
    __syncthreads();
    const float f = ms == -INFINITY ? 0.f : expf(ms - mm);
    s_f[t] = f;
    // sum of l_s f_s in rising s, by thread 0 after everyone has written its factor
    s_l[t] = ls * f;
    __syncthreads();
    if (t == 0) {
        float ll = 0.f;
        for (int s = 0; s < n_split; ++s) ll += s_l[s];
        s_inv = ll > 0.f ? 1.0f / ll : 0.f;
    }
    __syncthreads();
    const float inv = s_inv;
    for (int d = t; d < hd; d += blockDim.x) {
        float acc = 0.f;
        int s = 0;
        for (; s + 8 <= n_split; s += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part_o[(base + (s + u) * stride) * hdp + d];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u] * s_f[s + u];
        }
        for (; s < n_split; ++s) acc += part_o[(base + s * stride) * hdp + d] * s_f[s];
        out_row[d] = (bf16_t)(acc * inv);
    }
}

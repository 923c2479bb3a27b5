// A kernel that only a test knows: the activation of its toy feed-forward.
//   out[i] = h[i] * sigmoid(alpha * h[i]),  h 32-bit, out 32-bit or bfloat16 (rounded to nearest even).
// The launch function has the shape the framework's own have (pointers, int, long, float, the stream
// last; 0 or an error code), and the library exports a trampoline for it, so that a recorded step can
// replay the launch with the arguments it was first called with.
#include <hip/hip_runtime.h>
#include "recordable.h"

__global__ void toy_temper_kernel(const float* __restrict__ h, void* __restrict__ out, int out_bf16, long n, float alpha) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = h[i];
    float y = v / (1.0f + __expf(-alpha * v));
    if (out_bf16) {
        unsigned u = __float_as_uint(y);
        u += 0x7fffu + ((u >> 16) & 1u);
        ((unsigned short*)out)[i] = (unsigned short)(u >> 16);
    } else {
        ((float*)out)[i] = y;
    }
}

extern "C" int toy_temper(const float* h, void* out, int out_bf16, long n, float alpha, hipStream_t stream) {
    if (n < 0 || n > (1L << 31)) return 1;
    if (n == 0) return 0;
    hipLaunchKernelGGL(toy_temper_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, h, out, out_bf16, n, alpha);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

extern "C" int toy_temper_replay(const FlArg* args, hipStream_t stream) {
    return fl_rec::Tramp<&toy_temper>::call(args, stream);
}

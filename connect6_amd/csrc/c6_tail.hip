// HBM-bound kernels around the fused forward: stand-alone occupied-square
// masking, masked softmax + inverse-CDF sampling, and the D4 view gather /
// inverse-map-and-average.  Each streams its operands once.
#include "c6_common.h"
#include "c6_device.h"

namespace c6 {

// out = legal ? logits : fill   (connect6/model.py:123-125 of the reference)
// 4-byte elements, four per thread through 16-byte accesses, scalar tail.
__global__ void mask4_kernel(const uint32_t *__restrict__ in, const uint8_t *__restrict__ legal,
                             long long n, uint32_t fill, uint32_t *__restrict__ out) {
  const long long nv = n >> 2;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
    const v4i v = reinterpret_cast<const v4i *>(in)[i];
    const uint32_t m = reinterpret_cast<const uint32_t *>(legal)[i];
    v4i o;
    o[0] = (m & 0x000000ffu) ? v[0] : (int)fill;
    o[1] = (m & 0x0000ff00u) ? v[1] : (int)fill;
    o[2] = (m & 0x00ff0000u) ? v[2] : (int)fill;
    o[3] = (m & 0xff000000u) ? v[3] : (int)fill;
    reinterpret_cast<v4i *>(out)[i] = o;
  }
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
    const long long i = (nv << 2) + threadIdx.x;
    out[i] = legal[i] ? in[i] : fill;
  }
}

// 2-byte elements, eight per thread.
__global__ void mask2_kernel(const uint16_t *__restrict__ in, const uint8_t *__restrict__ legal,
                             long long n, uint16_t fill, uint16_t *__restrict__ out) {
  const long long nv = n >> 3;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
    const v4i v = reinterpret_cast<const v4i *>(in)[i];
    const v2i m = reinterpret_cast<const v2i *>(legal)[i];
    v4i o;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t mm = (uint32_t)m[w >> 1] >> ((w & 1) * 16);
      const uint32_t lo = (mm & 0x00ffu) ? ((uint32_t)v[w] & 0xffffu) : (uint32_t)fill;
      const uint32_t hi = (mm & 0xff00u) ? ((uint32_t)v[w] >> 16) : (uint32_t)fill;
      o[w] = (int)(lo | (hi << 16));
    }
    reinterpret_cast<v4i *>(out)[i] = o;
  }
  if (blockIdx.x == 0 && threadIdx.x < (n & 7)) {
    const long long i = (nv << 3) + threadIdx.x;
    out[i] = legal[i] ? in[i] : fill;
  }
}

// One wave per board: masked softmax over 361 logits and inverse-CDF draw
// (connect6/train.py:195-213 of the reference, with the uniform supplied).
__global__ __launch_bounds__(256) void sample_kernel(const float *__restrict__ logits,
                                                     const uint8_t *__restrict__ legal,
                                                     const float *__restrict__ u,
                                                     float inv_temperature, long long batch,
                                                     long long *__restrict__ actions,
                                                     float *__restrict__ logprob) {
  const int lane = threadIdx.x & 63;
  const long long b = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= batch) return;
  const float *row = logits + (size_t)b * kPix;
  const uint8_t *lrow = legal ? legal + (size_t)b * kPix : nullptr;
  int a;
  float lp;
  wave_sample(
      lane, u[b], [&](int i) { return row[i] * inv_temperature; },
      [&](int i) { return lrow ? lrow[i] != 0 : true; }, a, lp);
  if (lane == 0) {
    actions[b] = a;
    if (logprob) logprob[b] = lp;
  }
}

// out[p,b,ch,v] = x[b,ch,from_view(v,p)]   (connect6/train.py:222-230)
template <typename T>
__global__ void d4_expand_kernel(const T *__restrict__ x, long long batch, T *__restrict__ out) {
  const long long per_view = batch * 3 * kPix;
  const long long n = 8 * per_view;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int p = (int)(i / per_view);
    const long long rem = i - (long long)p * per_view;
    const long long plane = rem / kPix;
    const int v = (int)(rem - plane * kPix);
    out[i] = x[plane * kPix + d4_from_view(v, p)];
  }
}

// logits[b,a] = mean_p view_logits[p,b,to_view(a,p)]; values[b] = mean_p view_values[p,b]
__global__ void d4_reduce_kernel(const float *__restrict__ vl, const float *__restrict__ vv,
                                 long long batch, float *__restrict__ logits,
                                 float *__restrict__ values) {
  const long long n = batch * kPix;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const long long b = i / kPix;
    const int a = (int)(i - b * kPix);
    float s = 0.0f;
#pragma unroll
    for (int p = 0; p < 8; ++p) s += vl[((size_t)p * batch + b) * kPix + d4_to_view(a, p)];
    logits[i] = s * 0.125f;
    if (a == 0 && values != nullptr) {
      float t = 0.0f;
#pragma unroll
      for (int p = 0; p < 8; ++p) t += vv[(size_t)p * batch + b];
      values[b] = t * 0.125f;
    }
  }
}

static int check_launch(const char *what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s launch failed: %s", what, hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  return C6_OK;
}

static unsigned grid_for(long long work_items, int threads) {
  long long blocks = (work_items + threads - 1) / threads;
  const long long cap = 256LL * 32;  // 32 resident blocks per CU is plenty for a streaming kernel
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

int launch_mask(const void *logits, const uint8_t *legal, int elem_bytes, long long n,
                uint32_t fill_bits, void *out, hipStream_t st) {
  if (elem_bytes == 4) {
    hipLaunchKernelGGL(mask4_kernel, dim3(grid_for((n >> 2) + 1, 256)), dim3(256), 0, st,
                       (const uint32_t *)logits, legal, n, fill_bits, (uint32_t *)out);
  } else {
    hipLaunchKernelGGL(mask2_kernel, dim3(grid_for((n >> 3) + 1, 256)), dim3(256), 0, st,
                       (const uint16_t *)logits, legal, n, (uint16_t)fill_bits, (uint16_t *)out);
  }
  return check_launch("mask_logits");
}

int launch_sample(const float *logits, const uint8_t *legal, const float *u, float inv_t,
                  long long batch, long long *actions, float *logprob, hipStream_t st) {
  hipLaunchKernelGGL(sample_kernel, dim3((unsigned)((batch + 3) / 4)), dim3(256), 0, st, logits,
                     legal, u, inv_t, batch, actions, logprob);
  return check_launch("softmax_sample");
}

int launch_d4_expand(const void *x, int elem_bytes, long long batch, void *out, hipStream_t st) {
  const long long n = 8 * batch * 3 * kPix;
  if (elem_bytes == 4)
    hipLaunchKernelGGL(d4_expand_kernel<uint32_t>, dim3(grid_for(n, 256)), dim3(256), 0, st,
                       (const uint32_t *)x, batch, (uint32_t *)out);
  else
    hipLaunchKernelGGL(d4_expand_kernel<uint16_t>, dim3(grid_for(n, 256)), dim3(256), 0, st,
                       (const uint16_t *)x, batch, (uint16_t *)out);
  return check_launch("d4_expand");
}

int launch_d4_reduce(const float *vl, const float *vv, long long batch, float *logits,
                     float *values, hipStream_t st) {
  hipLaunchKernelGGL(d4_reduce_kernel, dim3(grid_for(batch * kPix, 256)), dim3(256), 0, st, vl, vv,
                     batch, logits, values);
  return check_launch("d4_reduce");
}

}  // namespace c6

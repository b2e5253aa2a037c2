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
    stream_store(&reinterpret_cast<v4i *>(out)[i], o);
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
    stream_store(&reinterpret_cast<v4i *>(out)[i], o);
  }
  if (blockIdx.x == 0 && threadIdx.x < (n & 7)) {
    const long long i = (nv << 3) + threadIdx.x;
    out[i] = legal[i] ? in[i] : fill;
  }
}

// One element per thread, for operands that are only element-aligned (a row slice such as
// logits[1:] starts 1444 bytes into its tensor).
template <typename T>
__global__ void mask_elem_kernel(const T *__restrict__ in, const uint8_t *__restrict__ legal,
                                 long long n, T fill, T *__restrict__ out) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = legal[i] ? in[i] : fill;
}

// Rows of 361 elements are only 4-byte aligned, but FOUR consecutive rows span 4*361*4 =
// 16*361 bytes and start 16-byte aligned (the tensor base is).  The kernels below therefore
// work on groups of four boards (32 planes for the view gather) and move them with 16-byte
// accesses; the last, partial group falls back to element accesses.

// Four boards per group (one per wave): masked softmax over 361 logits and inverse-CDF draw
// (connect6/train.py:195-213 of the reference, with the uniform supplied).  A workgroup walks
// over groups; while it works on one group out of LDS, the next group's rows are already on
// their way into registers, so that every CU always has reads in flight.  Small groups and many
// more workgroups than fit the chip at once (each takes about four groups) measured best: eight
// boards per group on exactly the resident number of workgroups took 118 us for 262,144 boards,
// this shape 98 us; one group per workgroup, with nothing fetched ahead, 112 us.
constexpr int kSampleBoards = 4;
__global__ __launch_bounds__(256) void sample_kernel(const float *__restrict__ logits,
                                                     const uint8_t *__restrict__ legal,
                                                     const float *__restrict__ u,
                                                     float inv_temperature, long long batch,
                                                     long long *__restrict__ actions,
                                                     float *__restrict__ logprob) {
  __shared__ __attribute__((aligned(16))) float s_logit[kSampleBoards * kPix];
  __shared__ __attribute__((aligned(16))) uint8_t s_legal[kSampleBoards * kPix];
  constexpr int NV = kSampleBoards * kPix / 4;       // 16-byte units of a group's logits (722)
  constexpr int NL = kSampleBoards * kPix / 4;       // 4-byte units of its legality bytes (361)
  constexpr int RV = (NV + 255) / 256, RL = (NL + 255) / 256;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const bool masked = legal != nullptr;
  const bool vec = (reinterpret_cast<uintptr_t>(logits) & 15u) == 0 &&
                   (!masked || (reinterpret_cast<uintptr_t>(legal) & 3u) == 0);
  const long long groups = (batch + kSampleBoards - 1) / kSampleBoards;
  f32x4 pv[RV];
  int pl[RL];
  // a full group with aligned operands travels through registers; anything else is copied
  // element by element when its turn comes
  auto prefetch = [&](long long g) {
    const long long b0 = g * kSampleBoards;
    if (g < groups && vec && batch - b0 >= kSampleBoards) {
#pragma unroll
      for (int r = 0; r < RV; ++r) {
        const int i = threadIdx.x + r * 256;
        if (i < NV) pv[r] = reinterpret_cast<const f32x4 *>(logits + (size_t)b0 * kPix)[i];
      }
      if (masked) {
#pragma unroll
        for (int r = 0; r < RL; ++r) {
          const int i = threadIdx.x + r * 256;
          if (i < NL) pl[r] = reinterpret_cast<const int *>(legal + (size_t)b0 * kPix)[i];
        }
      }
    }
  };
  long long g = blockIdx.x;
  prefetch(g);
  for (; g < groups; g += gridDim.x) {
    const long long b0 = g * kSampleBoards;
    const int nb = (int)(batch - b0 < kSampleBoards ? batch - b0 : kSampleBoards);
    if (vec && nb == kSampleBoards) {
#pragma unroll
      for (int r = 0; r < RV; ++r) {
        const int i = threadIdx.x + r * 256;
        if (i < NV) reinterpret_cast<f32x4 *>(s_logit)[i] = pv[r];
      }
      if (masked) {
#pragma unroll
        for (int r = 0; r < RL; ++r) {
          const int i = threadIdx.x + r * 256;
          if (i < NL) reinterpret_cast<int *>(s_legal)[i] = pl[r];
        }
      }
    } else {
      for (int i = threadIdx.x; i < nb * kPix; i += blockDim.x) {
        s_logit[i] = logits[(size_t)b0 * kPix + i];
        if (masked) s_legal[i] = legal[(size_t)b0 * kPix + i];
      }
    }
    __syncthreads();
    prefetch(g + gridDim.x);
#pragma unroll
    for (int r = 0; r < kSampleBoards / 4; ++r) {
      const int bl = w + 4 * r;
      if (bl < nb) {
        const float *row = s_logit + bl * kPix;
        const uint8_t *lrow = s_legal + bl * kPix;
        int a;
        float lp;
        wave_sample(
            lane, u[b0 + bl], inv_temperature, [&](int i) { return row[i]; },
            [&](int i) { return masked ? lrow[i] != 0 : true; }, a, lp);
        if (lane == 0) {
          actions[b0 + bl] = a;
          if (logprob) logprob[b0 + bl] = lp;
        }
      }
    }
    __syncthreads();  // the rows are consumed: the next group may overwrite them
  }
}

// out[p,plane,v] = x[plane, from_view(v,p)]   (connect6/train.py:222-230)
// Each workgroup stages 32 planes in LDS once and writes all eight permuted views of them, one
// view after the other: the input is read once, every output element is one LDS gather, stores
// are 16 bytes, and a workgroup's share of a view is one contiguous run of 46,208 bytes (4-byte
// elements) = 361 whole 128-byte lines.  The run length is what the store side is sensitive to:
// with 8 planes per workgroup (11.5 KB runs) the same stores alone, with nothing read, take
// 13 % longer.
constexpr int kExpandPlanes = 32;
constexpr int kExpandThreads = 512;
template <typename T>
__global__ __launch_bounds__(kExpandThreads) void d4_expand_kernel(const T *__restrict__ x,
                                                                   long long planes,
                                                                   T *__restrict__ out) {
  constexpr int VEC = 16 / sizeof(T);                       // elements per 16-byte access
  constexpr int SPAN = kExpandPlanes * kPix;                // 11552 elements: a multiple of VEC
  static_assert(SPAN % VEC == 0, "a group of planes must be whole 16-byte units");
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  __shared__ __attribute__((aligned(16))) T s_in[SPAN];
  const long long plane0 = (long long)blockIdx.x * kExpandPlanes;
  const int np = (int)((planes - plane0) < kExpandPlanes ? (planes - plane0) : kExpandPlanes);
  const T *src = x + plane0 * kPix;
  T *dst0 = out + plane0 * kPix;                              // view p adds p * planes * kPix
  const size_t view_stride = (size_t)planes * kPix;
  const bool aligned = np == kExpandPlanes &&
                       ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst0) |
                         (view_stride * sizeof(T))) & 15u) == 0;
  if (aligned) {
    for (int i = threadIdx.x; i < SPAN / VEC; i += kExpandThreads)
      reinterpret_cast<vec_t *>(s_in)[i] = reinterpret_cast<const vec_t *>(src)[i];
  } else {
    for (int i = threadIdx.x; i < np * kPix; i += kExpandThreads) s_in[i] = src[i];
  }
  __syncthreads();
  if (aligned) {
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      for (int i = threadIdx.x; i < SPAN / VEC; i += kExpandThreads) {
        vec_t o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const int idx = i * VEC + e;
          const int pl = idx / kPix, v = idx - pl * kPix;
          o[e] = s_in[pl * kPix + d4_from_view(v, p)];
        }
        reinterpret_cast<vec_t *>(dst0 + p * view_stride)[i] = o;
      }
    }
  } else {
    for (int i = threadIdx.x; i < np * kPix; i += kExpandThreads) {
      const int pl = i / kPix, v = i - pl * kPix;
#pragma unroll
      for (int p = 0; p < 8; ++p) dst0[p * view_stride + i] = s_in[pl * kPix + d4_from_view(v, p)];
    }
  }
}

// logits[b,a] = mean_p view_logits[p,b,to_view(a,p)]; values[b] = mean_p view_values[p,b]
// Four boards per workgroup; the eight views stream through a double buffer in LDS (the next
// view's rows are in flight while the current one is gathered), accumulators stay in registers.
__global__ __launch_bounds__(256) void d4_reduce_kernel(const float *__restrict__ vl,
                                                        const float *__restrict__ vv,
                                                        long long batch,
                                                        float *__restrict__ logits,
                                                        float *__restrict__ values) {
  constexpr int SPAN = 4 * kPix;            // 1444 floats = 361 16-byte units
  constexpr int PER = (SPAN + 255) / 256;   // outputs per thread
  __shared__ __attribute__((aligned(16))) float s_v[2][SPAN];
  const long long b0 = (long long)blockIdx.x * 4;
  const int nb = (int)(batch - b0 < 4 ? batch - b0 : 4);
  const int n = nb * kPix;
  const bool vec = nb == 4 && (batch & 3) == 0 && (reinterpret_cast<uintptr_t>(vl) & 15u) == 0;
  const int t = threadIdx.x;
  f32x4 stage[2];
  float stage1[PER];
  auto fetch = [&](int p) {
    const float *src = vl + ((size_t)p * batch + b0) * kPix;
    if (vec) {
      stage[0] = reinterpret_cast<const f32x4 *>(src)[t];
      if (t + 256 < kPix) stage[1] = reinterpret_cast<const f32x4 *>(src)[t + 256];
    } else {
#pragma unroll
      for (int k = 0; k < PER; ++k)
        if (t + 256 * k < n) stage1[k] = src[t + 256 * k];
    }
  };
  auto commit = [&](int buf) {
    if (vec) {
      reinterpret_cast<f32x4 *>(s_v[buf])[t] = stage[0];
      if (t + 256 < kPix) reinterpret_cast<f32x4 *>(s_v[buf])[t + 256] = stage[1];
    } else {
#pragma unroll
      for (int k = 0; k < PER; ++k)
        if (t + 256 * k < n) s_v[buf][t + 256 * k] = stage1[k];
    }
  };
  int bl[PER], a[PER];
  float acc[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = t + 256 * k;
    bl[k] = i / kPix;
    a[k] = i - bl[k] * kPix;
    acc[k] = 0.0f;
  }
  fetch(0);
  commit(0);
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    if (p < 7) fetch(p + 1);
#pragma unroll
    for (int k = 0; k < PER; ++k)
      if (t + 256 * k < n) acc[k] += s_v[p & 1][bl[k] * kPix + d4_to_view(a[k], p)];
    if (p < 7) commit((p + 1) & 1);
    __syncthreads();
  }
  float *dst = logits + (size_t)b0 * kPix;
#pragma unroll
  for (int k = 0; k < PER; ++k)
    if (t + 256 * k < n) dst[t + 256 * k] = acc[k] * 0.125f;
  if (t < nb && values != nullptr) {
    float s = 0.0f;
#pragma unroll
    for (int p = 0; p < 8; ++p) s += vv[(size_t)p * batch + b0 + t];
    values[b0 + t] = s * 0.125f;
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
  const bool vec = ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0 &&
                   (reinterpret_cast<uintptr_t>(legal) & 7u) == 0;
  if (!vec) {
    if (elem_bytes == 4)
      hipLaunchKernelGGL(mask_elem_kernel<uint32_t>, dim3(grid_for(n, 256)), dim3(256), 0, st,
                         (const uint32_t *)logits, legal, n, fill_bits, (uint32_t *)out);
    else
      hipLaunchKernelGGL(mask_elem_kernel<uint16_t>, dim3(grid_for(n, 256)), dim3(256), 0, st,
                         (const uint16_t *)logits, legal, n, (uint16_t)fill_bits, (uint16_t *)out);
    return check_launch("mask_logits");
  }
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
  const long long groups = (batch + kSampleBoards - 1) / kSampleBoards;
  const long long resident = 256LL * 64;  // (eight workgroups of 256 threads fit a CU at a time; see the kernel)
  hipLaunchKernelGGL(sample_kernel, dim3((unsigned)(groups < resident ? groups : resident)), dim3(256), 0, st, logits,
                     legal, u, inv_t, batch, actions, logprob);
  return check_launch("softmax_sample");
}

int launch_d4_expand(const void *x, int elem_bytes, long long batch, void *out, hipStream_t st) {
  const long long planes = batch * 3;
  const dim3 grid((unsigned)((planes + kExpandPlanes - 1) / kExpandPlanes));
  if (elem_bytes == 4)
    hipLaunchKernelGGL(d4_expand_kernel<uint32_t>, grid, dim3(kExpandThreads), 0, st,
                       (const uint32_t *)x, planes, (uint32_t *)out);
  else
    hipLaunchKernelGGL(d4_expand_kernel<uint16_t>, grid, dim3(kExpandThreads), 0, st,
                       (const uint16_t *)x, planes, (uint16_t *)out);
  return check_launch("d4_expand");
}

int launch_d4_reduce(const float *vl, const float *vv, long long batch, float *logits,
                     float *values, hipStream_t st) {
  hipLaunchKernelGGL(d4_reduce_kernel, dim3((unsigned)((batch + 3) / 4)), dim3(256), 0, st, vl, vv,
                     batch, logits, values);
  return check_launch("d4_reduce");
}

}  // namespace c6

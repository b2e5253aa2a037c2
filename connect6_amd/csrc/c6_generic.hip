// Layer-by-layer forward for ANY architecture the reference's PolicyValueNet accepts
// (connect6/model.py:26-77: any board size, any odd kernels, any channel counts).
// This is the compatibility path: plain direct convolution, one thread per output
// element, activations round-tripping through a caller-provided workspace.  The fused
// MFMA kernel in c6_forward.hip serves the default architecture.
#include <mutex>

#include "c6_common.h"

namespace c6 {

// Workspace of c6_forward_generic_static: callers that may not allocate device memory (code
// under HIP graph capture, serving loops, harnesses that forbid hipMalloc) run the generic
// forward through this array instead of a workspace of their own.  Every GPU the library runs
// on holds its own copy until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress: the per-device address it returns is what kernels receive.
constexpr size_t kStaticScratchBytes = size_t(16) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

size_t static_scratch_bytes() { return kStaticScratchBytes; }

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void **out) {
  constexpr int kMaxDevices = 64;
  static std::mutex lock;
  static void *addr[kMaxDevices] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("static scratch: no usable current device (%s, device %d)", hipGetErrorString(e), dev);
    return C6_ELAUNCH;
  }
  std::lock_guard<std::mutex> guard(lock);
  if (addr[dev] == nullptr) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error("static scratch: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return C6_ELAUNCH;
    }
    addr[dev] = ptr;
  }
  *out = addr[dev];
  return C6_OK;
}

__device__ __forceinline__ float round_to(float v, int mode) {
  if (mode == C6_DT_BF16) return (float)(__bf16)v;
  if (mode == C6_DT_F16) return (float)(_Float16)v;
  return v;
}

__device__ __forceinline__ float load_any(const void *x, int dt, size_t i) {
  if (dt == C6_DT_F32) return reinterpret_cast<const float *>(x)[i];
  const unsigned short b = reinterpret_cast<const unsigned short *>(x)[i];
  if (dt == C6_DT_BF16) return __builtin_bit_cast(float, (unsigned)b << 16);
  return (float)__builtin_bit_cast(_Float16, b);
}

// out[b,co,r,c] = act(bias[g,co] + sum_{ci,ky,kx} w[g,co,ci,ky,kx] * in[b,ci,r+ky-k/2,c+kx-k/2])
// with g = b / per_group: the weight sets of a group of models lie one after the other
// (connect6/history.py:224-240 stacks them that way) and board b belongs to set g -- one launch
// per layer for the whole ensemble, as the reference's grouped convolution
// (connect6/history.py:263-273).  A single model is per_group = batch.
__global__ void generic_conv_kernel(const void *__restrict__ in, int in_dtype,
                                    const float *__restrict__ w, const float *__restrict__ bias,
                                    float *__restrict__ out, long long batch, long long per_group,
                                    int cin, int cout, int n, int k, int silu, int round_w,
                                    int round_a, int round_out) {
  const long long total = batch * cout * n * n;
  const long long stride = (long long)gridDim.x * blockDim.x;
  const int pad = k / 2;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int c = (int)(i % n);
    const int r = (int)((i / n) % n);
    const int co = (int)((i / ((long long)n * n)) % cout);
    const long long b = i / ((long long)n * n * cout);
    const size_t g = (size_t)(b / per_group);
    float acc = bias ? bias[g * cout + co] : 0.0f;
    for (int ci = 0; ci < cin; ++ci) {
      const size_t plane = ((size_t)b * cin + ci) * n * n;
      const float *wk = w + ((g * cout + co) * cin + ci) * k * k;
      for (int ky = 0; ky < k; ++ky) {
        const int rr = r + ky - pad;
        if (rr < 0 || rr >= n) continue;
        for (int kx = 0; kx < k; ++kx) {
          const int cc = c + kx - pad;
          if (cc < 0 || cc >= n) continue;
          const float a = round_to(load_any(in, in_dtype, plane + (size_t)rr * n + cc), round_a);
          acc = fmaf(round_to(wk[ky * k + kx], round_w), a, acc);
        }
      }
    }
    if (silu) acc = acc / (1.0f + expf(-acc));
    out[i] = round_to(acc, round_out);
  }
}

// one workgroup per board: 1x1 policy head -> masked logits, 1x1 value head -> mean -> tanh
__global__ __launch_bounds__(256) void generic_heads_kernel(
    const float *__restrict__ feat, int channels, int n, const float *__restrict__ pol_w,
    const float *__restrict__ pol_b, const float *__restrict__ val_w,
    const float *__restrict__ val_b, const void *__restrict__ x, int x_dtype, int in_channels,
    int mask_mode, const uint8_t *__restrict__ legal, float fill, float *__restrict__ logits,
    float *__restrict__ value, long long per_group) {
  __shared__ float red[256];
  const long long b = blockIdx.x;
  const size_t g = (size_t)(b / per_group);
  pol_w += g * channels;
  if (val_w) val_w += g * channels;
  const int nn = n * n;
  float vsum = 0.0f;
  for (int p = threadIdx.x; p < nn; p += blockDim.x) {
    float pol = pol_b ? pol_b[g] : 0.0f;
    float val = 0.0f;
    for (int c = 0; c < channels; ++c) {
      const float f = feat[((size_t)b * channels + c) * nn + p];
      pol = fmaf(pol_w[c], f, pol);
      if (val_w) val = fmaf(val_w[c], f, val);
    }
    vsum += val;
    if (logits) {
      bool occupied = false;
      if (mask_mode == C6_MASK_LEGAL) occupied = legal[(size_t)b * nn + p] == 0;
      if (mask_mode == C6_MASK_INPUT)
        occupied = load_any(x, x_dtype, ((size_t)b * in_channels + 0) * nn + p) != 0.0f ||
                   load_any(x, x_dtype, ((size_t)b * in_channels + 1) * nn + p) != 0.0f;
      logits[(size_t)b * nn + p] = occupied ? fill : pol;
    }
  }
  red[threadIdx.x] = vsum;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0 && value != nullptr)
    value[b] = tanhf(red[0] / (float)nn + (val_b ? val_b[g] : 0.0f));
}

static unsigned blocks_for(long long items) {
  long long b = (items + 255) / 256;
  if (b > 256LL * 64) b = 256LL * 64;
  return (unsigned)(b < 1 ? 1 : b);
}

size_t generic_workspace_bytes(long long batch, int n, int layers, const int *channels) {
  int cmax = 1;
  for (int l = 0; l < layers; ++l) cmax = channels[l] > cmax ? channels[l] : cmax;
  return 2 * (size_t)batch * cmax * n * n * sizeof(float);
}

int launch_generic(const void *x, int x_dtype, long long batch, long long per_group, int n,
                   int layers, const int *kernels, const int *channels, const float *const *conv_w,
                   const float *const *conv_b, const float *pol_w, const float *pol_b,
                   const float *val_w, const float *val_b, int prec, void *workspace,
                   float *logits, float *value, int mask_mode, const uint8_t *legal, float fill,
                   hipStream_t st) {
  int cmax = 1;
  for (int l = 0; l < layers; ++l) cmax = channels[l] > cmax ? channels[l] : cmax;
  float *buf[2] = {static_cast<float *>(workspace),
                   static_cast<float *>(workspace) + (size_t)batch * cmax * n * n};
  // arithmetic contract of each mode: which operands are rounded to 16 bits
  // (C6_PREC_BF16F6W carries the weights' low part as well: nothing is rounded)
  const int round_w = (prec == C6_PREC_F32 || prec == C6_PREC_BF16F6W)
                          ? C6_DT_F32
                          : (prec == C6_PREC_F16 ? C6_DT_F16 : C6_DT_BF16);
  // (the hi+lo modes carry the activations' low-order bits: no activation rounding here)
  const int round_a = prec == C6_PREC_BF16 ? C6_DT_BF16 : (prec == C6_PREC_F16 ? C6_DT_F16 : C6_DT_F32);
  const void *in = x;
  int in_dtype = x_dtype;
  int cin = 3;
  for (int l = 0; l < layers; ++l) {
    float *out = buf[l & 1];
    const int last = l + 1 == layers;
    hipLaunchKernelGGL(generic_conv_kernel, dim3(blocks_for(batch * channels[l] * n * n)),
                       dim3(256), 0, st, in, in_dtype, conv_w[l], conv_b ? conv_b[l] : nullptr,
                       out, batch, per_group, cin, channels[l], n, kernels[l], 1, round_w,
                       round_a,
                       last ? C6_DT_F32 : round_a);
    in = out;
    in_dtype = C6_DT_F32;
    cin = channels[l];
  }
  hipLaunchKernelGGL(generic_heads_kernel, dim3((unsigned)batch), dim3(256), 0, st,
                     static_cast<const float *>(in), cin, n, pol_w, pol_b, val_w, val_b, x,
                     x_dtype, 3, mask_mode, legal, fill, logits, value, per_group);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("generic forward launch failed: %s", hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  return C6_OK;
}

}  // namespace c6

// The C ABI without Python: loads libconnect6_amd.so with dlopen, as a foreign-function binding
// would, drives it with plain HIP device pointers, and checks the result against the brute-force
// C oracle (oracle/conv_ref.c, linked into this test binary only).
//
//   c_abi_forward <path to libconnect6_amd.so>      exit status 0 = all checks passed
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "connect6_amd.h"

extern "C" int c6ref_forward(const float *x, long batch, int n, int in_channels, int layers,
                             const int *kernels, const int *channels, const float *conv_w,
                             const float *conv_b, const float *pol_w, const float *pol_b,
                             const float *val_w, const float *val_b, float *logits, float *value);

#define HIP_OK(call)                                                                  \
  do {                                                                                \
    hipError_t e_ = (call);                                                           \
    if (e_ != hipSuccess) {                                                           \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));          \
      return 2;                                                                       \
    }                                                                                 \
  } while (0)

static uint32_t g_state = 20250101u;
static float uniform() {  // [0, 1)
  g_state = g_state * 1664525u + 1013904223u;
  return (float)(g_state >> 8) * (1.0f / 16777216.0f);
}

static double rel_l2(const std::vector<float> &a, const std::vector<float> &b) {
  double num = 0, den = 0;
  for (size_t i = 0; i < a.size(); ++i) {
    num += ((double)a[i] - b[i]) * ((double)a[i] - b[i]);
    den += (double)b[i] * b[i];
  }
  return std::sqrt(num / (den > 0 ? den : 1e-300));
}

int main(int argc, char **argv) {
  if (argc < 2) {
    std::fprintf(stderr, "usage: %s <libconnect6_amd.so>\n", argv[0]);
    return 2;
  }
  void *lib = dlopen(argv[1], RTLD_NOW);
  if (!lib) {
    std::fprintf(stderr, "dlopen: %s\n", dlerror());
    return 2;
  }
  auto p_version = (int (*)(void))dlsym(lib, "c6_version");
  auto p_error = (const char *(*)(void))dlsym(lib, "c6_last_error");
  auto p_bytes = (decltype(&c6_packed_bytes))dlsym(lib, "c6_packed_bytes");
  auto p_pack = (decltype(&c6_pack_weights))dlsym(lib, "c6_pack_weights");
  auto p_forward = (decltype(&c6_forward))dlsym(lib, "c6_forward");
  if (!p_version || !p_error || !p_bytes || !p_pack || !p_forward) {
    std::fprintf(stderr, "missing symbol\n");
    return 2;
  }
  std::printf("c6_version %d\n", p_version());

  const int kernels[8] = {23, 3, 3, 3, 3, 3, 3, 3};
  const int channels[8] = {32, 32, 64, 64, 64, 96, 96, 96};
  const int B = 6, n = C6_BOARD, cells = C6_ACTIONS;

  // parameters: uniform with the variance of a He initialisation, small non-zero biases
  std::vector<std::vector<float>> w(8), b(8);
  std::vector<float> flat_w, flat_b;
  int cin = 3;
  for (int l = 0; l < 8; ++l) {
    const int k = kernels[l];
    const float bound = std::sqrt(6.0f / (float)(cin * k * k));
    w[l].resize((size_t)channels[l] * cin * k * k);
    b[l].resize(channels[l]);
    for (auto &v : w[l]) v = (2.0f * uniform() - 1.0f) * bound;
    for (auto &v : b[l]) v = (2.0f * uniform() - 1.0f) * 0.05f;
    flat_w.insert(flat_w.end(), w[l].begin(), w[l].end());
    flat_b.insert(flat_b.end(), b[l].begin(), b[l].end());
    cin = channels[l];
  }
  std::vector<float> pw(96), vw(96), pb(1, 0.01f), vb(1, -0.02f);
  for (auto &v : pw) v = (2.0f * uniform() - 1.0f) * 0.1f;
  for (auto &v : vw) v = (2.0f * uniform() - 1.0f) * 0.1f;

  // boards: binary own / opponent planes without overlap, third plane all ones or all zeros
  std::vector<float> x((size_t)B * 3 * cells, 0.0f);
  for (int i = 0; i < B; ++i) {
    const float fill = 0.1f + 0.4f * uniform();
    for (int a = 0; a < cells; ++a) {
      const float u = uniform();
      if (u < fill) x[((size_t)i * 3 + (u < fill / 2 ? 0 : 1)) * cells + a] = 1.0f;
    }
    if (i % 2)
      for (int a = 0; a < cells; ++a) x[((size_t)i * 3 + 2) * cells + a] = 1.0f;
  }

  std::vector<float> ref_logits((size_t)B * cells), ref_value(B);
  if (c6ref_forward(x.data(), B, n, 3, 8, kernels, channels, flat_w.data(), flat_b.data(), pw.data(),
                    pb.data(), vw.data(), vb.data(), ref_logits.data(), ref_value.data()) != 0) {
    std::fprintf(stderr, "oracle failed\n");
    return 2;
  }

  // device copies
  float *dw[8], *db[8], *dpw, *dpb, *dvw, *dvb, *dx, *dlogits, *dvalue;
  for (int l = 0; l < 8; ++l) {
    HIP_OK(hipMalloc(&dw[l], w[l].size() * 4));
    HIP_OK(hipMalloc(&db[l], b[l].size() * 4));
    HIP_OK(hipMemcpy(dw[l], w[l].data(), w[l].size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(db[l], b[l].data(), b[l].size() * 4, hipMemcpyHostToDevice));
  }
  HIP_OK(hipMalloc(&dpw, 96 * 4));
  HIP_OK(hipMalloc(&dvw, 96 * 4));
  HIP_OK(hipMalloc(&dpb, 4));
  HIP_OK(hipMalloc(&dvb, 4));
  HIP_OK(hipMemcpy(dpw, pw.data(), 96 * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dvw, vw.data(), 96 * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dpb, pb.data(), 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dvb, vb.data(), 4, hipMemcpyHostToDevice));
  HIP_OK(hipMalloc(&dx, x.size() * 4));
  HIP_OK(hipMemcpy(dx, x.data(), x.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMalloc(&dlogits, ref_logits.size() * 4));
  HIP_OK(hipMalloc(&dvalue, B * 4));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  int failures = 0;
  const struct {
    int prec;
    const char *name;
    double tol;
  } modes[] = {{C6_PREC_F32, "fp32", 1e-4}, {C6_PREC_BF16F6, "bf16f6", 2e-2}, {C6_PREC_BF16, "bf16", 2e-2}};
  for (const auto &m : modes) {
    size_t nbytes = 0;
    if (p_bytes(m.prec, &nbytes) != C6_OK) return 2;
    void *packed = nullptr;
    HIP_OK(hipMalloc(&packed, nbytes));
    if (p_pack(dw, db, dpw, dpb, dvw, dvb, m.prec, packed, stream) != C6_OK) {
      std::fprintf(stderr, "c6_pack_weights: %s\n", p_error());
      return 2;
    }
    const float lowest = -3.4028234663852886e38f;
    if (p_forward(dx, C6_DT_F32, 1, B, packed, nbytes, m.prec, dlogits, dvalue, C6_MASK_INPUT, nullptr,
                  lowest, nullptr, 1.0f, nullptr, nullptr, stream) != C6_OK) {
      std::fprintf(stderr, "c6_forward: %s\n", p_error());
      return 2;
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> logits(ref_logits.size()), value(B);
    HIP_OK(hipMemcpy(logits.data(), dlogits, logits.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(value.data(), dvalue, B * 4, hipMemcpyDeviceToHost));
    // occupied squares carry the fill, bit-exactly; the others are compared with the oracle
    std::vector<float> got, want;
    int mask_errors = 0;
    for (int i = 0; i < B; ++i)
      for (int a = 0; a < cells; ++a) {
        const bool occupied = x[((size_t)i * 3) * cells + a] != 0.0f || x[((size_t)i * 3 + 1) * cells + a] != 0.0f;
        const float v = logits[(size_t)i * cells + a];
        if (occupied) {
          mask_errors += (v != lowest);
        } else {
          got.push_back(v);
          want.push_back(ref_logits[(size_t)i * cells + a]);
        }
      }
    const double el = rel_l2(got, want), ev = rel_l2(value, ref_value);
    const bool ok = el <= m.tol && ev <= m.tol && mask_errors == 0;
    std::printf("%-7s logits rel-L2 %.3e  value rel-L2 %.3e  mask errors %d  %s\n", m.name, el, ev,
                mask_errors, ok ? "ok" : "FAIL");
    failures += !ok;
    HIP_OK(hipFree(packed));
  }
  // an invalid call must come back as an error code with a message, not a crash
  if (p_forward(nullptr, C6_DT_F32, 1, B, nullptr, 0, C6_PREC_F32, dlogits, dvalue, C6_MASK_NONE, nullptr,
                0.0f, nullptr, 1.0f, nullptr, nullptr, stream) != C6_EINVAL || p_error()[0] == '\0') {
    std::printf("null input was not rejected\n");
    ++failures;
  }
  std::printf(failures ? "FAILED\n" : "all checks passed\n");
  return failures ? 1 : 0;
}

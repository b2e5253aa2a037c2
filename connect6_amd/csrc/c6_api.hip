// extern "C" boundary of libconnect6_amd.so: argument validation and dispatch.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "c6_common.h"

namespace c6 {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int dispatch_pack(int prec, const PackParams &pp, hipStream_t st);
int dispatch_forward(int prec, const FwdParams &fp, hipStream_t st);
int dispatch_cascade(int prec, const FwdParams &fp, float threshold, void *workspace, hipStream_t st);
size_t packed_bytes(int prec);
int launch_mask(const void *, const uint8_t *, int, long long, uint32_t, void *, hipStream_t);
int launch_sample(const float *, const uint8_t *, const float *, float, long long, long long *,
                  float *, hipStream_t);
int launch_d4_expand(const void *, int, long long, void *, hipStream_t);
int launch_d4_reduce(const float *, const float *, long long, float *, float *, hipStream_t);
size_t generic_workspace_bytes(long long batch, int n, int layers, const int *channels);
int launch_generic(const void *x, int x_dtype, long long batch, long long per_group, int n, int layers,
                   const int *kernels, const int *channels, const float *const *conv_w,
                   const float *const *conv_b, const float *pol_w, const float *pol_b,
                   const float *val_w, const float *val_b, int prec, void *workspace,
                   float *logits, float *value, int mask_mode, const uint8_t *legal, float fill,
                   hipStream_t st);

size_t static_scratch_bytes();
int static_scratch(void **out);

int launch_env_step(const EnvParams &p, hipStream_t st);
int launch_canonical_input(const int8_t *boards, const int8_t *player, const int8_t *stones_left,
                           long long num, int n, float *out, hipStream_t st);

// The kernels exist for gfx950 only.  Checked once per device, just before an entry point's
// first launch there, so that another GPU gets C6_EARCH instead of a launch failure.
static int device_ok(const char *who) {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> state[kMaxDevices];  // 0 unknown, 1 gfx950, -1 something else
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("%s: no usable current device (%s)", who, hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  int s = state[dev].load(std::memory_order_relaxed);
  if (s == 0) {
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) {
      set_error("%s: hipGetDeviceProperties failed: %s", who, hipGetErrorString(e));
      return C6_ELAUNCH;
    }
    s = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
    if (s < 0) set_error("%s: device %d is %s; this library is built for gfx950 only", who, dev, prop.gcnArchName);
    state[dev].store(s, std::memory_order_relaxed);
  }
  if (s < 0) {
    set_error("%s: device %d is not gfx950; this library is built for gfx950 only", who, dev);
    return C6_EARCH;
  }
  return C6_OK;
}
#define C6_REQUIRE_DEVICE(who)                  \
  do {                                          \
    const int rc_dev_ = device_ok(who);         \
    if (rc_dev_ != C6_OK) return rc_dev_;       \
  } while (0)

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static int elem_bytes(int dt) { return dt == C6_DT_F32 ? 4 : ((dt == C6_DT_BF16 || dt == C6_DT_F16) ? 2 : 0); }
static bool valid_prec(int p) { return p >= C6_PREC_F32 && p <= C6_PREC_BF16C6; }

// the cascade's workspace argument, checked; `who` names the entry point in the message
static int check_cascade_workspace(const char *who, long long boards, const void *workspace, size_t bytes) {
  if (workspace == nullptr || !aligned16(workspace) || bytes < cascade_workspace_bytes(boards)) {
    set_error("%s: the workspace must be a 16-byte aligned device buffer of at least %zu bytes "
              "(c6_cascade_workspace_bytes), got %zu", who, cascade_workspace_bytes(boards), bytes);
    return C6_EINVAL;
  }
  return C6_OK;
}

}  // namespace c6

using namespace c6;

extern "C" {

int c6_version(void) { return 1; }

const char *c6_last_error(void) { return g_error; }

int c6_packed_bytes(int prec, size_t *bytes) {
  if (!valid_prec(prec) || bytes == nullptr) {
    set_error("c6_packed_bytes: bad precision mode %d or null output", prec);
    return C6_EINVAL;
  }
  *bytes = packed_bytes(prec);
  return C6_OK;
}

int c6_pack_weights_grouped(const float *const *conv_w, const float *const *conv_b,
                            const float *pol_w, const float *pol_b, const float *val_w,
                            const float *val_b, int64_t groups, int prec, void *packed,
                            size_t packed_stride, void *stream) {
  if (!valid_prec(prec)) {
    set_error("c6_pack_weights: unknown precision mode %d", prec);
    return C6_EINVAL;
  }
  if (groups < 1 || groups > 65535) {
    set_error("c6_pack_weights: %lld weight sets (one call packs 1 to 65535)", (long long)groups);
    return C6_EINVAL;
  }
  if (conv_w == nullptr || pol_w == nullptr || packed == nullptr) {
    set_error("c6_pack_weights: conv_w, pol_w and packed must not be null");
    return C6_EINVAL;
  }
  if (!aligned16(packed) || (packed_stride & 15u) != 0 || (groups > 1 && packed_stride < packed_bytes(prec))) {
    set_error("c6_pack_weights: packed buffer must be 16-byte aligned, its sets a multiple of 16 "
              "bytes and at least c6_packed_bytes() apart");
    return C6_EINVAL;
  }
  PackParams pp;
  for (int i = 0; i < 8; ++i) {
    if (conv_w[i] == nullptr) {
      set_error("c6_pack_weights: conv_w[%d] is null", i);
      return C6_EINVAL;
    }
    pp.conv_w[i] = conv_w[i];
    pp.conv_b[i] = conv_b ? conv_b[i] : nullptr;
  }
  pp.pol_w = pol_w;
  pp.pol_b = pol_b;
  pp.val_w = val_w;
  pp.val_b = val_b;
  pp.packed = static_cast<unsigned char *>(packed);
  pp.groups = (int)groups;
  pp.packed_stride = packed_stride;
  C6_REQUIRE_DEVICE("c6_pack_weights");
  return dispatch_pack(prec, pp, static_cast<hipStream_t>(stream));
}

int c6_pack_weights(const float *const *conv_w, const float *const *conv_b, const float *pol_w,
                    const float *pol_b, const float *val_w, const float *val_b, int prec,
                    void *packed, void *stream) {
  return c6_pack_weights_grouped(conv_w, conv_b, pol_w, pol_b, val_w, val_b, 1, prec, packed, 0, stream);
}

// c6_forward and c6_forward_cascade (workspace != nullptr: the latter)
static int forward_planes(const char *who, const void *x, int x_dtype, int64_t groups,
                          int64_t boards_per_group, const void *packed, size_t packed_stride,
                          int prec, void *logits, int logits_dtype, float *value, int mask_mode,
                          const uint8_t *legal, float fill, const float *u, float temperature,
                          int64_t *actions, float *logprob, bool cascade, float threshold,
                          void *workspace, size_t workspace_bytes, void *stream) {
  if (!valid_prec(prec) || is_cascade(prec) != cascade) {
    set_error("%s: precision mode %d is unknown or not served by this entry point (the cascade modes "
              "take c6_forward_cascade, every other mode c6_forward)", who, prec);
    return C6_EINVAL;
  }
  if (elem_bytes(x_dtype) == 0 || elem_bytes(logits_dtype) == 0) {
    set_error("%s: unknown element type of the input (%d) or of the logits (%d)", who, x_dtype, logits_dtype);
    return C6_EINVAL;
  }
  if (groups < 1 || boards_per_group < 0) {
    set_error("%s: groups=%lld boards_per_group=%lld out of range", who, (long long)groups,
              (long long)boards_per_group);
    return C6_EINVAL;
  }
  if (boards_per_group == 0) return C6_OK;  // empty batch: nothing to do
  if (groups > 0x7fffffffLL / boards_per_group) {
    set_error("%s: %lld x %lld boards exceed the 2^31-1 boards one launch can index", who,
              (long long)groups, (long long)boards_per_group);
    return C6_EINVAL;
  }
  if (x == nullptr || packed == nullptr) {
    set_error("%s: x and packed must not be null", who);
    return C6_EINVAL;
  }
  if (!aligned16(packed) || (packed_stride & 15u) != 0 ||
      (groups > 1 && packed_stride < packed_bytes(prec))) {
    set_error("%s: packed weights must be 16-byte aligned with stride >= one set", who);
    return C6_EINVAL;
  }
  if (mask_mode < C6_MASK_NONE || mask_mode > C6_MASK_LEGAL ||
      (mask_mode == C6_MASK_LEGAL && legal == nullptr)) {
    set_error("%s: bad mask_mode %d (legal mask %s)", who, mask_mode, legal ? "given" : "missing");
    return C6_EINVAL;
  }
  if (actions != nullptr && u == nullptr) {
    set_error("%s: sampling needs the uniform draws u", who);
    return C6_EINVAL;
  }
  FwdParams fp;
  fp.x = x;
  fp.x_dtype = x_dtype;
  fp.total_boards = groups * boards_per_group;
  fp.boards_per_group = boards_per_group;
  fp.packed = static_cast<const unsigned char *>(packed);
  fp.packed_stride = packed_stride;
  fp.logits = logits;
  fp.logits_dtype = logits_dtype;
  fp.value = value;
  fp.mask_mode = mask_mode;
  fp.legal = legal;
  fp.fill = fill;
  fp.u = u;
  fp.inv_temperature = 1.0f / (temperature > 1e-4f ? temperature : 1e-4f);
  fp.actions = reinterpret_cast<long long *>(actions);
  fp.logprob = logprob;
  fp.player = nullptr;
  fp.stones_left = nullptr;
  fp.index = nullptr;
  fp.num_states = 0;
  fp.view = 0;
  if (cascade) {
    const int rc = check_cascade_workspace(who, fp.total_boards, workspace, workspace_bytes);
    if (rc != C6_OK) return rc;
  }
  C6_REQUIRE_DEVICE(who);
  if (cascade) return dispatch_cascade(prec, fp, threshold, workspace, static_cast<hipStream_t>(stream));
  return dispatch_forward(prec, fp, static_cast<hipStream_t>(stream));
}

int c6_forward(const void *x, int x_dtype, int64_t groups, int64_t boards_per_group,
               const void *packed, size_t packed_stride, int prec, float *logits, float *value,
               int mask_mode, const uint8_t *legal, float fill, const float *u, float temperature,
               int64_t *actions, float *logprob, void *stream) {
  return forward_planes("c6_forward", x, x_dtype, groups, boards_per_group, packed, packed_stride, prec,
                        logits, C6_DT_F32, value, mask_mode, legal, fill, u, temperature, actions, logprob, false,
                        0.0f, nullptr, 0, stream);
}

int c6_cascade_workspace_bytes(int64_t boards, size_t *bytes) {
  if (boards < 0 || boards > 0x7fffffffLL || bytes == nullptr) {
    set_error("c6_cascade_workspace_bytes: board count out of range or null output");
    return C6_EINVAL;
  }
  *bytes = cascade_workspace_bytes(boards);
  return C6_OK;
}

int c6_forward_cascade(const void *x, int x_dtype, int64_t groups, int64_t boards_per_group,
                       const void *packed, size_t packed_stride, int prec, void *logits, int logits_dtype,
                       float *value, int mask_mode, const uint8_t *legal, float fill, const float *u,
                       float temperature, int64_t *actions, float *logprob, float threshold,
                       void *workspace, size_t workspace_bytes, void *stream) {
  return forward_planes("c6_forward_cascade", x, x_dtype, groups, boards_per_group, packed, packed_stride,
                        prec, logits, logits_dtype, value, mask_mode, legal, fill, u, temperature,
                        actions, logprob, true, threshold, workspace, workspace_bytes, stream);
}


static int forward_states(const char *who, const int8_t *boards, const int8_t *player,
                          const int8_t *stones_left, int64_t num_states, const int64_t *index,
                          int view, int64_t batch, const void *packed, int prec, void *logits,
                          int logits_dtype, float *value, int mask_mode, float fill, const float *u,
                          float temperature, int64_t *actions, float *logprob, bool cascade,
                          float threshold, void *workspace, size_t workspace_bytes, void *stream) {
  if (!valid_prec(prec) || is_cascade(prec) != cascade || elem_bytes(logits_dtype) == 0 || batch < 0 ||
      batch > 0x7fffffffLL || view < 0 || view > 7 || num_states < 0) {
    set_error("%s: bad precision %d, batch %lld, states %lld or view %d", who, prec,
              (long long)batch, (long long)num_states, view);
    return C6_EINVAL;
  }
  if (batch == 0) return C6_OK;
  if (num_states < 1 || (index == nullptr && batch > num_states)) {
    set_error("%s: %lld boards requested from %lld states", who, (long long)batch,
              (long long)num_states);
    return C6_EINVAL;
  }
  if (boards == nullptr || player == nullptr || stones_left == nullptr || packed == nullptr) {
    set_error("%s: boards, player, stones_left and packed must not be null", who);
    return C6_EINVAL;
  }
  if (!aligned16(packed)) {
    set_error("%s: packed weights must be 16-byte aligned", who);
    return C6_EINVAL;
  }
  if (mask_mode != C6_MASK_NONE && mask_mode != C6_MASK_INPUT) {
    set_error("%s: mask_mode must be C6_MASK_NONE or C6_MASK_INPUT, got %d", who, mask_mode);
    return C6_EINVAL;
  }
  if (actions != nullptr && u == nullptr) {
    set_error("%s: sampling needs the uniform draws u", who);
    return C6_EINVAL;
  }
  FwdParams fp;
  fp.x = boards;
  fp.x_dtype = C6_DT_BOARD_I8;
  fp.total_boards = batch;
  fp.boards_per_group = batch;
  fp.packed = static_cast<const unsigned char *>(packed);
  fp.packed_stride = 0;
  fp.logits = logits;
  fp.logits_dtype = logits_dtype;
  fp.value = value;
  fp.mask_mode = mask_mode;
  fp.legal = nullptr;
  fp.fill = fill;
  fp.u = u;
  fp.inv_temperature = 1.0f / (temperature > 1e-4f ? temperature : 1e-4f);
  fp.actions = reinterpret_cast<long long *>(actions);
  fp.logprob = logprob;
  fp.player = player;
  fp.stones_left = stones_left;
  fp.index = reinterpret_cast<const long long *>(index);
  fp.num_states = num_states;
  fp.view = view;
  if (cascade) {
    const int rc = check_cascade_workspace(who, batch, workspace, workspace_bytes);
    if (rc != C6_OK) return rc;
  }
  C6_REQUIRE_DEVICE(who);
  if (cascade) return dispatch_cascade(prec, fp, threshold, workspace, static_cast<hipStream_t>(stream));
  return dispatch_forward(prec, fp, static_cast<hipStream_t>(stream));
}

int c6_forward_boards(const int8_t *boards, const int8_t *player, const int8_t *stones_left,
                      int64_t num_states, const int64_t *index, int view, int64_t batch,
                      const void *packed, int prec,
                      float *logits, float *value, int mask_mode, float fill, const float *u,
                      float temperature, int64_t *actions, float *logprob, void *stream) {
  return forward_states("c6_forward_boards", boards, player, stones_left, num_states, index, view, batch,
                        packed, prec, logits, C6_DT_F32, value, mask_mode, fill, u, temperature, actions, logprob,
                        false, 0.0f, nullptr, 0, stream);
}

int c6_forward_boards_cascade(const int8_t *boards, const int8_t *player,
                              const int8_t *stones_left, int64_t num_states,
                              const int64_t *index, int view, int64_t batch, const void *packed,
                              int prec, void *logits, int logits_dtype, float *value, int mask_mode, float fill,
                              const float *u, float temperature, int64_t *actions,
                              float *logprob, float threshold, void *workspace,
                              size_t workspace_bytes, void *stream) {
  return forward_states("c6_forward_boards_cascade", boards, player, stones_left, num_states, index, view,
                        batch, packed, prec, logits, logits_dtype, value, mask_mode, fill, u,
                        temperature, actions, logprob, true, threshold, workspace, workspace_bytes, stream);
}


static int check_arch(const char *who, int board, int layers, const int *kernels,
                      const int *channels) {
  if (board < 1 || layers < 1 || channels == nullptr) {
    set_error("%s: board=%d layers=%d out of range or null channel list", who, board, layers);
    return C6_EINVAL;
  }
  for (int l = 0; l < layers; ++l) {
    if (channels[l] < 1 || (kernels && (kernels[l] < 1 || kernels[l] % 2 == 0))) {
      set_error("%s: layer %d needs a positive channel count and a positive odd kernel", who, l);
      return C6_EINVAL;
    }
  }
  return C6_OK;
}

int c6_generic_workspace_bytes(int64_t batch, int board, int layers, const int *channels,
                               size_t *bytes) {
  if (batch < 0 || bytes == nullptr) {
    set_error("c6_generic_workspace_bytes: negative batch or null output");
    return C6_EINVAL;
  }
  const int rc = check_arch("c6_generic_workspace_bytes", board, layers, nullptr, channels);
  if (rc != C6_OK) return rc;
  *bytes = generic_workspace_bytes(batch, board, layers, channels);
  return C6_OK;
}

static int forward_generic(const char *who, const void *x, int x_dtype, int64_t groups,
                           int64_t boards_per_group, int board, int layers, const int *kernels,
                           const int *channels, const float *const *conv_w,
                           const float *const *conv_b, const float *pol_w, const float *pol_b,
                           const float *val_w, const float *val_b, int prec, void *workspace,
                           size_t workspace_bytes, float *logits, float *value, int mask_mode,
                           const uint8_t *legal, float fill, void *stream) {
  if (!valid_prec(prec) || elem_bytes(x_dtype) == 0 || groups < 1 || boards_per_group < 0 ||
      kernels == nullptr || (boards_per_group > 0 && groups > INT64_MAX / boards_per_group)) {
    set_error("%s: bad precision %d, input type %d, groups %lld, boards %lld or null kernels", who,
              prec, x_dtype, (long long)groups, (long long)boards_per_group);
    return C6_EINVAL;
  }
  const int rc = check_arch(who, board, layers, kernels, channels);
  if (rc != C6_OK) return rc;
  const int64_t batch = groups * boards_per_group;
  if (batch == 0) return C6_OK;
  if (x == nullptr || conv_w == nullptr || pol_w == nullptr || workspace == nullptr ||
      (value != nullptr && val_w == nullptr)) {
    set_error("%s: null pointer (x, conv_w, pol_w, workspace, or value without val_w)", who);
    return C6_EINVAL;
  }
  for (int l = 0; l < layers; ++l)
    if (conv_w[l] == nullptr) {
      set_error("%s: conv_w[%d] is null", who, l);
      return C6_EINVAL;
    }
  if (workspace_bytes < generic_workspace_bytes(batch, board, layers, channels) ||
      !aligned16(workspace)) {
    set_error("%s: workspace too small or not 16-byte aligned", who);
    return C6_EINVAL;
  }
  if (mask_mode < C6_MASK_NONE || mask_mode > C6_MASK_LEGAL ||
      (mask_mode == C6_MASK_LEGAL && legal == nullptr)) {
    set_error("%s: bad mask_mode %d", who, mask_mode);
    return C6_EINVAL;
  }
  C6_REQUIRE_DEVICE(who);
  return launch_generic(x, x_dtype, batch, boards_per_group, board, layers, kernels, channels,
                        conv_w, conv_b, pol_w, pol_b, val_w, val_b, prec, workspace, logits, value,
                        mask_mode, legal, fill, static_cast<hipStream_t>(stream));
}

int c6_forward_generic(const void *x, int x_dtype, int64_t batch, int board, int layers,
                       const int *kernels, const int *channels, const float *const *conv_w,
                       const float *const *conv_b, const float *pol_w, const float *pol_b,
                       const float *val_w, const float *val_b, int prec, void *workspace,
                       size_t workspace_bytes, float *logits, float *value, int mask_mode,
                       const uint8_t *legal, float fill, void *stream) {
  if (batch < 0) {
    set_error("c6_forward_generic: negative batch");
    return C6_EINVAL;
  }
  return forward_generic("c6_forward_generic", x, x_dtype, 1, batch, board, layers, kernels,
                         channels, conv_w, conv_b, pol_w, pol_b, val_w, val_b, prec, workspace,
                         workspace_bytes, logits, value, mask_mode, legal, fill, stream);
}

int c6_forward_generic_grouped(const void *x, int x_dtype, int64_t groups,
                               int64_t boards_per_group, int board, int layers,
                               const int *kernels, const int *channels,
                               const float *const *conv_w, const float *const *conv_b,
                               const float *pol_w, const float *pol_b, const float *val_w,
                               const float *val_b, int prec, void *workspace,
                               size_t workspace_bytes, float *logits, float *value, int mask_mode,
                               const uint8_t *legal, float fill, void *stream) {
  return forward_generic("c6_forward_generic_grouped", x, x_dtype, groups, boards_per_group, board,
                         layers, kernels, channels, conv_w, conv_b, pol_w, pol_b, val_w, val_b,
                         prec, workspace, workspace_bytes, logits, value, mask_mode, legal, fill,
                         stream);
}

int c6_forward_generic_static(const void *x, int x_dtype, int64_t batch, int board, int layers,
                              const int *kernels, const int *channels,
                              const float *const *conv_w, const float *const *conv_b,
                              const float *pol_w, const float *pol_b, const float *val_w,
                              const float *val_b, int prec, float *logits, float *value,
                              int mask_mode, const uint8_t *legal, float fill, void *stream) {
  if (batch < 0) {
    set_error("c6_forward_generic_static: negative batch");
    return C6_EINVAL;
  }
  int rc = check_arch("c6_forward_generic_static", board, layers, kernels, channels);
  if (rc != C6_OK) return rc;
  const size_t need = generic_workspace_bytes(batch, board, layers, channels);
  if (need > static_scratch_bytes()) {
    set_error("c6_forward_generic_static: this batch needs %zu bytes of workspace, the built-in "
              "one holds %zu; use c6_forward_generic with a workspace of your own",
              need, static_scratch_bytes());
    return C6_EINVAL;
  }
  if (batch == 0) return C6_OK;
  C6_REQUIRE_DEVICE("c6_forward_generic_static");
  void *ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != C6_OK) return rc;
  return c6_forward_generic(x, x_dtype, batch, board, layers, kernels, channels, conv_w, conv_b,
                            pol_w, pol_b, val_w, val_b, prec, ws, static_scratch_bytes(), logits,
                            value, mask_mode, legal, fill, stream);
}

int c6_mask_logits(const void *logits, const uint8_t *legal, int dtype, int64_t batch,
                   uint32_t fill_bits, void *out, void *stream) {
  const int eb = elem_bytes(dtype);
  if (eb == 0 || batch < 0) {
    set_error("c6_mask_logits: bad dtype %d or batch %lld", dtype, (long long)batch);
    return C6_EINVAL;
  }
  if (batch == 0) return C6_OK;
  if (logits == nullptr || legal == nullptr || out == nullptr) {
    set_error("c6_mask_logits: null pointer");
    return C6_EINVAL;
  }
  if ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(out)) & (uintptr_t)(eb - 1)) {
    set_error("c6_mask_logits: logits/out must be aligned to their element size");
    return C6_EINVAL;
  }
  C6_REQUIRE_DEVICE("c6_mask_logits");
  return launch_mask(logits, legal, eb, (long long)batch * C6_ACTIONS, fill_bits, out,
                     static_cast<hipStream_t>(stream));
}

int c6_softmax_sample(const float *logits, const uint8_t *legal, const float *u, float temperature,
                      int64_t batch, int64_t *actions, float *logprob, void *stream) {
  if (batch < 0) {
    set_error("c6_softmax_sample: negative batch");
    return C6_EINVAL;
  }
  if (batch == 0) return C6_OK;
  if (logits == nullptr || u == nullptr || actions == nullptr) {
    set_error("c6_softmax_sample: logits, u and actions must not be null");
    return C6_EINVAL;
  }
  const float inv_t = 1.0f / (temperature > 1e-4f ? temperature : 1e-4f);
  C6_REQUIRE_DEVICE("c6_softmax_sample");
  return launch_sample(logits, legal, u, inv_t, batch, reinterpret_cast<long long *>(actions),
                       logprob, static_cast<hipStream_t>(stream));
}

int c6_env_step(int8_t *boards, int8_t *current_player, int8_t *stones_left, int16_t *empty_count,
                int16_t *move_count, const int64_t *actions, int view, int64_t num_envs,
                int board_size, int win_length, float *reward, uint8_t *done, int8_t *winner,
                int8_t *transition_sign, int16_t *game_lengths, void *stream) {
  if (num_envs < 0 || board_size < 1 || board_size > 181 || win_length < 1 || view < 0 || view > 7) {
    set_error("c6_env_step: bad sizes (num_envs %lld, board_size %d, win_length %d) or view %d",
              (long long)num_envs, board_size, win_length, view);
    return C6_EINVAL;
  }
  if (num_envs > 0 && (!boards || !current_player || !stones_left || !empty_count || !move_count ||
                       !actions || !reward || !done || !winner || !transition_sign || !game_lengths)) {
    set_error("c6_env_step: null state, action or result pointer");
    return C6_EINVAL;
  }
  EnvParams p;
  p.boards = boards;
  p.player = current_player;
  p.stones_left = stones_left;
  p.empty_count = empty_count;
  p.move_count = move_count;
  p.actions = reinterpret_cast<const long long *>(actions);
  p.num = num_envs;
  p.n = board_size;
  p.win = win_length;
  p.view = view;
  p.reward = reward;
  p.done = done;
  p.winner = winner;
  p.sign = transition_sign;
  p.lengths = game_lengths;
  if (num_envs == 0) return C6_OK;
  C6_REQUIRE_DEVICE("c6_env_step");
  return launch_env_step(p, static_cast<hipStream_t>(stream));
}

int c6_canonical_input(const int8_t *boards, const int8_t *current_player,
                       const int8_t *stones_left, int64_t num_envs, int board_size, float *out,
                       void *stream) {
  if (num_envs < 0 || board_size < 1 || board_size > 181) {
    set_error("c6_canonical_input: bad sizes (num_envs %lld, board_size %d)", (long long)num_envs,
              board_size);
    return C6_EINVAL;
  }
  if (num_envs > 0 && (!boards || !current_player || !stones_left || !out)) {
    set_error("c6_canonical_input: null pointer");
    return C6_EINVAL;
  }
  if (num_envs == 0) return C6_OK;
  C6_REQUIRE_DEVICE("c6_canonical_input");
  return launch_canonical_input(boards, current_player, stones_left, num_envs, board_size, out,
                                static_cast<hipStream_t>(stream));
}

int c6_d4_expand(const void *x, int dtype, int64_t batch, void *out, void *stream) {
  const int eb = elem_bytes(dtype);
  if (eb == 0 || batch < 0) {
    set_error("c6_d4_expand: bad dtype %d or batch %lld", dtype, (long long)batch);
    return C6_EINVAL;
  }
  if (batch == 0) return C6_OK;
  if (x == nullptr || out == nullptr) {
    set_error("c6_d4_expand: null pointer");
    return C6_EINVAL;
  }
  C6_REQUIRE_DEVICE("c6_d4_expand");
  return launch_d4_expand(x, eb, batch, out, static_cast<hipStream_t>(stream));
}

int c6_d4_reduce(const float *view_logits, const float *view_values, int64_t batch, float *logits,
                 float *values, void *stream) {
  if (batch < 0) {
    set_error("c6_d4_reduce: negative batch");
    return C6_EINVAL;
  }
  if (batch == 0) return C6_OK;
  if (view_logits == nullptr || logits == nullptr || (values != nullptr && view_values == nullptr)) {
    set_error("c6_d4_reduce: null pointer");
    return C6_EINVAL;
  }
  C6_REQUIRE_DEVICE("c6_d4_reduce");
  return launch_d4_reduce(view_logits, view_values, batch, logits, values,
                          static_cast<hipStream_t>(stream));
}

}  // extern "C"

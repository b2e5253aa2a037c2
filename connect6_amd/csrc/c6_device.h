// Device helpers shared by the connect6_amd kernels (wave64 reductions, sampling, D4 maps).
#pragma once
#include "c6_common.h"

namespace c6 {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wave_max_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}

// Masked softmax + inverse-CDF draw over 361 entries by ONE wave.
// z(i) must return the tempered logit of entry i, ok(i) its legality.
// action = first i with running sum of exp(z - max) > u * total, clamped to
// the last legal entry; logp = z[a] - max - log(total).
template <class FZ, class FOK>
__device__ __forceinline__ void wave_sample(int lane, float u, FZ z, FOK ok, int &action,
                                            float &logp) {
  constexpr int PER = 6;  // 64 lanes x 6 = 384 >= 361
  float zz[PER];
  bool lg[PER];
  float m = -INFINITY;
  int lastlegal = -1;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = lane * PER + e;
    lg[e] = (i < kPix) && ok(i);
    zz[e] = lg[e] ? z(i) : -INFINITY;
    m = fmaxf(m, zz[e]);
    if (lg[e]) lastlegal = i;
  }
  m = wave_max(m);
  lastlegal = wave_max_i(lastlegal);
  float ex[PER];
  float local = 0.0f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    ex[e] = lg[e] ? __expf(zz[e] - m) : 0.0f;
    local += ex[e];
  }
  // inclusive scan of lane sums
  float incl = local;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float t = __shfl_up(incl, o, 64);
    if (lane >= o) incl += t;
  }
  const float total = __shfl(incl, 63, 64);
  const float target = u * total;
  float run = incl - local;
  int first = 1 << 30;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    run += ex[e];
    if (lg[e] && run > target && first == (1 << 30)) first = lane * PER + e;
  }
  first = wave_min_i(first);
  if (first == (1 << 30)) first = lastlegal;
  if (first < 0) first = 0;  // no legal square at all: defined but meaningless
  action = first;
  // fetch z[action] from the lane that holds it
  float za = 0.0f;
#pragma unroll
  for (int e = 0; e < PER; ++e)
    if (lane * PER + e == first) za = zz[e];
  za = wave_max(lane == first / PER ? za : -INFINITY);
  logp = za - m - __logf(total);
}


// D4 views, numbered as _symmetry_for_phase (connect6/train.py:216-219 of the
// reference): view p = rotate by (p%4) quarter turns, then mirror columns if p >= 4.
// canonical square a -> its square in view p (connect6/train.py:233-253)
__device__ __forceinline__ int d4_to_view(int a, int p) {
  const int n = kBoard, k = p & 3;
  int r = a / n, c = a - r * n;
  int rr = r, cc = c;
  if (k == 1) { rr = n - 1 - c; cc = r; }
  else if (k == 2) { rr = n - 1 - r; cc = n - 1 - c; }
  else if (k == 3) { rr = c; cc = n - 1 - r; }
  if (p >= 4) cc = n - 1 - cc;
  return rr * n + cc;
}
// square v of view p -> canonical square (connect6/train.py:256-277)
__device__ __forceinline__ int d4_from_view(int v, int p, int n = kBoard) {
  const int k = p & 3;
  int r = v / n, c = v - r * n;
  if (p >= 4) c = n - 1 - c;
  int rr = r, cc = c;
  if (k == 1) { rr = c; cc = n - 1 - r; }
  else if (k == 2) { rr = n - 1 - r; cc = n - 1 - c; }
  else if (k == 3) { rr = n - 1 - c; cc = r; }
  return rr * n + cc;
}

}  // namespace c6

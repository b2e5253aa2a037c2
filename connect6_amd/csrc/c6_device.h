// Device helpers shared by the connect6_amd kernels (wave64 reductions, sampling, D4 maps).
#pragma once
#include <type_traits>

#include "c6_common.h"

namespace c6 {

// A non-temporal store, for an output that is streamed to HBM and not read again here.  Measured
// on 0.85 GB of masked logits it is worth 3 %; the view gather gains nothing from it and the
// canonical planes lose 7 %, so only the masking kernels use it.
template <class T> __device__ __forceinline__ void stream_store(T *p, const T &v) {
  __builtin_nontemporal_store(v, p);
}

// Wave64 all-reduce without LDS traffic: DPP inside a row of 16 lanes (quad swaps, then the
// mirrored lane of the 8- and the 16-group, which belongs to the half not yet combined), then
// v_permlane16_swap / v_permlane32_swap across rows.  Every lane ends with the result.
template <class Op> __device__ __forceinline__ int wave_allreduce_bits(int v, Op op) {
  v = op(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
  v = op(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
  v = op(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xF, 0xF, false));  // row_half_mirror
  v = op(v, __builtin_amdgcn_update_dpp(v, v, 0x140, 0xF, 0xF, false));  // row_mirror
  {
    const auto r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false);
    const unsigned r0 = r[0], r1 = r[1];  // this row's and the neighbouring row's value
    v = op((int)r0, (int)r1);
  }
  {
    const auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
    const unsigned r0 = r[0], r1 = r[1];  // this half's and the other half's value
    v = op((int)r0, (int)r1);
  }
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  return __builtin_bit_cast(float, wave_allreduce_bits(__builtin_bit_cast(int, v), [](int a, int b) {
    return __builtin_bit_cast(int, __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b));
  }));
}
__device__ __forceinline__ float wave_max(float v) {
  return __builtin_bit_cast(float, wave_allreduce_bits(__builtin_bit_cast(int, v), [](int a, int b) {
    return __builtin_bit_cast(int, fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b)));
  }));
}
__device__ __forceinline__ int wave_min_i(int v) {
  return wave_allreduce_bits(v, [](int a, int b) { return a < b ? a : b; });
}
__device__ __forceinline__ int wave_max_i(int v) {
  return wave_allreduce_bits(v, [](int a, int b) { return a > b ? a : b; });
}
// Inclusive prefix sum over the 64 lanes: shifts inside each row of 16 (lanes without a source
// add 0), then the totals of the rows before: lane 15 of rows 0 and 2 into rows 1 and 3, lane
// 31 (by then the total of rows 0-1) into rows 2 and 3.
__device__ __forceinline__ float wave_inclusive_sum(float v) {
  auto shifted = [](float x, auto ctrl, auto rows) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value,
                                                                 decltype(rows)::value, 0xF, false));
  };
  using std::integral_constant;
  v += shifted(v, integral_constant<int, 0x111>{}, integral_constant<int, 0xF>{});  // row_shr:1
  v += shifted(v, integral_constant<int, 0x112>{}, integral_constant<int, 0xF>{});  // row_shr:2
  v += shifted(v, integral_constant<int, 0x114>{}, integral_constant<int, 0xF>{});  // row_shr:4
  v += shifted(v, integral_constant<int, 0x118>{}, integral_constant<int, 0xF>{});  // row_shr:8
  v += shifted(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xA>{});  // row_bcast:15 -> rows 1, 3
  v += shifted(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xC>{});  // row_bcast:31 -> rows 2, 3
  return v;
}

// the same for integers
__device__ __forceinline__ int wave_inclusive_sum_i(int v) {
  auto shifted = [](int x, auto ctrl, auto rows) {
    return __builtin_amdgcn_update_dpp(0, x, decltype(ctrl)::value, decltype(rows)::value, 0xF, false);
  };
  using std::integral_constant;
  v += shifted(v, integral_constant<int, 0x111>{}, integral_constant<int, 0xF>{});  // row_shr:1
  v += shifted(v, integral_constant<int, 0x112>{}, integral_constant<int, 0xF>{});  // row_shr:2
  v += shifted(v, integral_constant<int, 0x114>{}, integral_constant<int, 0xF>{});  // row_shr:4
  v += shifted(v, integral_constant<int, 0x118>{}, integral_constant<int, 0xF>{});  // row_shr:8
  v += shifted(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xA>{});  // row_bcast:15 -> rows 1, 3
  v += shifted(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xC>{});  // row_bcast:31 -> rows 2, 3
  return v;
}

__device__ __forceinline__ float wave_min(float v) {
  return __builtin_bit_cast(float, wave_allreduce_bits(__builtin_bit_cast(int, v), [](int a, int b) {
    return __builtin_bit_cast(int, fminf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b)));
  }));
}

// Is the decision of a board (the largest of its 361 logits, entries with ok(i) only) closer than
// the rounding noise of the plain bf16 pass?  Yes when the largest logit leads the second largest
// by less than `tau` standard deviations of those logits, or when at least two other logits lie
// within 2 tau standard deviations of it (several near-ties multiply the chance that one of them
// overtakes).  One wave; tau < 0 answers yes for every board, and a board with fewer than two
// such entries has no decision to judge: no.  Everything is taken relative to the largest logit,
// so a large common offset of the logits (flat policies) costs no precision.
template <class FZ, class FOK>
__device__ __forceinline__ bool wave_margin_below(int lane, float tau, FZ z, FOK ok) {
  constexpr int PER = 6;  // 64 lanes x 6 = 384 >= 361
  float d[PER];           // largest - logit (>= 0), inf for entries that do not count
  float m = -INFINITY;
  int n = 0;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = lane * PER + e;
    const bool use = (i < kPix) && ok(i);
    d[e] = use ? z(i) : -INFINITY;
    m = fmaxf(m, d[e]);
    n += use ? 1 : 0;
  }
  m = wave_max(m);
  // the margin is the second smallest d (the smallest is 0)
  float d1 = INFINITY, d2 = INFINITY, s = 0.0f, ss = 0.0f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    if (d[e] != -INFINITY) {
      d[e] = m - d[e];
      s += d[e];
      ss = fmaf(d[e], d[e], ss);
      d2 = d[e] < d1 ? d1 : fminf(d2, d[e]);
      d1 = fminf(d1, d[e]);
    } else {
      d[e] = INFINITY;
    }
  }
  const float cnt = wave_sum((float)n);
  s = wave_sum(s);
  ss = wave_sum(ss);
  // one lane that holds a largest logit answers with its second smallest d, every other lane
  // with its smallest (a second lane with a largest logit answers 0: a tie)
  const unsigned long long tops = __builtin_amdgcn_ballot_w64(d1 == 0.0f);
  const int owner = tops != 0 ? __builtin_ctzll(tops) : 0;
  const float gap = wave_min(lane == owner ? d2 : d1);
  if (cnt < 2.0f) return false;
  if (tau < 0.0f) return true;
  const float mean = s / cnt;
  const float var = fmaxf(ss / cnt - mean * mean, 0.0f);
  const float t2 = tau * tau * var;
  int near = 0;  // entries within 2 tau standard deviations of the largest (itself included)
#pragma unroll
  for (int e = 0; e < PER; ++e) near += (d[e] * d[e] < 4.0f * t2) ? 1 : 0;
  const float nearf = wave_sum((float)near);
  return gap * gap < t2 || nearf >= 3.0f;
}

// Masked softmax + inverse-CDF draw over 361 entries by ONE wave.
// z(i) must return the logit of entry i, ok(i) its legality; inv_t = 1 / temperature.
// action = first i with running sum of exp(z/T - max) > u * total, clamped to the last legal
// entry; logp = z[a]/T - max - log(total).
// The kernels that call this are bound by its VALU instructions, so it is written to need few:
// logits are carried in units of log2 (one multiply per entry, a bare v_exp_f32 each), an illegal
// entry is -inf and exponentiates to 0 by itself, the lane that holds the draw is found with a
// ballot, and the last legal entry is only looked for when no running sum exceeds the target
// (u * total rounding up to the total).
template <class FZ, class FOK>
__device__ __forceinline__ void wave_sample(int lane, float u, float inv_t, FZ z, FOK ok, int &action,
                                            float &logp) {
  constexpr int PER = 6;  // 64 lanes x 6 = 384 >= 361
  constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;
  const float s2 = inv_t * kLog2e;
  float zz[PER];
  float m = -INFINITY;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = lane * PER + e;
    zz[e] = ((i < kPix) && ok(i)) ? z(i) * s2 : -INFINITY;
    m = fmaxf(m, zz[e]);
  }
  m = wave_max(m);
  const float mc = fmaxf(m, -3.0e38f);  // (no legal entry at all: exp2(-inf - mc) stays 0, not NaN)
  float run[PER];
  float local = 0.0f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    local += __builtin_amdgcn_exp2f(zz[e] - mc);
    run[e] = local;  // running sum inside the lane
  }
  const float incl = wave_inclusive_sum(local);
  const float total = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, incl), 63));
  const float target = u * total;
  // the first lane whose inclusive sum exceeds the target holds the draw
  const unsigned long long over = __builtin_amdgcn_ballot_w64(incl > target);
  int first;
  if (over != 0) {
    const int owner = __builtin_ctzll(over);
    const float before = incl - local;
    int cnt = 0;  // entries of this lane whose running sum does not exceed the target yet
#pragma unroll
    for (int e = 0; e < PER; ++e) cnt += (before + run[e] > target) ? 0 : 1;
    cnt = cnt < PER ? cnt : PER - 1;  // ((incl - local) + local may round below incl)
    float zsel = zz[PER - 1];
#pragma unroll
    for (int e = PER - 2; e >= 0; --e) zsel = cnt == e ? zz[e] : zsel;
    first = owner * PER + __builtin_amdgcn_readlane(cnt, owner);
    float za = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, zsel), owner));
    if (za == -INFINITY) {
      // Rounding put the draw on an illegal entry next to the step it belongs to (the lanes'
      // sums disagree in the last bit): take the nearest legal entry below, else above.
      int below = -1, above = 1 << 30;
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        const int i = lane * PER + e;
        if (zz[e] != -INFINITY) {
          if (i <= first) below = i;
          if (i > first && above == (1 << 30)) above = i;
        }
      }
      below = wave_max_i(below);
      above = wave_min_i(above);
      first = below >= 0 ? below : above;
      float zf = -INFINITY;
#pragma unroll
      for (int e = 0; e < PER; ++e)
        if (lane * PER + e == first) zf = zz[e];
      za = wave_max(zf);
    }
    logp = (za - m) * kLn2 - __logf(total);
  } else {
    int lastlegal = -1;
#pragma unroll
    for (int e = 0; e < PER; ++e)
      if (zz[e] != -INFINITY) lastlegal = lane * PER + e;
    lastlegal = wave_max_i(lastlegal);
    first = lastlegal < 0 ? 0 : lastlegal;  // no legal square at all: defined but meaningless
    float za = -INFINITY;
#pragma unroll
    for (int e = 0; e < PER; ++e)
      if (lane * PER + e == first) za = zz[e];
    za = wave_max(za);
    logp = (za - m) * kLn2 - __logf(total);
  }
  action = first;
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

// Fused forward of the Connect6 policy/value CNN for gfx950 (MI355X).
//
// One workgroup (4 waves) carries one board through all eight convolutions and
// both heads without leaving the CU: the 19x19xC activation tile stays in LDS
// (channel-last, written in place after a barrier because every wave keeps its
// whole output tile in MFMA accumulators), weights stream from L2 straight
// into registers in MFMA-fragment order, and the grid is persistent over
// boards.  Replaces PolicyValueNet.forward (connect6/model.py:96-111 of the
// reference) and, with several weight sets, HistoricalPolicyEnsemble
// .forward_grouped (connect6/history.py:276-303).
//
// Implicit GEMM orientation: D[cout, pixel] += W[cout, k] * X[k, pixel], so an
// accumulator lane holds ONE pixel and 16 channels -- the epilogue writes four
// consecutive channels per store and the 1x1 heads reduce mostly inside a lane.
#include "c6_common.h"
#include "c6_device.h"

namespace c6 {

// Optional phase timestamps for kernel tuning (connect6_amd/profiling.py builds a traced copy;
// the shipped library contains none of this).
#ifdef C6_TRACE
__device__ long long g_trace[256 * 4 * 64];
#define C6_MARK(idx)                                                                       \
  do {                                                                                     \
    if (trace_on && lane == 0 && blockIdx.x < 256) {                                       \
      g_trace[(blockIdx.x * 4 + wave) * 64 + (idx)] = (long long)__builtin_readcyclecounter(); \
      if ((idx) == 0 || (idx) == 20) /* the constant 100 MHz clock beside it */            \
        g_trace[(blockIdx.x * 4 + wave) * 64 + 50 + (idx) / 20] = (long long)__builtin_amdgcn_s_memrealtime(); \
    }                                                                                      \
  } while (0)
#else
#define C6_MARK(idx) do { } while (0)
#endif

// ------------------------------------------------------------------------
// precision-specific primitives
// ------------------------------------------------------------------------
template <class P> __device__ __forceinline__ void mma(const v4i &a, const v4i &b, f32x16 &c);

template <> __device__ __forceinline__ void mma<PrecBF16>(const v4i &a, const v4i &b, f32x16 &c) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                              __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ void mma<PrecBF16F6>(const v4i &a, const v4i &b, f32x16 &c) {
  mma<PrecBF16>(a, b, c);
}
template <> __device__ __forceinline__ void mma<PrecBF16F6W>(const v4i &a, const v4i &b, f32x16 &c) {
  mma<PrecBF16>(a, b, c);
}
template <> __device__ __forceinline__ void mma<PrecF16>(const v4i &a, const v4i &b, f32x16 &c) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                             __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ void mma<PrecF32>(const v4i &a, const v4i &b, f32x16 &c) {
  const f32x4 af = __builtin_bit_cast(f32x4, a);
  const f32x4 bf = __builtin_bit_cast(f32x4, b);
#pragma unroll
  for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(af[e], bf[e], c, 0, 0, 0);
}

template <class P> __device__ __forceinline__ unsigned short bits16(float v) {
  if constexpr (P::ID == C6_PREC_F16) {
    return __builtin_bit_cast(unsigned short, (_Float16)v);
  } else {
    return __builtin_bit_cast(unsigned short, (__bf16)v);  // RNE
  }
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// two fp32 -> one dword of two 16-bit values (round to nearest even), low half first
template <class P> __device__ __forceinline__ int pack2(float a, float b) {
  const f32x2 v = {a, b};
  if constexpr (P::ID == C6_PREC_F16) {
    return __builtin_bit_cast(int, __builtin_convertvector(v, f16x2));
  } else {
    return __builtin_bit_cast(int, __builtin_convertvector(v, bf16x2));
  }
}
// What rounding to bf16 dropped: a - float(low half of w) and b - float(high half of w), each
// ONE v_dot2c_f32_bf16 (acc + w.lo * m.lo + w.hi * m.hi with m = {-1, 0} or {0, -1}) instead of
// an unpack and a subtract.  The difference is exactly representable, so the result is exact.
// The multiplier pairs must sit in registers: as inline constants the compiler encodes them wrongly.
struct DropConsts {
  bf16x2 lo, hi;
};
template <class P> __device__ __forceinline__ DropConsts drop_consts() {
  unsigned b0 = 0x0000BF80u, b1 = 0xBF800000u;
  if constexpr (P::LO6) asm volatile("" : "+v"(b0), "+v"(b1));  // (only the mode that uses them)
  return DropConsts{__builtin_bit_cast(bf16x2, b0), __builtin_bit_cast(bf16x2, b1)};
}
__device__ __forceinline__ float dropped_lo(float a, int w, const DropConsts &k) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), k.lo, a, false);
}
__device__ __forceinline__ float dropped_hi(float b, int w, const DropConsts &k) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), k.hi, b, false);
}

// XOR term of the granule swizzle for position `pos` (0 for the padded layout)
template <class P> __device__ __forceinline__ int swz_of(int pos) {
  if constexpr (Geo<P>::PADDED) {
    return 0;
  } else {
    return ((pos >> 1) & 7) << 4;
  }
}

// four consecutive channels of one position, converted to the storage type
template <class P> struct Packed4 {
  v2i hi;  // 16-bit modes: 4 values
};
template <> struct Packed4<PrecF32> {
  f32x4 v;
};

template <class P> __device__ __forceinline__ Packed4<P> pack4(const float (&v)[4]) {
  Packed4<P> r;
  if constexpr (P::EB == 4) {
    r.v = f32x4{v[0], v[1], v[2], v[3]};
  } else {
    r.hi[0] = pack2<P>(v[0], v[1]);
    r.hi[1] = pack2<P>(v[2], v[3]);
  }
  return r;
}

// store at logical byte offset `o` inside the record of the position at `pbase` (swizzle `sw`)
template <class P>
__device__ __forceinline__ void put4(unsigned char *smem, int pbase, int sw, int o,
                                     const Packed4<P> &r) {
  if constexpr (P::EB == 4) {
    *reinterpret_cast<f32x4 *>(smem + pbase + (o ^ sw)) = r.v;
  } else {
    *reinterpret_cast<v2i *>(smem + pbase + (o ^ sw)) = r.hi;
  }
}

// The 16-bit modes carry every pre-activation and activation multiplied by kActScale = -log2(e):
// the packed first-layer weights and all biases are scaled by it, the head weights by its
// inverse, and the weights of layers 2-8 not at all (their inputs already carry the factor).
// SiLU then needs no multiply in front of its exp2:  u = kActScale * v  ->
// u / (1 + 2^u) = kActScale * v * sigmoid(v).
constexpr float kActScale = -1.4426950408889634f;
template <class P> __device__ __forceinline__ float silu(float v) {
  if constexpr (P::EB == 4) {
    return v / (1.0f + expf(-v));
  } else {
    return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v));
  }
}
template <class P> __host__ __device__ constexpr float act_scale() { return P::EB == 4 ? 1.0f : kActScale; }

__device__ __forceinline__ float load_x(const void *x, int dt, size_t i) {
  if (dt == C6_DT_F32) return reinterpret_cast<const float *>(x)[i];
  const unsigned short b = reinterpret_cast<const unsigned short *>(x)[i];
  if (dt == C6_DT_BF16) return __builtin_bit_cast(float, (unsigned)b << 16);
  return (float)__builtin_bit_cast(_Float16, b);
}

// ------------------------------------------------------------------------
// weight-fragment prefetch rings.  A ring holds the fragments of the next
// kRing k-steps; the ring of layer L+1 is loaded before the epilogue of layer
// L so that no layer starts by waiting on L2.
// ------------------------------------------------------------------------
template <class P> struct L1Pipe {
  static constexpr int CPR = Geo<P>::CPR;
  static constexpr int ROWS_BODY = (CPR == 3) ? 7 : 1;
  static constexpr int U = ROWS_BODY * CPR;
  static constexpr int D = (CPR == 3) ? 7 : 6;
  static constexpr int ITERS = kL1RowsHalf / ROWS_BODY;
  static_assert(U % D == 0 && ITERS * ROWS_BODY == kL1RowsHalf, "first-layer pipeline shape");
};

// A run of 1 KiB weight fragments of one packed buffer, read 16 bytes per lane with buffer loads:
// the fragment's offset travels in a scalar register and the lane's part (lane * 16) in one
// vector register that never changes, so a load needs no per-lane 64-bit address arithmetic and
// issues in a few cycles (a global load with a per-lane address costs the wave ~20-30 cycles of
// issue time next to MFMAs; measured, this form ~2).
struct WFrags {
  __amdgpu_buffer_rsrc_t rsrc;
  int lane_off;  // lane * 16
  int base;      // byte offset of fragment 0 (wave-uniform)
  __device__ __forceinline__ v4i operator[](int f) const {
    return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off, base + f * 1024, 0));
  }
  // 8 bytes per lane of a fragment whose lanes lie 8 bytes apart (the fragment's first 512 bytes):
  // the load then touches 8 of the L1's 64-byte sectors instead of 16 half-used ones
  __device__ __forceinline__ v2i dense8(int f) const {
    return __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rsrc, lane_off >> 1, base + f * 1024, 0));
  }
  __device__ __forceinline__ WFrags operator+(int f) const { return WFrags{rsrc, lane_off, base + f * 1024}; }
};
template <class P>
__device__ __forceinline__ WFrags packed_frags(const unsigned char *packed, int lane, int frag) {
  // (packed is the same for every lane: a board's weight set)
  return WFrags{__builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char *>(packed), 0,
                                                  (int)Geo<P>::TAIL_OFF, 0x00020000),
                lane * 16, frag * 1024};
}

// fragments (k-step s, cout tile t) of a layer with NT cout tiles sit at index s*NT + t
template <int D, int NT>
__device__ __forceinline__ void preload_ring(v4i (&ring)[D][NT], const WFrags &wl) {
#pragma unroll
  for (int d = 0; d < D; ++d)
#pragma unroll
    for (int t = 0; t < NT; ++t) ring[d][t] = wl[d * NT + t];
}

template <int N> __device__ __forceinline__ void preload_flat(v4i (&ring)[N], const WFrags &wl) {
#pragma unroll
  for (int f = 0; f < N; ++f) ring[f] = wl[f];
}

template <class P, int L>
__device__ __forceinline__ WFrags layer_weights(const unsigned char *packed, int lane) {
  return packed_frags<P>(packed, lane, Geo<P>::frag_offset(L));
}

// compile-time loop: f(IC<B>{}), f(IC<B+1>{}), ... (the index is a constant expression inside f)
template <int I> struct IC {
  static constexpr int value = I;
};
template <int B, int E, class F> __device__ __forceinline__ void static_for(F &&f) {
  if constexpr (B < E) {
    f(IC<B>{});
    static_for<B + 1, E>(f);
  }
}

constexpr int kAhead = 2;  // k-steps between the LDS read of an activation fragment and its MFMAs

// Issue order inside one k-step: memory instructions are dealt out one at a time between
// MFMAs instead of in a burst.
template <int N_MFMA, int N_DSREAD, int N_VMEM> __device__ __forceinline__ void interleave_step() {
#pragma unroll
  for (int i = 0; i < N_MFMA; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
    if (i < N_DSREAD) {
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
    } else if (i < N_DSREAD + N_VMEM) {
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
    }
  }
}

// ------------------------------------------------------------------------
// first layer: 23x23 on 3 planes, K = (ky, plane, kx24) split over lane halves
// ------------------------------------------------------------------------
template <class P>
__device__ __forceinline__ void conv1_pass(const unsigned char *smem, const WFrags &wl,
                                           v4i (&ring)[L1Pipe<P>::D][1], const int (&l1base)[3],
                                           f32x16 (&acc)[1][3]) {
  using G = Geo<P>;
  using PP = L1Pipe<P>;
  constexpr int CPR = PP::CPR, U = PP::U, D = PP::D, ITERS = PP::ITERS, W = G::W;
  constexpr int ROWB = kL1RowPitch * G::EB;
  static_assert((U * W) % D == 0, "the ring must line up across loop iterations");

  // activation fragments are fetched kAhead k-steps before their MFMAs (an LDS read issued
  // during one k-step of three MFMAs would not be back by the next)
  static_assert(U % (kAhead + 1) == 0, "fragment queue must line up across loop iterations");
  v4i bq[kAhead + 1][3];
#pragma unroll
  for (int a = 0; a < kAhead; ++a)
#pragma unroll
    for (int j = 0; j < 3; ++j)
      bq[a][j] = *reinterpret_cast<const v4i *>(smem + l1base[j] + (a / CPR) * ROWB + (a % CPR) * 16);
#pragma unroll 1
  for (int it = 0; it < ITERS; ++it) {
    const int adv = it * PP::ROWS_BODY * ROWB;
    const WFrags wn = wl + (it * U * W + D);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // after the last steps this reads the zero row / the next copy, which is harmless
      const int un = u + kAhead;
      const int offn = (un / CPR) * ROWB + (un % CPR) * 16;
#pragma unroll
      for (int j = 0; j < 3; ++j)
        bq[un % (kAhead + 1)][j] = *reinterpret_cast<const v4i *>(smem + l1base[j] + adv + offn);
#pragma unroll
      for (int w = 0; w < W; ++w) {  // the weights, then (WLO) what their rounding dropped
#pragma unroll
        for (int j = 0; j < 3; ++j) mma<P>(ring[(u * W + w) % D][0], bq[u % (kAhead + 1)][j], acc[0][j]);
        ring[(u * W + w) % D][0] = wn[u * W + w];  // fragment (it*U + u) * W + w + D (the tail over-reads the next layer)
      }
      interleave_step<3 * W * (P::EB == 4 ? 4 : 1), 3, W>();
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// First layer when the third input plane is constant: K = (ky, kx24) of planes 0 and 1, plane h
// in lane half h (Geo::FAST1_*).  l1fast[j]: as l1base, for halo row 3 r + h.
// `ring`: a FIFO over the fragment stream (fragment s in slot s % D), filled with its first D.
template <class P>
__device__ __forceinline__ void conv1_fast_pass(const unsigned char *smem, const WFrags &wl,
                                                v4i (&ring)[L1Pipe<P>::D][1], const int (&l1fast)[3],
                                                f32x16 (&acc)[1][3]) {
  using G = Geo<P>;
  constexpr int CPR = G::CPR, D = L1Pipe<P>::D, QN = kAhead + 1, S = G::FAST1_STEPS, W = G::W;
  constexpr int ROWB = kL1RowPitch * G::EB;
  static_assert(S % QN == 0, "fragment queue must line up");
  auto frag = [&](int j, int s) {  // kernel row s / CPR is three halo rows further down
    return *reinterpret_cast<const v4i *>(smem + l1fast[j] + (s / CPR) * 3 * ROWB + (s % CPR) * 16);
  };
  v4i bq[QN][3];
#pragma unroll
  for (int a = 0; a < kAhead; ++a)
#pragma unroll
    for (int j = 0; j < 3; ++j) bq[a][j] = frag(j, a);
  static_for<0, S>([&](auto sc) __attribute__((always_inline)) {
    constexpr int s = decltype(sc)::value;
    if constexpr (s + kAhead < S) {
#pragma unroll
      for (int j = 0; j < 3; ++j) bq[(s + kAhead) % QN][j] = frag(j, s + kAhead);
    }
#pragma unroll
    for (int w = 0; w < W; ++w) {
      constexpr int f0 = s * W;
#pragma unroll
      for (int j = 0; j < 3; ++j) mma<P>(ring[(f0 + w) % D][0], bq[s % QN][j], acc[0][j]);
      ring[(f0 + w) % D][0] = wl[f0 + w + D];  // (the tail over-reads the zero fragments behind the stream)
    }
    interleave_step<3 * W, 3, W>();
    __builtin_amdgcn_sched_barrier(0);
  });
}

// ------------------------------------------------------------------------
// 3x3 layers: K = (tap, cin), cin fastest; taps are constant position offsets
// ------------------------------------------------------------------------
template <class P, int CIN, int COUT>
__device__ __forceinline__ void conv3_pass(const unsigned char *smem, const WFrags &wl,
                                           v4i (&ring)[kRing][COUT / 32], const int (&ci)[3], int h,
                                           f32x16 (&acc)[COUT / 32][3]) {
  using G = Geo<P>;
  constexpr int NT = COUT / 32;
  constexpr int KC = CIN / G::KSTEP;
  constexpr int U = 3 * KC;  // k-steps of one kernel row
  constexpr int D = kRing;
  static_assert(U % D == 0, "ring depth must divide the k-steps of a kernel row");

  // LDS address of logical record offset `o` at tap (j, kx): pb + (x ^ o), x = lane-half ^ swizzle
  int pb[3][3], xo[3][3];
  auto set_row = [&](int ky) {
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
      for (int kx = 0; kx < 3; ++kx) {
        const int pos = ci[j] + (ky - 1) * kPitch + (kx - 1);
        pb[j][kx] = pos * G::PIXB;
        xo[j][kx] = (h << 4) ^ swz_of<P>(pos);
      }
  };
  auto frag_at = [&](int j, int kx, int o) {
    if constexpr (G::PADDED) {
      return *reinterpret_cast<const v4i *>(smem + pb[j][kx] + xo[j][kx] + o);
    } else {
      return *reinterpret_cast<const v4i *>(smem + pb[j][kx] + (xo[j][kx] ^ o));
    }
  };
  set_row(0);
  static_assert(U % (kAhead + 1) == 0 && kAhead <= KC, "fragment queue must line up across kernel rows");
  v4i bq[kAhead + 1][3];
#pragma unroll
  for (int a = 0; a < kAhead; ++a)
#pragma unroll
    for (int j = 0; j < 3; ++j) bq[a][j] = frag_at(j, 0, a * 32);

#pragma unroll 1
  for (int ky = 0; ky < 3; ++ky) {
    const WFrags wn = wl + (ky * U + D) * NT;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // fetch the activation fragments of k-step u + kAhead while this step's MFMAs run
      // (after the last tap this wraps to kernel row 0: harmless extra fetches)
      if (u + kAhead == U) set_row(ky == 2 ? 0 : ky + 1);
      constexpr int QN = kAhead + 1;
      const int un = (u + kAhead) % U;
      const int kxn = un / KC, on = (un % KC) * 32;
#pragma unroll
      for (int j = 0; j < 3; ++j) bq[(u + kAhead) % QN][j] = frag_at(j, kxn, on);
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < 3; ++j) mma<P>(ring[u % D][t], bq[u % QN][j], acc[t][j]);
      // weights of k-step u+D (the tail over-reads into the next layer)
#pragma unroll
      for (int t = 0; t < NT; ++t) ring[u % D][t] = wn[u * NT + t];
      interleave_step<NT * 3 * (P::EB == 4 ? 4 : 1), 3, NT>();
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// Second pass of the bf16 + fp6 mode over a 3x3 layer: acc += Wlo * LO, both e2m3, K = 64 per
// MFMA.  Lane half h of chunk c contracts half-chunk g = 2c + h = (tap, 32-channel block); the
// block's scale byte rides in dword 6 of the 32 bytes the lane reads.
//
// Its weight ring: a lane's operand is 24 bytes, piece 0 = 16 bytes and piece 1 = 8.  (Filling
// the ring before the layer's main pass was measured slower: the extra loads and registers cost
// the main pass more than the second pass gains.)
template <class P>
__device__ __forceinline__ void lo_load_pieces(const WFrags &src, v4i &p0, v4i &p1) {
  p0 = src[0];
  const v2i q = src.dense8(1);
  p1 = v4i{q[0], q[1], 0, 0};
}
template <class P, int L> struct LoRing {
  static constexpr int NT = kCoutArr[L] / 32;
  static constexpr int NC = Geo<P>::lo_chunks(L);
  // ring depth in 64-wide chunks: the weights of a chunk are asked for D chunks before its MFMAs
  static constexpr int D = P::LO6 ? kLoRing : 1;
  __device__ __forceinline__ static WFrags base(const unsigned char *packed, int lane) {
    return packed_frags<P>(packed, lane, Geo<P>::lo_frag_offset(L));
  }
};
template <class P, int L, int D, int NT>
__device__ __forceinline__ void lo_preload(v4i (&f0)[D][NT], v4i (&f1)[D][NT],
                                           const unsigned char *packed, int lane) {
  static_assert(D == LoRing<P, L>::D && NT == LoRing<P, L>::NT, "ring shape");
  const WFrags wl = LoRing<P, L>::base(packed, lane);
#pragma unroll
  for (int d = 0; d < D; ++d)
#pragma unroll
    for (int t = 0; t < NT; ++t) lo_load_pieces<P>(wl + (d * NT + t) * 2, f0[d][t], f1[d][t]);
  __builtin_amdgcn_sched_barrier(0);  // issue here: do not sink the loads to their first use
}

// A runtime loop over groups of D chunks (D = ring depth) keeps the compiler from hoisting
// every fragment load of the layer to the front.
//   INIT: the accumulators are undefined on entry; the first chunk's MFMAs start from `bias`
//   wb[j]: byte address of the lane's position record + 8 * lane half (what the epilogue stores
//   through): the pass has no address registers of its own
template <class P, int L, bool INIT, int D, int NT>
__device__ __forceinline__ void conv3_lo_pass(const unsigned char *smem,
                                              const unsigned char *packed, int scale_w,
                                              v4i (&ring0)[D][NT], v4i (&ring1)[D][NT],
                                              const int (&wb)[3], int h, int lane,
                                              f32x16 (&acc)[NT][3], const f32x16 (&bias)[NT]) {
  using G = Geo<P>;
  static_assert(D == LoRing<P, L>::D && NT == kCoutArr[L] / 32, "ring shape");
  constexpr int PER32 = kCinArr[L] / 32;
  constexpr int HC = G::lo_half_chunks(L), NC = G::lo_chunks(L);
  typedef int v8i __attribute__((ext_vector_type(8)));
  const WFrags wl = LoRing<P, L>::base(packed, lane);
  // scale_w: E8M0 exponent undoing the weight copy's 2^sw.  (It arrives as an argument, read once
  // per board: a load here would be the newest of ~36 loads in flight, and waiting for it before the
  // first MFMA would drain them all.)

  // Byte offset of a half-chunk relative to wb[].  Half-chunk g = 2 c + (lane half) of chunk
  // c = 3 grp + dd is g = 6 grp + r with r = 2 dd + half: with `r` a constant, the tap and the
  // channel block of g need no division by the tile count, and for 64 input channels (6
  // half-chunks = 3 taps = one kernel row) no division at all.  The group number may be a
  // run-time value (scalar unit); both halves' offsets are formed and the lane half selects.
  // (The lane half through an opaque copy: the selected offsets of the unrolled chunks are then
  // formed in this pass and not once per kernel, in registers that get spilled.)
  static_assert(D == 3, "the half-chunk arithmetic below assumes groups of three chunks");
  int hh = h;
  asm volatile("" : "+v"(hh));
  auto off_g = [&](int grp, int r) __attribute__((always_inline)) {
    int ky, kx, cb;
    if constexpr (PER32 == 3) {
      const unsigned tap = 2u * (unsigned)grp + (unsigned)(r / 3);
      cb = r % 3;
      ky = (int)(tap / 3u);
      kx = (int)tap - 3 * ky;
    } else if constexpr (PER32 == 2) {
      cb = r % 2;
      ky = grp + (r / 2) / 3;
      kx = (r / 2) % 3;
    } else {
      static_assert(PER32 == 1, "32, 64 or 96 input channels");
      cb = 0;
      ky = 2 * grp + r / 3;
      kx = r % 3;
    }
    return ((ky - 1) * kPitch + (kx - 1)) * G::PIXB + cb * 32 + G::LO_OFF;
  };
  // chunk 3 grp + dd; STATIC: grp is a constant after unrolling, and the chunk may lie beyond the
  // last one (harmless re-reads of the last) or hold the padding half-chunk (which re-reads the
  // half-chunk before it: its weights are zero)
  auto fetch = [&](int grp, int dd, auto is_static, v4i (&b)[3][2]) __attribute__((always_inline)) {
    auto of_chunk = [&](int c, int &o0, int &o1) __attribute__((always_inline)) {  // constant c
      c = c < NC ? c : NC - 1;
      const int g0 = 2 * c, g1 = 2 * c + 1 < HC ? 2 * c + 1 : HC - 1;
      o0 = off_g(g0 / 6, g0 % 6);
      o1 = off_g(g1 / 6, g1 % 6);
    };
    int o0, o1;
    if constexpr (decltype(is_static)::value) {
      of_chunk(D * grp + dd, o0, o1);
    } else {
      // (run-time group: never the last chunk nor beyond it, see the loop bounds below)
      o0 = off_g(grp, 2 * dd);
      o1 = off_g(grp, 2 * dd + 1);
    }
    const int off = hh ? o1 - 8 : o0;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      b[j][0] = *reinterpret_cast<const v4i *>(smem + wb[j] + off);
      // The last two data dwords with an 8-byte read, straight into the operand's registers 4
      // and 5, and the scale on its own (volatile: the compiler would merge the two into one
      // 12-byte read again, whose three registers cannot be part of the six-register operand,
      // and copy two of them; a 16-byte read would leave a dead register that the compiler
      // reuses at once, waiting for the read to land first).
      const v2i q = *reinterpret_cast<const v2i *>(smem + wb[j] + off + 16);
      typedef const volatile __attribute__((address_space(3))) int *LdsVolatileInt;
      const int sc = *(LdsVolatileInt)(smem + wb[j] + off + 24);
      b[j][1] = v4i{q[0], q[1], sc, sc};
    }
  };
  // activation blocks are fetched kAhead chunks ahead, like the main pass's fragments
  static_assert(D % (kAhead + 1) == 0 && NC > kAhead, "low-order ring and fragment queue shapes");
  v4i bq[kAhead + 1][3][2];
#pragma unroll
  for (int a = 0; a < kAhead; ++a) fetch(0, a, IC<1>{}, bq[a]);
  // chunk 3 grp + d: its MFMAs, the LDS reads of the chunk kAhead further on and the refill of
  // ring slot d
  auto chunk = [&](int grp, int d, auto first, auto is_static) __attribute__((always_inline)) {
    const WFrags wn = wl + (grp + 1) * (D * NT * 2);
    v4i(&bcur)[3][2] = bq[d % (kAhead + 1)];
    fetch(grp + (d + kAhead) / D, (d + kAhead) % D, is_static, bq[(d + kAhead) % (kAhead + 1)]);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const v8i a = __builtin_shufflevector(ring0[d][t], ring1[d][t], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const v8i b = __builtin_shufflevector(bcur[j][0], bcur[j][1], 0, 1, 2, 3, 4, 5, 6, 7);
        f32x16 c;
        if constexpr (decltype(first)::value) {
          c = bias[t];
        } else {
          c = acc[t][j];
        }
        acc[t][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 2, 2, 0, scale_w, 0, b[6]);
      }
    }
    // weights of chunk c0 + d + D (the tail over-reads the next layer's copy or the zero padding)
#pragma unroll
    for (int t = 0; t < NT; ++t) lo_load_pieces<P>(wn + (d * NT + t) * 2, ring0[d][t], ring1[d][t]);
    interleave_step<NT * 3, 2 * 3, 2 * NT>();
    __builtin_amdgcn_sched_barrier(0);
  };
  // Whole groups of D chunks in a runtime loop with a single basic block (a branch inside the
  // body makes the compiler wait for every LDS read in flight at each group boundary), then the
  // chunks that are left, unrolled.  The loop only takes the groups whose reads ahead stay in
  // front of the last chunk, so that its body needs neither of the two special cases (a select
  // per read costs more than the longer unrolled tail).
  constexpr int LIM = NC - 2 - (D - 1) - kAhead;  // last chunk such a group may start at
  constexpr int GROUPS = LIM >= 0 ? LIM / D + 1 : 0;
  constexpr int FIRST = INIT ? 1 : 0;
  static_assert(NC >= D, "at least one whole group");
  if constexpr (INIT) {  // (the first group apart: its first chunk initialises the accumulators)
    chunk(0, 0, IC<1>{}, IC<1>{});
#pragma unroll
    for (int d = 1; d < D; ++d) chunk(0, d, IC<0>{}, IC<1>{});
  }
#pragma unroll 1
  for (int grp = FIRST; grp < GROUPS; ++grp) {
#pragma unroll
    for (int d = 0; d < D; ++d) chunk(grp, d, IC<0>{}, IC<0>{});
  }
  constexpr int REST = (GROUPS > FIRST ? GROUPS : FIRST) * D;
#pragma unroll
  for (int c = REST; c < NC; ++c) chunk(c / D, c % D, IC<0>{}, IC<1>{});
}

// SiLU of the four accumulators (tile t, pixel tile j, quad q): bias was added at init
template <class P, int NT>
__device__ __forceinline__ Packed4<P> silu_quad(const f32x16 (&acc)[NT][3], int t, int j, int q) {
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = silu<P>(acc[t][j][4 * q + e]);
  return pack4<P>(v);
}

// SiLU + store of one pixel tile's accumulators (all cout tiles).  Lanes beyond pixel
// 360 shadow pixel 360 (same inputs, same results, same address), so every lane stores
// unconditionally.  The lane's addresses are recomputed here every time: hoisted out of the
// board loop they would occupy ~100 registers for the whole kernel and end up in scratch.
template <class P, int NT>
__device__ __forceinline__ void store_tile(unsigned char *smem, int pos_in, int h,
                                           const f32x16 (&acc)[NT][3], int j) {
  using G = Geo<P>;
  int pos = pos_in;
  asm volatile("" : "+v"(pos));
  const int pbase = pos * G::PIXB;
  const int sw = swz_of<P>(pos);
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q)
      put4<P>(smem, pbase, sw, (32 * t + 8 * q + 4 * h) * G::EB, silu_quad<P, NT>(acc, t, j, q));
}

// fp6 mode: 32 low-order values of one position -> 24 bytes of e2m3 + the block's E8M0 scale.
// The scale is 2^(E-2) for a largest magnitude in [2^E, 2^(E+1)), so values land in (-8, 8)
// and the conversion saturates the few above 7.5.  even[i] goes to K slot 2i, odd[i] to 2i+1.
typedef float f32x16v __attribute__((ext_vector_type(16)));
typedef unsigned u32x6 __attribute__((ext_vector_type(6)));
__device__ __forceinline__ u32x6 to_fp6_block(const f32x16v &even, const f32x16v &odd, float scale) {
  u32x6 r = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(even, odd, scale);
  // the instruction must not write where it still reads: keep every source live past it
  asm volatile("" : "+v"(r) : "v"(even), "v"(odd), "v"(scale));
  return r;
}
typedef const __attribute__((address_space(1))) float *GlobalF32;
typedef const __attribute__((address_space(1))) f32x4 *GlobalF32x4;

// accumulators start at the layer's bias: lane (h) register i holds channel 32t + 8(i/4) + 4h + i%4
template <int N>
__device__ __forceinline__ void init_acc(f32x16 (&acc)[N][3], const float *__restrict__ bias, int h) {
  const float *blg = bias + 4 * h;  // one per-lane base; every load below is base + constant
  asm volatile("" : "+v"(blg));
  // (the laundering hides that this is global memory; say so again, or the loads become flat
  // loads, which also count against the LDS counter)
  const GlobalF32 bl = (GlobalF32)blg;
#pragma unroll
  for (int t = 0; t < N; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x4 b4 = *(GlobalF32x4)(bl + 32 * t + 8 * q);
#pragma unroll
      for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[t][j][4 * q + e] = b4[e];
    }
}

// the layer's bias as the lane sees it in an accumulator tile: register i of cout tile t holds
// channel 32t + 8(i/4) + 4h + i%4.  The first MFMA of each accumulator takes this as its C
// operand, so the accumulators themselves are never initialised.
template <int N>
__device__ __forceinline__ void load_bias_tiles(f32x16 (&bt)[N], const float *__restrict__ bias, int h) {
  const float *blg = bias + 4 * h;
  asm volatile("" : "+v"(blg));
  const GlobalF32 bl = (GlobalF32)blg;
#pragma unroll
  for (int t = 0; t < N; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x4 b4 = *(GlobalF32x4)(bl + 32 * t + 8 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) bt[t][4 * q + e] = b4[e];
    }
}

// the same from the copy of the tail in LDS (`tail_lds`: byte address of the copy)
template <int N>
__device__ __forceinline__ void load_bias_tiles_lds(f32x16 (&bt)[N], const unsigned char *smem,
                                                    int tail_lds, int layer_off, int h) {
  // one address register, made opaque here: otherwise every address below is computed once per
  // kernel, kept in a register of its own and ends up in scratch memory (and so would the sum
  // below, per layer, were the layer's constant added in front of the asm statement)
  int base = 16 * h;
  asm volatile("" : "+v"(base));
  base += tail_lds + 4 * layer_off;
  // (opaque again behind the sum: the copy sits beyond the 64 KiB that an LDS instruction's
  // offset field reaches, and folded into one constant per read it costs an addition per read)
  asm volatile("" : "+v"(base));
#pragma unroll
  for (int t = 0; t < N; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x4 b4 = *reinterpret_cast<const f32x4 *>(smem + base + 4 * (32 * t + 8 * q));
#pragma unroll
      for (int e = 0; e < 4; ++e) bt[t][4 * q + e] = b4[e];
    }
}

// barrier; every wave writes its share of the layer's output over the layer's input; barrier
template <class P, int NT, class Pre>
__device__ __forceinline__ void finish_layer(unsigned char *smem, const int (&ci)[3], int h,
                                             const f32x16 (&acc)[NT][3], Pre before_store) {
  __syncthreads();  // every wave has finished reading the layer's input
  before_store();
#pragma unroll
  for (int j = 0; j < 3; ++j) store_tile<P, NT>(smem, ci[j], h, acc, j);
  __syncthreads();
}

// one 3x3 layer that is not the last (layer-by-layer kernel)
template <class P, int L>
__device__ __forceinline__ void mid_layer(
    unsigned char *smem, const unsigned char *packed, const float *tail,
    v4i (&ring)[kRing][kCoutArr[L] / 32], v4i (&next)[kRing][kCoutArr[L + 1] / 32],
    const int (&ci)[3], int h, int lane, int wave, bool trace_on) {
  constexpr int CIN = kCinArr[L], COUT = kCoutArr[L], NT = COUT / 32;
  f32x16 acc[NT][3];
  init_acc(acc, tail + bias_offset(L), h);
  conv3_pass<P, CIN, COUT>(smem, layer_weights<P, L>(packed, lane), ring, ci, h, acc);
  C6_MARK(30 + L);
  // With equal channel counts the main pass's over-read has already left the next layer's first
  // kRing k-steps in the ring (same fragment order, contiguous in memory): `next` is `ring`.
  if constexpr (kCoutArr[L + 1] != kCoutArr[L])
    preload_ring<kRing, kCoutArr[L + 1] / 32>(next, layer_weights<P, L + 1>(packed, lane));
  C6_MARK(4 + 2 * L);
  finish_layer<P, NT>(smem, ci, h, acc, [] {});
  C6_MARK(5 + 2 * L);
  (void)wave;
  (void)trace_on;
}

// ------------------------------------------------------------------------
// Pipelined kernel (16-bit modes with padded records: bf16, fp16, bf16 + fp6).
//
// With one wave per SIMD nothing runs beside a wave's own instruction stream, and the SiLU
// epilogue of a layer (two transcendentals per element) used to run with the matrix pipe idle.
// A few VALU instructions issued behind each MFMA of a K-loop cost little (a lone wave issues
// one instruction per ~5 cycles and an MFMA occupies the matrix pipe for 32), so the epilogues
// are issued from inside K-loops.  A 3x3 layer's K is ordered phase-major, a phase being all nine
// taps of 32 input channels = one cout tile of the layer before.  Phase p carries the epilogue of
// tile p+1 of the layer before (whose accumulators stay live next to this layer's), and the last
// phase runs cout tile 0 first and carries that tile's own epilogue behind the other tiles' MFMAs
// (pipe_layer).  Only single-tile layers convert anything with the matrix pipe idle.
// ------------------------------------------------------------------------
constexpr int kPhaseSteps = 18;   // k-steps of one phase: 9 taps x 2 k-steps of 16 channels

// The epilogue of one cout tile (SiLU, bf16 store, low-order fp6 blocks) as a list of atoms --
// single instructions or short groups -- that a compile-time schedule deals out over the MFMA
// slots of a K-loop segment.  A lone wave issues one instruction every ~5 cycles and an MFMA
// occupies the matrix pipe for 32, so about six instructions fit into a slot, the MFMA, the
// K-loop's own LDS reads, weight loads and waits included; measured, about two VALU instructions
// per slot ride for free and every further one costs its full issue time.  The schedule
// therefore spreads the atoms evenly: every slot gets the same small budget.
// The lane's elements (3 pixel tiles x its channels of the cout tile) stream through a software
// pipeline, so that consecutive atoms never depend on each other:
//   step s:  exp2 of element s | 1 + . of element s-1 | rcp of element s-2 | x * . of element s-3
//            | pack pair | low-order parts of a pair | running maximum over a pair | store quad
//            | the three stages that build a pixel tile's fp6 block
enum : int { kAtE, kAtA, kAtR, kAtM, kAtC, kAtD, kAtX, kAtW, kAtF1, kAtF2, kAtF3, kAtKinds };
__host__ __device__ constexpr int atom_cost(int kind) {  // issue cycles, roughly
  constexpr int cost[kAtKinds] = {10, 5, 10, 5, 5, 10, 5, 5, 15, 20, 30};
  return cost[kind];
}

// Which elements an epilogue covers: channels (accumulator registers) [I0, I0 + CNT) of each of
// the three pixel tiles; CNT is a multiple of 4 (a stored quad = 4 consecutive channels).
template <int I0_, int CNT_> struct EpiRange {
  static constexpr int I0 = I0_, CNT = CNT_, N = 3 * CNT_;
};

struct EpiSched {
  static constexpr int MAXS = 256, MAXA = 10;
  unsigned short atom[MAXS][MAXA];  // kind << 8 | index (element, pair, quad or pixel tile)
  unsigned char count[MAXS];
  int slots;                        // slots that hold atoms
};

// Atoms in pipeline order, packed into slots of `budget` cycles each.
//   n_elems: elements in the stream (3 * CNT); lo6: low-order atoms too; finish: the pixel
//   tiles' fp6 blocks are built here (all 16 channels of the tile have been through)
__host__ __device__ constexpr EpiSched pack_sched(int cnt, bool lo6, bool finish, int budget) {
  EpiSched sc{};
  const int N = 3 * cnt, NP = N / 2, NQ = N / 4;
  int slot = 0, used = 0;
  auto put = [&](int kind, int idx) {
    const int c = atom_cost(kind);
    if (sc.count[slot] > 0 && (used + c > budget || sc.count[slot] == EpiSched::MAXA)) {
      ++slot;
      used = 0;
    }
    sc.atom[slot][sc.count[slot]++] = (unsigned short)(kind << 8 | idx);
    used += c;
  };
  const int last_step = N + 12;
  for (int s = 0; s <= last_step; ++s) {
    if (s < N) put(kAtE, s);
    if (s - 1 >= 0 && s - 1 < N) put(kAtA, s - 1);
    if (s - 2 >= 0 && s - 2 < N) put(kAtR, s - 2);
    if (s - 3 >= 0 && s - 3 < N) put(kAtM, s - 3);
    // pair P = elements 2P, 2P+1: packed at step 2P+5, low-order parts at 2P+6, maximum at 2P+8
    if (s >= 5 && (s - 5) % 2 == 0 && (s - 5) / 2 < NP) put(kAtC, (s - 5) / 2);
    if (lo6 && s >= 6 && (s - 6) % 2 == 0 && (s - 6) / 2 < NP) put(kAtD, (s - 6) / 2);
    if (lo6 && s >= 8 && (s - 8) % 2 == 0 && (s - 8) / 2 < NP) put(kAtX, (s - 8) / 2);
    // quad Q = pairs 2Q, 2Q+1: stored at step 4Q+8
    if (s >= 8 && (s - 8) % 4 == 0 && (s - 8) / 4 < NQ) put(kAtW, (s - 8) / 4);
    // pixel tile j: its last pair's maximum is taken at step 2 * (cnt/2 * (j+1) - 1) + 8
    if (lo6 && finish) {
      for (int j = 0; j < 3; ++j) {
        const int after = 2 * (cnt / 2 * (j + 1) - 1) + 8;
        if (s == after + 1) put(kAtF1, j);
        if (s == after + 2) put(kAtF2, j);
        if (s == after + 3) put(kAtF3, j);
      }
    }
  }
  sc.slots = slot + 1;
  return sc;
}
// the smallest budget (multiple of 5) that fits the stream into `slots` slots
__host__ __device__ constexpr EpiSched make_sched(int cnt, bool lo6, bool finish, int slots) {
  for (int budget = 10; budget < 200; budget += 5) {
    const EpiSched sc = pack_sched(cnt, lo6, finish, budget);
    if (sc.slots <= slots) return sc;
  }
  return pack_sched(cnt, lo6, finish, 1000);
}

struct EpiCarry {
  float e[4];       // sigmoid denominators in flight (element n at n % 4)
  float v[8];       // activations (fp32) until they are packed and their low-order parts taken
  int hi[4];        // packed bf16 pairs until they are stored (pair P at P % 4)
  float lo[2][16];  // what the rounding dropped, per pixel tile (two tiles in flight)
  float m[2];       // their largest magnitude
  int sc[2];
};

// One atom of the epilogue of cout tile t (accumulators `acc`), channels per EpiRange R.
//   wb[j]: byte address of the lane's position record + 8 * lane half;  h4 = 4 * lane half
//   blk: the record's 32-channel block that receives the tile (its fp6 block goes to block t)
// UNDER_MFMA: the atom is issued while matrix instructions are in flight.  v_dot2c_f32_bf16 then
// costs the matrix pipe ~20 cycles per group (measured: one MFMA + two of them take 56 cycles
// instead of 33, one MFMA + four plain VALU instructions 35), so the low-order parts are taken
// with an unpack and a subtract there.
template <class P, int NT, class R, bool UNDER_MFMA>
__device__ __forceinline__ void epi_atom(unsigned char *smem, const int (&wb)[3], int h4,
                                         const f32x16 (&acc)[NT][3], int t, int blk, int code,
                                         EpiCarry &c, const DropConsts &k) {
  using G = Geo<P>;
  const int kind = code >> 8, idx = code & 255;
  auto tile_of = [](int n) __attribute__((always_inline)) { return n / R::CNT; };
  auto reg_of = [](int n) __attribute__((always_inline)) { return R::I0 + n % R::CNT; };
  if (kind == kAtE) {
    c.e[idx % 4] = __builtin_amdgcn_exp2f(acc[t][tile_of(idx)][reg_of(idx)]);
  } else if (kind == kAtA) {
    c.e[idx % 4] = 1.0f + c.e[idx % 4];
  } else if (kind == kAtR) {
    c.e[idx % 4] = __builtin_amdgcn_rcpf(c.e[idx % 4]);
  } else if (kind == kAtM) {
    c.v[idx % 8] = acc[t][tile_of(idx)][reg_of(idx)] * c.e[idx % 4];
  } else if (kind == kAtC) {
    c.hi[idx % 4] = pack2<P>(c.v[(2 * idx) % 8], c.v[(2 * idx + 1) % 8]);
  } else if (kind == kAtD) {
    const int b = tile_of(2 * idx) & 1, i = reg_of(2 * idx);
    if constexpr (UNDER_MFMA) {
      const int w = c.hi[idx % 4];
      c.lo[b][i] = c.v[(2 * idx) % 8] - __builtin_bit_cast(float, w << 16);
      c.lo[b][i + 1] = c.v[(2 * idx + 1) % 8] - __builtin_bit_cast(float, w & (int)0xffff0000);
    } else {
      c.lo[b][i] = dropped_lo(c.v[(2 * idx) % 8], c.hi[idx % 4], k);
      c.lo[b][i + 1] = dropped_hi(c.v[(2 * idx + 1) % 8], c.hi[idx % 4], k);
    }
  } else if (kind == kAtX) {
    // largest magnitude: med3(|x|, m, inf) = max(|x|, m); the compiler folds two of them into
    // one v_max3_f32 with |.| modifiers.  (Not an asm statement: a dot2 result needs three
    // wait states before another VALU instruction may read it, and the compiler keeps them
    // only for instructions it can see.)
    const int b = tile_of(2 * idx) & 1, i = reg_of(2 * idx);
    float m = i == 0 ? 0.0f : c.m[b];
    m = __builtin_amdgcn_fmed3f(__builtin_fabsf(c.lo[b][i]), m, __builtin_inff());
    m = __builtin_amdgcn_fmed3f(__builtin_fabsf(c.lo[b][i + 1]), m, __builtin_inff());
    c.m[b] = m;
  } else if (kind == kAtW) {
    const int j = tile_of(4 * idx), q = reg_of(4 * idx) / 4;
    *reinterpret_cast<v2i *>(smem + wb[j] + 64 * blk + 16 * q) = v2i{c.hi[(2 * idx) % 4], c.hi[(2 * idx + 1) % 4]};
  } else if constexpr (P::LO6) {
    // fp6 block of pixel tile j = idx: the tile's 32 channels of a position sit in two lanes
    // (lane halves), 16 each.  They agree on the scale (2^(E-2) for a largest magnitude in
    // [2^E, 2^(E+1)), so values land in (-8, 8)); then each converts its own 16 values into 16
    // K slots = 12 bytes: the lower lane's go to bytes 0-11 of the block, the upper lane's to
    // bytes 12-23, the scale to byte 24.
    const int j = idx, b = j & 1;
    if (kind == kAtF1) {
      const unsigned mb = __builtin_bit_cast(unsigned, c.m[b]);
      const auto x = __builtin_amdgcn_permlane32_swap(mb, mb, false, false);
      const unsigned x0 = x[0], x1 = x[1];
      c.m[b] = __builtin_bit_cast(float, x0 > x1 ? x0 : x1);  // (non-negative floats order like integers)
    } else if (kind == kAtF2) {
      const int sc = (__builtin_bit_cast(int, c.m[b]) >> 23) - 2;  // biased exponent of the block scale
      c.sc[b] = sc < 1 ? 1 : sc;
    } else if (kind == kAtF3) {
      // slot 2i <- first[i], slot 2i+1 <- second[i]; only slots 0-15 (i < 8) are kept.  The upper
      // halves are never used, but the instruction reads them: left undefined they get registers
      // that weight loads in flight are about to write, and the hardware then waits for every
      // such load before the conversion.  So the upper half of each operand is eight registers
      // that an empty asm statement "defines" (no instruction; they are only reserved for the
      // length of the conversion).
      typedef float f32x8v __attribute__((ext_vector_type(8)));
      f32x8v p0, p1, fill0, fill1;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        p0[i] = c.lo[b][i];
        p1[i] = c.lo[b][8 + i];
      }
      asm volatile("" : "=v"(fill0));
      asm volatile("" : "=v"(fill1));
      const f32x16v first = __builtin_shufflevector(p0, fill0, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
      const f32x16v second = __builtin_shufflevector(p1, fill1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
      const u32x6 r = to_fp6_block(first, second, __builtin_bit_cast(float, c.sc[b] << 23));
      unsigned char *dst = smem + wb[j] + G::LO_OFF + 32 * t;  // + 8h from wb: data at + 4h more = 12h
      // (three dwords at a 4-byte aligned address: dword stores)
      int *d32 = reinterpret_cast<int *>(dst + h4);
      d32[0] = (int)r[0];
      d32[1] = (int)r[1];
      d32[2] = (int)r[2];
      *reinterpret_cast<int *>(dst - h4 + 24) = c.sc[b];  // byte 24 (lower lane) / 28 (upper lane: unused)
    }
  }
}

// A schedule as a type: the epilogue of channels R over `SLOTS` MFMA slots.
template <class P, class R, bool LO, bool FINISH, int SLOTS> struct EpiPlan {
  static constexpr EpiSched sched = make_sched(R::CNT, LO && P::LO6 != 0, FINISH, SLOTS);
  static_assert(sched.slots <= EpiSched::MAXS, "schedule too long");
  // the atoms of slot g
  template <int NT, bool UNDER_MFMA = true>
  __device__ __forceinline__ static void run(unsigned char *smem, const int (&wb)[3], int h4,
                                             const f32x16 (&acc)[NT][3], int t, int blk, int g,
                                             EpiCarry &c, const DropConsts &k) {
    if (g >= sched.slots) return;
#pragma unroll
    for (int a = 0; a < EpiSched::MAXA; ++a)
      if (a < sched.count[g])
        epi_atom<P, NT, R, UNDER_MFMA>(smem, wb, h4, acc, t, blk, sched.atom[g][a], c, k);
  }
  // everything at once (no MFMAs to ride behind)
  template <int NT>
  __device__ __forceinline__ static void run_all(unsigned char *smem, const int (&wb)[3], int h4,
                                                 const f32x16 (&acc)[NT][3], int t, int blk,
                                                 EpiCarry &c, const DropConsts &k) {
    static_for<0, sched.slots>([&](auto gc) __attribute__((always_inline)) {
      run<NT, false>(smem, wb, h4, acc, t, blk, decltype(gc)::value, c, k);
    });
  }
};

// Where the 32-channel tiles of an activation live in a position's record.  The record has three
// 64-byte blocks; input tile p of 3x3 layer l sits in block (act_rot(l) + p) % 3 and output tile t
// goes to block (act_rot(l + 1) + t) % 3 with act_rot(l + 1) = act_rot(l) + (input tiles of l).
// Output tile 0 is written while the layer's last input tile is still being read (see
// pipe_layer), so it must not land on that tile's block: it takes the next one, which holds
// either input tile 0 (read long ago) or nothing.  The fp6 block of tile t is always block t of
// the low-order area: it is only written once the layer's low-order pass has read all of them.
__host__ __device__ constexpr int act_rot(int l) {
  int r = 0;
  for (int i = 1; i < l; ++i) r = (r + kCinArr[i] / 32) % 3;
  return r;
}

// Fragment order of a 3x3 layer's weights in the pipelined kernel: phase-major (a phase = the nine
// taps of one input tile = 18 k-steps of 16 channels), inside a phase k-step-major, then cout tile
// -- except the last phase of a layer with several cout tiles, which first runs all k-steps of
// cout tile 0 (part A) and then all k-steps of the other tiles (part B).
struct PipeFrag {
  int ph, u, t;
};
__host__ __device__ constexpr PipeFrag pipe_frag(int cin, int cout, int fi) {
  const int nt = cout / 32, ntp = cin / 32, per = kPhaseSteps * nt;
  const int ph = fi / per, r = fi % per;
  if (ph == ntp - 1 && nt > 1) {
    if (r < kPhaseSteps) return PipeFrag{ph, r, 0};
    const int r2 = r - kPhaseSteps;
    return PipeFrag{ph, r2 / (nt - 1), 1 + r2 % (nt - 1)};
  }
  return PipeFrag{ph, r / nt, r % nt};
}

// One segment of a 3x3 layer's K-loop: a whole phase (all cout tiles), or part A / part B of the
// last phase.  Every MFMA opens a slot that ends with a scheduling barrier: the MFMA, at most
// two memory instructions (the activation fragments of two k-steps ahead, the weight fragment
// that replaces the one whose last MFMA this was) and a few instructions of an epilogue.
//   rb[j]: byte address of the record one row and one column before the lane's position, + 16 * lane half
//   wl:    the layer's first weight fragment; `ring` is a FIFO over the layer's fragment stream
//          (fragment f in slot f % RN), which runs on into the next layer
//   bq:    activation fragments of k-step ks at ks % 3; part B continues part A's k-step count
//   hidden(g): epilogue work to issue in slot g
//   bias:  the accumulators are undefined before a tile's first k-step, whose MFMAs start from these
enum : int { kSegFull, kSegA, kSegB };
template <class P, int L, int KIND, int PH, class Hidden>
__device__ __forceinline__ void conv3_seg(const unsigned char *smem, const WFrags &wl,
                                          v4i (&ring)[kRing * (kCoutArr[L] / 32)], v4i (&bq)[kAhead + 1][3],
                                          const int (&rb)[3], f32x16 (&acc)[kCoutArr[L] / 32][3],
                                          const f32x16 (&bias)[kCoutArr[L] / 32], Hidden hidden) {
  using G = Geo<P>;
  constexpr int NT = kCoutArr[L] / 32, NTP = kCinArr[L] / 32, W = G::W;
  constexpr int U = kPhaseSteps, RN = kRing * NT, QN = kAhead + 1;
  constexpr int T0 = KIND == kSegB ? 1 : 0;
  constexpr int NTS = KIND == kSegFull ? NT : (KIND == kSegA ? 1 : NT - 1);
  // (WLO: every weight fragment is followed by the fragment of what its rounding dropped; the two
  // meet the same activation fragment and the same accumulator, so a tile takes W MFMAs per
  // k-step and pixel tile, and the ring, unchanged in size, reaches kRing / W k-steps ahead)
  constexpr int NV = NTS * W;
  constexpr int F0 = (PH * U * NT + (KIND == kSegB ? U : 0)) * W;
  constexpr int KS0 = KIND == kSegB ? U : 0;
  constexpr int BLK = (act_rot(L) + PH) % 3;
  static_assert(G::KSTEP == 16 && G::PADDED && U % QN == 0 && (U * NTP * NT * W) % RN == 0, "segment shape");
  static_assert(KIND == kSegFull || (PH == NTP - 1 && NT > 1), "parts A and B split the last phase");
  auto frag = [&](int j, int u) {
    const int tap = u / 2;
    const int off = ((tap / 3) * kPitch + tap % 3) * G::PIXB + BLK * 64 + (u % 2) * 32;
    return *reinterpret_cast<const v4i *>(smem + rb[j] + off);
  };
  if constexpr (KIND != kSegB) {
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
#pragma unroll
      for (int j = 0; j < 3; ++j) bq[a][j] = frag(j, a);
  }
  static_for<0, U * NV * 3>([&](auto gc) __attribute__((always_inline)) {
    constexpr int g = decltype(gc)::value;
    constexpr int u = g / (NV * 3), vi = (g / 3) % NV, ti = vi / W, t = T0 + ti, j = g % 3;
    constexpr int f = F0 + u * NV + vi;
    // (a layer with one input tile runs its low-order pass first, and that one starts from the bias)
    constexpr bool kLoFirst = P::LO6 && ((P::LO_MASK >> L) & 1) && NTP == 1;
    if constexpr (PH == 0 && u == 0 && vi % W == 0 && !kLoFirst) {
      f32x16 c0 = bias[t];
      mma<P>(ring[f % RN], bq[(KS0 + u) % QN][j], c0);
      acc[t][j] = c0;
    } else {
      mma<P>(ring[f % RN], bq[(KS0 + u) % QN][j], acc[t][j]);
    }
    // fragments of k-step u + kAhead; part A runs on into part B, which reads the same ones again
    if constexpr (vi == 0 && (u + kAhead < U || KIND == kSegA))
      bq[(KS0 + u + kAhead) % QN][j] = frag(j, (u + kAhead) % U);
    if constexpr (j == 2) ring[f % RN] = wl[f + RN];
    hidden(g);
    __builtin_amdgcn_sched_barrier(0);
  });
}

// One 3x3 layer L (1..7) of the pipelined kernel.  Order of work, for NTP input tiles and NT
// cout tiles:
//   phases 0 .. NTP-2, all cout tiles; phase p carries the epilogue of tile p+1 of layer L-1
//     (whose accumulators arrive in `prev`), with a barrier before the next phase reads it;
//   the low-order pass over the whole input (all of layer L-1 has been written by now);
//   the last phase in two parts: A = cout tile 0 alone, B = the other tiles, carrying the
//     epilogue of this layer's own tile 0, which is final after part A.
// So only single-tile layers convert anything with the matrix pipe idle, and a layer with
// several cout tiles hands `acc` on with tile 0 already stored.
template <class P, int L, class Rezero, class LastHidden>
__device__ __forceinline__ void pipe_layer(
    unsigned char *smem, const unsigned char *packed, int tail_lds,
    v4i (&ring)[kRing * (kCoutArr[L] / 32)], const int (&ci)[3], int h, int lane, int wave,
    bool trace_on, const int (&lo_scale_w)[8], const f32x16 (&prev)[kCinArr[L] / 32][3],
    f32x16 (&acc)[kCoutArr[L] / 32][3], Rezero rezero, LastHidden last_hidden) {
  using G = Geo<P>;
  constexpr int NT = kCoutArr[L] / 32, NTP = kCinArr[L] / 32;
  constexpr int RIN = act_rot(L), ROUT = act_rot(L + 1);
  constexpr bool kLast = (L == 7);  // its output feeds the heads from the accumulators
  int rb[3], wb[3];
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    int pos = ci[j];
    asm volatile("" : "+v"(pos));  // (recomputed per layer: keeps six address registers out of the board loop)
    rb[j] = (pos - kPitch - 1) * G::PIXB + 16 * h;
    wb[j] = pos * G::PIXB + 8 * h;
  }
  const DropConsts k = drop_consts<P>();
  const int h4 = 4 * h;
  EpiCarry carry;
  f32x16 bias[NT];
  v4i bq[kAhead + 1][3];
  using Whole = EpiRange<0, 16>;
  constexpr bool kLoPass = P::LO6 && ((P::LO_MASK >> L) & 1);
  constexpr bool kLoNext = P::LO6 && L + 1 < kLayers && ((P::LO_MASK >> (L + 1)) & 1);  // this layer's output needs its low-order part
  v4i lor0[LoRing<P, L>::D][LoRing<P, L>::NT], lor1[LoRing<P, L>::D][LoRing<P, L>::NT];
  __syncthreads();  // every wave has finished layer L-1 (its reads, and tile 0 if it stored it there)
  if constexpr (NTP == 1) {
    // a single-tile layer L-1 has nothing to hide its epilogue under
    // (a compile-time loop: `#pragma unroll` gives up on a body this size, and a runtime index
    // would put the accumulators into scratch memory)
    rezero();
    // (the low-order ring is asked for in front of the open epilogue, whose arithmetic covers the
    // round trip to L2)
    if constexpr (kLoPass) lo_preload<P, L>(lor0, lor1, packed, lane);
    EpiPlan<P, Whole, kLoPass, true, EpiSched::MAXS>::template run_all<NTP>(smem, wb, h4, prev, 0, RIN, carry, k);
    load_bias_tiles_lds(bias, smem, tail_lds, bias_offset(L), h);
    __syncthreads();
  } else {
    load_bias_tiles_lds(bias, smem, tail_lds, bias_offset(L), h);
  }
  C6_MARK(L == 1 ? 3 : 3 + 2 * L);
  const WFrags wl = layer_weights<P, L>(packed, lane);
  // phases 0 .. NTP-2 carry tiles 1 .. NTP-1 of layer L-1
  static_for<0, NTP - 1>([&](auto pc) __attribute__((always_inline)) {
    constexpr int p = decltype(pc)::value;
    using Plan = EpiPlan<P, Whole, kLoPass, true, kPhaseSteps * NT * G::W * 3 - 8>;
    conv3_seg<P, L, kSegFull, p>(smem, wl, ring, bq, rb, acc, bias, [&](int g) __attribute__((always_inline)) {
      Plan::template run<NTP>(smem, wb, h4, prev, p + 1, (RIN + p + 1) % 3, g, carry, k);
    });
    // (The low-order weight ring is filled in one burst in front of the barrier that precedes its
    // pass.  Dealt out over this phase's MFMA slots instead, the phase gets 4 % shorter and the
    // kernel no faster, for two or three spilled registers.)
    if constexpr (kLoPass && p == NTP - 2) lo_preload<P, L>(lor0, lor1, packed, lane);
    __syncthreads();
  });
  C6_MARK(30 + L);
  if constexpr (kLoPass) {
    conv3_lo_pass<P, L, NTP == 1>(smem, packed, lo_scale_w[L], lor0, lor1, wb, h, lane, acc, bias);
    // before part B overwrites fp6 block 0, every wave must have read it
    if constexpr (NT > 1 && !kLast) __syncthreads();
  }
  C6_MARK(40 + L);
  if constexpr (NT == 1) {
    conv3_seg<P, L, kSegFull, NTP - 1>(smem, wl, ring, bq, rb, acc, bias, [](int) {});
  } else {
    conv3_seg<P, L, kSegA, NTP - 1>(smem, wl, ring, bq, rb, acc, bias, [](int) {});
    using Plan = EpiPlan<P, Whole, kLoNext, true, kPhaseSteps * (NT - 1) * G::W * 3 - 8>;
    conv3_seg<P, L, kSegB, NTP - 1>(smem, wl, ring, bq, rb, acc, bias, [&](int g) __attribute__((always_inline)) {
      if constexpr (!kLast) {
        Plan::template run<NT>(smem, wb, h4, acc, 0, ROUT, g, carry, k);
      } else {
        last_hidden(g);  // (the last layer's tile 0 feeds the heads from the accumulators)
      }
    });
  }
  C6_MARK(4 + 2 * L);
#ifdef C6_IDLE_PER_LAYER
  // (profiling builds only: idle cycles with no work attached, to see how the card's power
  // management trades them against the shader clock; s_sleep counts in units of 64 cycles)
  __builtin_amdgcn_s_sleep(C6_IDLE_PER_LAYER);
#endif
  (void)wave;
  (void)trace_on;
}

template <class P>
__global__ __launch_bounds__(256) void fused_pipe_kernel(const FwdParams prm) {
  using G = Geo<P>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int THREADS = 256, NWAVES = THREADS / 64;
  constexpr int ROUNDS = (kPix + THREADS - 1) / THREADS;  // pixels per thread when staging

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int h = lane >> 5;
  const int n = lane & 31;

  // Per-lane pixel geometry of the three 32-pixel tiles of this quarter.  Only the activation
  // tile's position index lives through the kernel; what the first layer and the heads need is
  // recomputed per board from an opaque copy of the thread index (a dozen instructions), since
  // values kept from here to there end up in scratch memory.
  auto tile_pixel = [](int t, int j, bool &ok) __attribute__((always_inline)) {
    const int p = (t >> 6) * kPixPerWave + j * 32 + (t & 31);
    ok = p < kPix;
    return ok ? p : (kPix - 1);
  };
  int ci[3];
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    bool ok;
    const int pc = tile_pixel(tid, j, ok);
    const int r = pc / kBoard, c = pc - r * kBoard;
    ci[j] = (r + 1) * kPitch + (c + 1);
  }
  (void)n;

  unsigned char *occ = smem + G::OCC_OFF;
  float *lgt = reinterpret_cast<float *>(smem + G::LGT_OFF);
  float *red = reinterpret_cast<float *>(smem + G::RED_OFF);

  const unsigned per_group = (unsigned)prm.boards_per_group;  // board counts fit 32 bits (host-checked)
  auto packed_of = [&](unsigned b) {
    return prm.packed + (size_t)(b / per_group) * prm.packed_stride;
  };
  // Input of one board, asked for a whole board ahead: loads that write LDS directly, 64
  // consecutive elements per instruction (lane l's element lands in word l behind the
  // instruction's LDS base).  Wave w issues chunks w, w + 4, ...
  typedef const __attribute__((address_space(1))) void *GPtr;
  typedef __attribute__((address_space(3))) void *LPtr;
  auto board_row = [&](unsigned b) {  // board-state input: which row of the state tensors
    long long src = prm.index ? prm.index[b] : b;
    return src < 0 ? 0 : (src >= prm.num_states ? prm.num_states - 1 : src);
  };
  auto issue_fetch = [&](unsigned b) {
    // (lane and wave opaque per call: the chunk addresses are then computed here and not kept,
    // one register pair per chunk, for the whole kernel)
    int ln = lane, wv = wave;
    asm volatile("" : "+v"(ln), "+v"(wv));
    unsigned char *dst = smem + G::NEXT_IN_OFF;
    if (prm.x_dtype == C6_DT_BOARD_I8) {
      // environment state (connect6/vector_env.py:196-218 of the reference), seen through D4
      // view prm.view (connect6/train.py:222-230): the stones, the side to move, stones left
      const long long src = board_row(b);
      const int8_t *board = reinterpret_cast<const int8_t *>(prm.x) + (size_t)src * kPix;
      for (int i = wv; i < (kPix + 63) / 64; i += NWAVES) {
        const int p = i * 64 + ln;
        if (p < kPix)
          __builtin_amdgcn_global_load_lds((GPtr)(board + (prm.view ? d4_from_view(p, prm.view) : p)),
                                           (LPtr)(dst + (G::NEXT_IN_BYTES_AT + i * 64) * 4), 1, 0, 0);
      }
      if (wv == 0 && ln < 2)
        __builtin_amdgcn_global_load_lds((GPtr)((ln == 0 ? prm.player : prm.stones_left) + src),
                                         (LPtr)(dst + G::NEXT_IN_AUX * 4), 1, 0, 0);
      return;
    }
    constexpr int NE = 3 * kPix;
    if (prm.x_dtype == C6_DT_F32) {
      const float *xf = reinterpret_cast<const float *>(prm.x) + (size_t)b * NE;
      for (int i = wv; i < (NE + 63) / 64; i += NWAVES) {
        const int e = i * 64 + ln;
        if (e < NE) __builtin_amdgcn_global_load_lds((GPtr)(xf + e), (LPtr)(dst + i * 256), 4, 0, 0);
      }
    } else {
      const unsigned short *xh = reinterpret_cast<const unsigned short *>(prm.x) + (size_t)b * NE;
      for (int i = wv; i < (NE + 63) / 64; i += NWAVES) {
        const int e = i * 64 + ln;
        if (e < NE) __builtin_amdgcn_global_load_lds((GPtr)(xh + e), (LPtr)(dst + i * 256), 2, 0, 0);
      }
    }
    if (prm.mask_mode == C6_MASK_LEGAL) {
      const uint8_t *lg = prm.legal + (size_t)b * kPix;
      for (int i = wv; i < (kPix + 63) / 64; i += NWAVES) {
        const int p = i * 64 + ln;
        if (p < kPix)
          __builtin_amdgcn_global_load_lds((GPtr)(lg + p), (LPtr)(dst + (G::NEXT_IN_BYTES_AT + i * 64) * 4), 1, 0, 0);
      }
    }
  };
  // what arrived for square p: the three planes and the occupancy flag
  auto staged_input = [&](int p, float (&v)[3], unsigned &o) {
    const unsigned *raw = reinterpret_cast<const unsigned *>(smem + G::NEXT_IN_OFF);
    const unsigned aux = raw[G::NEXT_IN_BYTES_AT + p] & 0xffu;
    if (prm.x_dtype == C6_DT_BOARD_I8) {
      const int stone = (int8_t)aux, me = (int8_t)(raw[G::NEXT_IN_AUX] & 0xffu);
      v[0] = stone == me ? 1.0f : 0.0f;
      v[1] = stone == -me ? 1.0f : 0.0f;
      v[2] = (raw[G::NEXT_IN_AUX + 1] & 0xffu) == 1 ? 1.0f : 0.0f;
    } else {
#pragma unroll
      for (int ch = 0; ch < 3; ++ch) {
        const unsigned w = raw[ch * kPix + p];
        const float as_bf16 = __builtin_bit_cast(float, w << 16);
        const float as_f16 = (float)__builtin_bit_cast(_Float16, (unsigned short)w);
        v[ch] = prm.x_dtype == C6_DT_F32 ? __builtin_bit_cast(float, w)
                                          : (prm.x_dtype == C6_DT_BF16 ? as_bf16 : as_f16);
      }
    }
    // bit 0: the square's logit is masked in the output; bit 1: the square counts as occupied
    // when the margin of the board's decision is judged (cascade), whatever the output mask
    const unsigned taken = prm.mask_mode == C6_MASK_LEGAL ? (aux == 0) : ((v[0] != 0.0f) || (v[1] != 0.0f));
    o = (prm.mask_mode != C6_MASK_NONE ? taken : 0u) | (taken << 1);
  };
  // the third plane's value at square 0, and whether square p holds another one
  auto plane2_differs = [&](int p) {
    const unsigned *raw = reinterpret_cast<const unsigned *>(smem + G::NEXT_IN_OFF);
    // (a 16-bit element arrives in the low half of its word; what the load leaves in the
    // upper half is not part of the value)
    const unsigned keep = prm.x_dtype == C6_DT_F32 ? 0xffffffffu : 0xffffu;
    return prm.x_dtype != C6_DT_BOARD_I8 && ((raw[2 * kPix + p] ^ raw[2 * kPix]) & keep) != 0;
  };
  auto fast1_weights = [&](unsigned b) { return packed_frags<P>(packed_of(b), lane, G::FAST1_OFF); };

  // Each workgroup takes one contiguous run of boards, and the runs are dealt out so that the
  // workgroups of one XCD (workgroup i runs on XCD i % 8) cover one contiguous eighth of the
  // batch: with several weight sets an XCD's L2 then holds only the sets of its own boards, and
  // consecutive boards of a workgroup mostly reuse the set it has just streamed.
  // Cascade, second pass (prm.redo_mode == kRedoConsume): the boards to evaluate are the ones the
  // first pass listed, run by run (run r: redo_counts[r] boards at redo_list[r * redo_per ...]).
  // Every workgroup sums the counts up for itself -- `runs[r]` = boards listed by the runs before
  // r, `runs[redo_runs]` = all of them -- and the listed boards, numbered in that order, are dealt
  // out like the boards of any batch.
  // (compiled into the kernels that can be a cascade's passes only: the first pass is plain bf16,
  // the second one of the modes that carry low parts)
  constexpr bool kCanDetect = P::ID == C6_PREC_BF16, kCanConsume = P::LO6 != 0;
  const bool from_list = kCanConsume && prm.redo_mode == kRedoConsume;
  const bool detect = kCanDetect && prm.redo_mode == kRedoDetect;
  int *runs = reinterpret_cast<int *>(smem + G::RUNS_OFF);
  unsigned n_items = (unsigned)prm.total_boards;
  if (from_list) {
    int *part = reinterpret_cast<int *>(red);   // the four waves' sums
    int before = 0;
    for (int r0 = 0; r0 < prm.redo_runs; r0 += THREADS) {
      const int r = r0 + tid;
      const int c = r < prm.redo_runs ? prm.redo_counts[r] : 0;
      const int incl = wave_inclusive_sum_i(c);
      if (lane == 63) part[wave] = incl;
      __syncthreads();
      int lower = before;
#pragma unroll
      for (int w = 0; w < NWAVES; ++w) {
        lower += w < wave ? part[w] : 0;
        before += part[w];
      }
      if (r < prm.redo_runs) runs[r] = lower + incl - c;
      __syncthreads();
    }
    if (tid == 0) {
      runs[prm.redo_runs] = before;
      if (blockIdx.x == 0) *prm.redo_count = before;   // for the caller: boards evaluated twice
    }
    __syncthreads();
    n_items = (unsigned)before;
  }
  // listed board i: the run r with runs[r] <= i < runs[r + 1] (a bisection; the same in every thread)
  auto board_of = [&](unsigned i) {
    if (!from_list) return i;
    int lo = 0, hi = prm.redo_runs;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if ((unsigned)runs[mid] <= i) lo = mid; else hi = mid;
    }
    return (unsigned)prm.redo_list[(size_t)lo * prm.redo_per + (i - (unsigned)runs[lo])];
  };
  const unsigned per = (n_items + gridDim.x - 1) / gridDim.x;
  const unsigned xcds = (gridDim.x % 8 == 0) ? 8 : 1;
  const unsigned run = (blockIdx.x % xcds) * (gridDim.x / xcds) + blockIdx.x / xcds;
  // (board counts fit 31 bits, host-checked; a run beyond the last board starts past n_items)
  const unsigned long long first_item = (unsigned long long)run * per;
  if (first_item >= n_items) {
    if (detect && tid == 0) prm.redo_counts[run] = 0;   // (a run without boards lists none)
    return;
  }
  unsigned it = (unsigned)first_item;  // position in the run of boards; `b` below is the board itself
  const unsigned it_end = n_items - it > per ? it + per : n_items;
  int listed = 0;                      // cascade, first pass: boards of this run listed so far (wave 1 counts)
  [[maybe_unused]] const unsigned it_first = it;
  v4i r1[L1Pipe<P>::D][1];
  // (the first layer's weight ring is filled, a board ahead, with the stream for a constant
  // third plane; a board that has none refills it)
  unsigned b = board_of(it);
  preload_ring<L1Pipe<P>::D, 1>(r1, fast1_weights(b));
  issue_fetch(b);
  if (tid == 0) reinterpret_cast<int *>(red)[8] = 0;  // (the first board's flag, see the staging)
  const unsigned char *packed_before = nullptr;

  for (; it < it_end; ++it) {
    int tidv = tid;  // opaque per board: keeps per-thread staging addresses out of long-lived registers
    asm volatile("" : "+v"(tidv));
    const unsigned char *packed = packed_of(b);
    const float *tail = reinterpret_cast<const float *>(packed + G::TAIL_OFF);
    // the weight set's fp32 tail goes to LDS whenever the set changes (see the staging)
    constexpr int TAILN = kBiasTotal + 2 * kHeadC + 4;
    const bool new_set = packed != packed_before;
    packed_before = packed;
    const int tail_lds = G::TAIL_LDS_OFF;
    // block-scale exponents of the low-order weight copies (E8M0: 127 - log2 of the copy's scale),
    // fetched here, long before any second pass needs them
    int lo_scale_w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (P::LO6) {
#pragma unroll
      for (int l = 1; l < 8; ++l) lo_scale_w[l] = 127 - reinterpret_cast<const int *>(tail)[G::TAIL_SW + l];
    }

#if defined(C6_TRACE)
    const bool trace_on = (it == it_first + 2);  // third board of this workgroup
#else
    const bool trace_on = false;
#endif
    __builtin_amdgcn_s_waitcnt(0);  // this wave's share of the board's input has landed in LDS
    __syncthreads();  // ... and everybody's; previous board fully written out; LDS is free
    C6_MARK(0);
    const bool has_next = it + 1 < it_end;
    const unsigned bn = has_next ? board_of(it + 1) : b;
    // The third plane's share of the first layer, should the plane turn out constant: the
    // per-square sums of its weights (register i of pixel tile j = channel 8 (i / 4) + 4 h + i % 4),
    // asked for now so that the loads are long back when the K-loop starts; there they are
    // multiplied by the plane's value and joined by the bias.
    f32x16 a0[1][3];
    {
      // (the wave number through a scalar register: the loads take the fragment offset from one)
      const WFrags tb = packed_frags<P>(packed, lane, G::PLANE2_FRAG_OFF + __builtin_amdgcn_readfirstlane(wave) * 12);
#pragma unroll
      for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4 t4 = __builtin_bit_cast(f32x4, tb[j * 4 + q]);
#pragma unroll
          for (int e = 0; e < 4; ++e) a0[0][j][4 * q + e] = t4[e];
        }
      __builtin_amdgcn_sched_barrier(0);  // (issue here)
    }
    // ---- stage the input: zero the shifted copies, then scatter the board ----
    // Does the third plane vary?  Any thread that sees it differ from square 0 raises this board's
    // flag (two flags, used in turn: the other one is cleared for the next board meanwhile).
    int *plane2_flag = reinterpret_cast<int *>(red) + 8 + (int)((it - it_first) & 1);
    {
      bool varies = false;
#pragma unroll
      for (int r = 0; r < ROUNDS; ++r)
        if (tidv + r * THREADS < kPix) varies |= plane2_differs(tidv + r * THREADS);
      if (varies) *plane2_flag = 1;
      if (tid == 0) reinterpret_cast<int *>(red)[8 + (int)((it - it_first + 1) & 1)] = 0;
    }
    {
      // (unrolled, one address register and immediate offsets: as a loop the same stores take
      // twice as long, 2.0 k cycles against 1.1 k measured alone -- LDS stores are bound by the
      // wave's own instruction issue here)
      const v4i z = {0, 0, 0, 0};
      constexpr int WHOLE = G::COPIES_BYTES / 16 / THREADS;
      unsigned char *zp = smem + tidv * 16;
#pragma unroll
      for (int u = 0; u < WHOLE; ++u) *reinterpret_cast<v4i *>(zp + u * (THREADS * 16)) = z;
      if (tidv * 16 + WHOLE * (THREADS * 16) < G::COPIES_BYTES)
        *reinterpret_cast<v4i *>(zp + WHOLE * (THREADS * 16)) = z;
    }
    __syncthreads();
    const bool plane2_varies = *plane2_flag != 0;
    const int planes_staged = plane2_varies ? 3 : 2;  // (a constant third plane is not contracted)
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int p = tidv + r * THREADS;
      if (p < kPix) {
        const int row = p / kBoard, c = p - row * kBoard;
        float v[3];
        unsigned o;
        staged_input(p, v, o);
        occ[p] = (unsigned char)o;
#pragma unroll
        for (int ch = 0; ch < 3; ++ch) {
          if (ch >= planes_staged) break;
          const int hrow = (row + kK1 / 2) * 3 + ch;
          const unsigned short v16 = bits16<P>(v[ch]);
#pragma unroll
          for (int s = 0; s < G::E; ++s) {
            const int a = s * G::COPY_BYTES + (hrow * kL1RowPitch + (c + kK1 / 2 - s)) * G::EB;
            *reinterpret_cast<unsigned short *>(smem + a) = v16;
          }
        }
      }
    }
    if (new_set) {
      // straight into LDS, 64 floats per instruction (lane l's float lands in word l behind the
      // instruction's base); the barrier below waits for loads that write LDS
      for (int i = tidv >> 6; i < (TAILN + 63) / 64; i += NWAVES) {
        const int e = i * 64 + (tidv & 63);
        if (e < TAILN)
          __builtin_amdgcn_global_load_lds((GPtr)(tail + e), (LPtr)(smem + G::TAIL_LDS_OFF + i * 256), 4, 0, 0);
      }
      __builtin_amdgcn_s_waitcnt(0);  // landed before this wave reaches the barrier
    }
    __syncthreads();
    C6_MARK(1);

    v4i r2[kRing], r3[kRing * 2], r6[kRing * 3];  // weight rings of layers 2, 3-5, 6-8
    f32x16 a1[1][3];
    // ---- layer 1 ----
    {
      int l1base[3];
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        bool ok;
        const int pc = tile_pixel(tidv, j, ok);
        const int r = pc / kBoard, c = pc - r * kBoard, s = c % G::E;
        l1base[j] = s * G::COPY_BYTES + ((r * 3 + kL1RowsHalf * ((tidv >> 5) & 1)) * kL1RowPitch + (c - s)) * G::EB;
      }
      f32x16 b0[1];
      load_bias_tiles_lds(b0, smem, tail_lds, bias_offset(0), h);
      if (!plane2_varies) {
        float v2[3];
        unsigned o2;
        staged_input(0, v2, o2);
        const float c2 = v2[2];
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
          for (int i = 0; i < 16; ++i) a0[0][j][i] = fmaf(c2, a0[0][j][i], b0[0][i]);
        int l1fast[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) l1fast[j] = l1base[j] - (kL1RowsHalf - 1) * h * kL1RowPitch * G::EB;
        conv1_fast_pass<P>(smem, fast1_weights(b), r1, l1fast, a0);
      } else {
#pragma unroll
        for (int j = 0; j < 3; ++j) a0[0][j] = b0[0];
        preload_ring<L1Pipe<P>::D, 1>(r1, layer_weights<P, 0>(packed, lane));
        conv1_pass<P>(smem, layer_weights<P, 0>(packed, lane), r1, l1base, a0);
      }
    }
    preload_flat<kRing>(r2, layer_weights<P, 1>(packed, lane));
    C6_MARK(2);
    pipe_layer<P, 1>(smem, packed, tail_lds, r2, ci, h, lane, wave, trace_on, lo_scale_w, a0, a1, [&] {
      // the first layer's shifted copies overlapped the activation tile: restore its zero padding
      for (int i = tidv; i < 60 * (G::PIXB / 16); i += THREADS) {
        const int k = i / (G::PIXB / 16), w16 = i - k * (G::PIXB / 16);
        // pad positions: 0..19 (top row), 400..420 (bottom row + tail), 20*R (left column)
        const int pos = k < 20 ? k : (k < 41 ? 400 + (k - 20) : (k - 40) * kPitch);
        const v4i z = {0, 0, 0, 0};
        *reinterpret_cast<v4i *>(smem + pos * G::PIXB + w16 * 16) = z;
      }
    }, [](int) {});
    preload_flat<kRing * 2>(r3, layer_weights<P, 2>(packed, lane));
    f32x16 a2[2][3];
    pipe_layer<P, 2>(smem, packed, tail_lds, r3, ci, h, lane, wave, trace_on, lo_scale_w, a1, a2, [] {}, [](int) {});
    f32x16 a3[2][3];
    pipe_layer<P, 3>(smem, packed, tail_lds, r3, ci, h, lane, wave, trace_on, lo_scale_w, a2, a3, [] {}, [](int) {});
    f32x16 a4[2][3];
    pipe_layer<P, 4>(smem, packed, tail_lds, r3, ci, h, lane, wave, trace_on, lo_scale_w, a3, a4, [] {}, [](int) {});
    preload_flat<kRing * 3>(r6, layer_weights<P, 5>(packed, lane));
    f32x16 a5[3][3];
    pipe_layer<P, 5>(smem, packed, tail_lds, r6, ci, h, lane, wave, trace_on, lo_scale_w, a4, a5, [] {}, [](int) {});
    f32x16 a6[3][3];
    pipe_layer<P, 6>(smem, packed, tail_lds, r6, ci, h, lane, wave, trace_on, lo_scale_w, a5, a6, [] {}, [](int) {});
    f32x16 acc[3][3];
    // The heads' share of channel tile 0 rides behind the MFMAs of the last layer's other two
    // tiles (tile 0 is final before them): element e = (quad, pixel tile, channel of the quad)
    // takes exp2 in slot 2e, 1 + . in slot 2e+1, rcp in slot 2e+2 and x * . with the two
    // multiply-adds in slot 2e+3 -- three instructions per slot in the mean.
    float pol[3] = {0.0f, 0.0f, 0.0f}, val0[3] = {0.0f, 0.0f, 0.0f};
    f32x4 hpw[4], hvw[4];
    float hden[2];
    auto head_slot = [&](int g) __attribute__((always_inline)) {
      constexpr int NE = 48;
      if (g == 0) {
        int hb0 = tail_lds + 4 * kBiasTotal + 16 * h;
        asm volatile("" : "+v"(hb0));
        const float *w0 = reinterpret_cast<const float *>(smem + hb0);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          hpw[q] = *reinterpret_cast<const f32x4 *>(w0 + 8 * q);
          hvw[q] = *reinterpret_cast<const f32x4 *>(w0 + kHeadC + 8 * q);
        }
      }
      auto reg_of = [](int e) __attribute__((always_inline)) { return 4 * (e / 12) + e % 4; };
      auto tile_of = [](int e) __attribute__((always_inline)) { return (e / 4) % 3; };
      // (each result through an empty asm statement: pure arithmetic whose only use comes behind
      // the K-loop would otherwise be moved there)
      if (g % 2 == 0) {
        const int e = g / 2;
        if (e < NE) {
          hden[e % 2] = __builtin_amdgcn_exp2f(acc[0][tile_of(e)][reg_of(e)]);
          asm volatile("" : "+v"(hden[e % 2]));
        }
        if (e - 1 >= 0 && e - 1 < NE) {
          hden[(e - 1) % 2] = __builtin_amdgcn_rcpf(hden[(e - 1) % 2]);
          asm volatile("" : "+v"(hden[(e - 1) % 2]));
        }
      } else {
        const int e = g / 2;
        if (e < NE) {
          hden[e % 2] = 1.0f + hden[e % 2];
          asm volatile("" : "+v"(hden[e % 2]));
        }
        if (e - 1 >= 0 && e - 1 < NE) {
          const int d = e - 1, j = tile_of(d);
          const float a = acc[0][j][reg_of(d)] * hden[d % 2];
          pol[j] = fmaf(a, hpw[d / 12][d % 4], pol[j]);
          val0[j] = fmaf(a, hvw[d / 12][d % 4], val0[j]);
          asm volatile("" : "+v"(pol[j]), "+v"(val0[j]));
        }
      }
    };
    pipe_layer<P, 7>(smem, packed, tail_lds, r6, ci, h, lane, wave, trace_on, lo_scale_w, a6, acc, [] {},
                     [&](int g) __attribute__((always_inline)) { head_slot(g); });

    // ---- both 1x1 heads straight from the fp32 accumulators of layer 8 ----
    {
      // head weights from the tail's copy in LDS: channel 32t + 8q + 4h + e
      int hb = tail_lds + 4 * kBiasTotal + 16 * h;
      asm volatile("" : "+v"(hb));  // (one address register for all head weights)
      const float *pwg = reinterpret_cast<const float *>(smem + hb);
      const float *tl = pwg - 4 * h - kBiasTotal;
      int pix[3];
      bool valid[3];
      int th = tidv;
      asm volatile("" : "+v"(th));  // (computed here, not at the top of the board and kept)
#pragma unroll
      for (int j = 0; j < 3; ++j) pix[j] = tile_pixel(th, j, valid[j]);
      if (has_next) preload_ring<L1Pipe<P>::D, 1>(r1, fast1_weights(bn));
      float vsum = 0.0f;
#pragma unroll
      for (int j = 0; j < 3; ++j) vsum += valid[j] ? val0[j] : 0.0f;  // (tile 0: done behind the last layer)
#pragma unroll
      for (int t = 1; t < 3; ++t)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4 pw = *reinterpret_cast<const f32x4 *>(pwg + 32 * t + 8 * q);
          const f32x4 vw = *reinterpret_cast<const f32x4 *>(pwg + kHeadC + 32 * t + 8 * q);
#pragma unroll
          for (int j = 0; j < 3; ++j) {
            float vs = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float a = silu<P>(acc[t][j][4 * q + e]);
              pol[j] = fmaf(a, pw[e], pol[j]);
              vs = fmaf(a, vw[e], vs);
            }
            vsum += valid[j] ? vs : 0.0f;
          }
        }
      const float polb = tl[kBiasTotal + 2 * kHeadC], valb = tl[kBiasTotal + 2 * kHeadC + 1];
      float tot[3];
#pragma unroll
      for (int j = 0; j < 3; ++j) {  // add the other lane half's channels
        const unsigned bits = __builtin_bit_cast(unsigned, pol[j]);
        const auto r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
        const unsigned r0 = r[0], r1 = r[1];
        tot[j] = __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
      }
#pragma unroll
      for (int j = 0; j < 3; ++j)
        if (h == 0 && valid[j]) lgt[pix[j]] = tot[j] + polb;
      vsum = wave_sum(vsum);
      if (lane == 0) red[wave] = vsum;
      __syncthreads();
      // The next board's input is asked for here, behind the board's last barrier but one (a
      // barrier waits for loads that write LDS) and with no K-loop ahead: the counter of loads in
      // flight is served in order, so in front of a K-loop these loads from HBM would hold up
      // its weight fragments.
      if (has_next) issue_fetch(bn);
      if (tid == 0 && prm.value != nullptr) {
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) s += red[w];
        prm.value[b] = tanhf(s * (1.0f / kPix) + valb);
      }
      C6_MARK(19);
    }

    // ---- write out: masked logits, optional sampled action ----
    if (prm.logits != nullptr) {
      for (int p = tidv; p < kPix; p += THREADS) {
        const float v = (occ[p] & 1) ? prm.fill : lgt[p];
        const size_t at = (size_t)b * kPix + p;
        if (prm.logits_dtype == C6_DT_F32) {
          static_cast<float *>(prm.logits)[at] = v;
        } else if (prm.logits_dtype == C6_DT_BF16) {  // (round to nearest even, as Tensor.to does)
          static_cast<unsigned short *>(prm.logits)[at] = __builtin_bit_cast(unsigned short, (__bf16)v);
        } else {
          static_cast<unsigned short *>(prm.logits)[at] = __builtin_bit_cast(unsigned short, (_Float16)v);
        }
      }
    }
    if (prm.actions != nullptr && wave == 0) {
      float inv_t = prm.inv_temperature;
      asm volatile("" : "+s"(inv_t));  // (what is derived from it is derived here, not kept)
      int a;
      float lp;
      int lane_here = lane;  // opaque per board: the entries' LDS addresses are computed here,
      asm volatile("" : "+v"(lane_here));  // not once per kernel into registers that get spilled
      wave_sample(
          lane_here, prm.u[b], inv_t, [&](int i) { return lgt[i]; }, [&](int i) { return (occ[i] & 1) == 0; },
          a, lp);
      if (lane == 0) {
        prm.actions[b] = a;
        if (prm.logprob != nullptr) prm.logprob[b] = lp;
      }
    }
    if (detect && wave == 1) {
      // Cascade, first pass: a board whose best free square leads the second best by less than
      // the threshold (in standard deviations of its free squares' logits) is put on the list
      // of boards that the second pass evaluates again with the corrected arithmetic.
      float tau = prm.redo_threshold;
      asm volatile("" : "+s"(tau));
      int lane_here = lane;
      asm volatile("" : "+v"(lane_here));
      const bool again = wave_margin_below(
          lane_here, tau, [&](int i) { return lgt[i]; }, [&](int i) { return (occ[i] & 2) == 0; });
      if (again) {   // (wave-uniform)
        if (lane == 0) prm.redo_list[(size_t)run * prm.redo_per + listed] = (int)b;
        ++listed;
      }
    }
    C6_MARK(20);
    b = bn;
  }
  if (detect && wave == 1 && lane == 0) prm.redo_counts[run] = listed;
}

// ------------------------------------------------------------------------
// the fused kernel: a persistent loop over boards; one wave per SIMD, each wave owning all
// output channels of its 96 pixels
// ------------------------------------------------------------------------
template <class P>
__global__ __launch_bounds__(256) void fused_forward_kernel(const FwdParams prm) {
  using G = Geo<P>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int THREADS = 256, NWAVES = THREADS / 64;
  constexpr int ROUNDS = (kPix + THREADS - 1) / THREADS;  // pixels per thread when staging

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int h = lane >> 5;
  const int n = lane & 31;

  // per-lane pixel geometry of the three 32-pixel tiles of this quarter
  int ci[3], l1base[3], pix[3];
  bool valid[3];
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    const int p = wave * kPixPerWave + j * 32 + n;
    valid[j] = p < kPix;
    const int pc = valid[j] ? p : (kPix - 1);
    pix[j] = pc;
    const int r = pc / kBoard, c = pc - r * kBoard;
    ci[j] = (r + 1) * kPitch + (c + 1);
    const int s = c % G::E;
    l1base[j] = s * G::COPY_BYTES + ((r * 3 + kL1RowsHalf * h) * kL1RowPitch + (c - s)) * G::EB;
  }

  unsigned char *occ = smem + G::OCC_OFF;
  float *lgt = reinterpret_cast<float *>(smem + G::LGT_OFF);
  float *red = reinterpret_cast<float *>(smem + G::RED_OFF);

  const unsigned per_group = (unsigned)prm.boards_per_group;  // board counts fit 32 bits (host-checked)
  auto packed_of = [&](long long b) {
    return prm.packed + (size_t)((unsigned)b / per_group) * prm.packed_stride;
  };
  // input of one board: each thread owns pixels tid, tid + THREADS, ... (three planes + occupancy)
  float xin[ROUNDS][3];
  unsigned char occin[ROUNDS];
  auto fetch_board = [&](long long b) {
    int tid = threadIdx.x;  // (opaque per call: the per-square addresses are formed here, not kept)
    asm volatile("" : "+v"(tid));
    if (prm.x_dtype == C6_DT_BOARD_I8) {
      // environment state in, network planes out (connect6/vector_env.py:196-218 of the
      // reference), seen through D4 view prm.view (connect6/train.py:222-230)
      long long src = prm.index ? prm.index[b] : b;
      src = src < 0 ? 0 : (src >= prm.num_states ? prm.num_states - 1 : src);
      const int8_t *board = reinterpret_cast<const int8_t *>(prm.x) + (size_t)src * kPix;
      const int me = prm.player[src];
      const float last = prm.stones_left[src] == 1 ? 1.0f : 0.0f;
#pragma unroll
      for (int r = 0; r < ROUNDS; ++r) {
        const int p = tid + r * THREADS;
        if (p < kPix) {
          const int stone = board[prm.view ? d4_from_view(p, prm.view) : p];
          xin[r][0] = stone == me ? 1.0f : 0.0f;
          xin[r][1] = stone == -me ? 1.0f : 0.0f;
          xin[r][2] = last;
          occin[r] = 0;
        }
      }
      return;
    }
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int p = tid + r * THREADS;
      if (p < kPix) {
#pragma unroll
        for (int ch = 0; ch < 3; ++ch)
          xin[r][ch] = load_x(prm.x, prm.x_dtype, ((size_t)b * 3 + ch) * kPix + p);
        occin[r] = prm.mask_mode == C6_MASK_LEGAL ? (prm.legal[(size_t)b * kPix + p] == 0) : 0;
      }
    }
  };

  // Each workgroup takes one contiguous run of boards, and the runs are dealt out so that the
  // workgroups of one XCD (workgroup i runs on XCD i % 8) cover one contiguous eighth of the
  // batch: with several weight sets an XCD's L2 then holds only the sets of its own boards, and
  // consecutive boards of a workgroup mostly reuse the set it has just streamed.
  const long long per = (prm.total_boards + gridDim.x - 1) / gridDim.x;
  const unsigned xcds = (gridDim.x % 8 == 0) ? 8 : 1;
  const long long run = (long long)(blockIdx.x % xcds) * (gridDim.x / xcds) + blockIdx.x / xcds;
  long long b = run * per;
  const long long b_end = b + per < prm.total_boards ? b + per : prm.total_boards;
  if (b >= b_end) return;
  [[maybe_unused]] const long long b_first = b;
  v4i r1[L1Pipe<P>::D][1];
  preload_ring<L1Pipe<P>::D, 1>(r1, layer_weights<P, 0>(packed_of(b), lane));
  fetch_board(b);

  for (; b < b_end; ++b) {
    int tidv = tid;  // opaque per board: keeps per-thread staging addresses out of long-lived registers
    asm volatile("" : "+v"(tidv));
    const unsigned char *packed = packed_of(b);
    const float *tail = reinterpret_cast<const float *>(packed + G::TAIL_OFF);
#ifdef C6_TRACE
    const bool trace_on = (b == b_first + 2);  // third board of this workgroup
#else
    const bool trace_on = false;
#endif
    __syncthreads();  // previous board fully written out; LDS is free
    C6_MARK(0);
    // ---- stage the input: zero the shifted copies, then scatter the board ----
    {
      const v4i z = {0, 0, 0, 0};
      for (int i = tidv * 16; i < G::COPIES_BYTES; i += THREADS * 16)
        *reinterpret_cast<v4i *>(smem + i) = z;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int p = tidv + r * THREADS;
      if (p < kPix) {
        const int row = p / kBoard, c = p - row * kBoard;
        unsigned char o = occin[r];
        if (prm.mask_mode == C6_MASK_INPUT) o = (xin[r][0] != 0.0f) || (xin[r][1] != 0.0f);
        occ[p] = o;
#pragma unroll
        for (int ch = 0; ch < 3; ++ch) {
          const int hrow = (row + kK1 / 2) * 3 + ch;
#pragma unroll
          for (int s = 0; s < G::E; ++s) {
            const int a = s * G::COPY_BYTES + (hrow * kL1RowPitch + (c + kK1 / 2 - s)) * G::EB;
            if constexpr (G::EB == 4) {
              *reinterpret_cast<float *>(smem + a) = xin[r][ch];
            } else {
              *reinterpret_cast<unsigned short *>(smem + a) = bits16<P>(xin[r][ch]);
            }
          }
        }
      }
    }
    const long long bn = b + 1;
    if (bn < b_end) fetch_board(bn);  // lands while this board is computed
    __syncthreads();
    C6_MARK(1);

    v4i r2[kRing][1], r345[kRing][2], r678[kRing][3];  // weight rings of layers 2, 3-5, 6-8
    // ---- layer 1 ----
    {
      f32x16 acc[1][3];
      init_acc(acc, tail + bias_offset(0), h);
      conv1_pass<P>(smem, layer_weights<P, 0>(packed, lane), r1, l1base, acc);
      preload_ring<kRing, 1>(r2, layer_weights<P, 1>(packed, lane));
      C6_MARK(2);
      finish_layer<P, 1>(smem, ci, h, acc, [&] {
        // the copies overlapped the activation tile: restore its zero padding
        for (int i = tidv; i < 60 * (G::PIXB / 16); i += THREADS) {
          const int k = i / (G::PIXB / 16), w16 = i - k * (G::PIXB / 16);
          // pad positions: 0..19 (top row), 400..420 (bottom row + tail), 20*R (left column)
          const int pos = k < 20 ? k : (k < 41 ? 400 + (k - 20) : (k - 40) * kPitch);
          const v4i z = {0, 0, 0, 0};
          *reinterpret_cast<v4i *>(smem + pos * G::PIXB + w16 * 16) = z;
        }
      });
    }
    C6_MARK(3);
    mid_layer<P, 1>(smem, packed, tail, r2, r345, ci, h, lane, wave, trace_on);
    mid_layer<P, 2>(smem, packed, tail, r345, r345, ci, h, lane, wave, trace_on);
    mid_layer<P, 3>(smem, packed, tail, r345, r345, ci, h, lane, wave, trace_on);
    mid_layer<P, 4>(smem, packed, tail, r345, r678, ci, h, lane, wave, trace_on);
    mid_layer<P, 5>(smem, packed, tail, r678, r678, ci, h, lane, wave, trace_on);
    mid_layer<P, 6>(smem, packed, tail, r678, r678, ci, h, lane, wave, trace_on);

    // ---- layer 8 + both 1x1 heads straight from the fp32 accumulators ----
    {
      f32x16 acc[3][3];
      init_acc(acc, tail + bias_offset(7), h);
      const float *polw = tail + kBiasTotal;
      const float *valw = polw + kHeadC;
      const float *pwl = polw + 4 * h;  // per-lane base: channel 32t + 8q + 4h + e
      asm volatile("" : "+v"(pwl));
      const GlobalF32 pwg = (GlobalF32)pwl;
      conv3_pass<P, 96, 96>(smem, layer_weights<P, 7>(packed, lane), r678, ci, h, acc);
      C6_MARK(37);
      if (bn < b_end) preload_ring<L1Pipe<P>::D, 1>(r1, layer_weights<P, 0>(packed_of(bn), lane));
      C6_MARK(18);
      float pol[3] = {0.0f, 0.0f, 0.0f};
      float vsum = 0.0f;
#pragma unroll
      for (int t = 0; t < 3; ++t)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4 pw = *(GlobalF32x4)(pwg + 32 * t + 8 * q);
          const f32x4 vw = *(GlobalF32x4)(pwg + kHeadC + 32 * t + 8 * q);
#pragma unroll
          for (int j = 0; j < 3; ++j) {
            float vs = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float a = silu<P>(acc[t][j][4 * q + e]);
              pol[j] = fmaf(a, pw[e], pol[j]);
              vs = fmaf(a, vw[e], vs);
            }
            vsum += valid[j] ? vs : 0.0f;
          }
        }
      const float polb = valw[kHeadC], valb = valw[kHeadC + 1];
      float tot[3];
#pragma unroll
      for (int j = 0; j < 3; ++j) {  // add the other lane half's channels
        const unsigned bits = __builtin_bit_cast(unsigned, pol[j]);
        const auto r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
        const unsigned r0 = r[0], r1 = r[1];
        tot[j] = __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
      }
#pragma unroll
      for (int j = 0; j < 3; ++j)
        if (h == 0 && valid[j]) lgt[pix[j]] = tot[j] + polb;
      vsum = wave_sum(vsum);
      if (lane == 0) red[wave] = vsum;
      __syncthreads();
      if (tid == 0 && prm.value != nullptr) {
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) s += red[w];
        prm.value[b] = tanhf(s * (1.0f / kPix) + valb);
      }
      C6_MARK(19);
    }

    // ---- write out: masked logits, optional sampled action ----
    if (prm.logits != nullptr) {
      for (int p = tid; p < kPix; p += THREADS) {
        const float v = lgt[p];
        static_cast<float *>(prm.logits)[(size_t)b * kPix + p] = occ[p] ? prm.fill : v;
      }
    }
    if (prm.actions != nullptr && wave == 0) {
      float it = prm.inv_temperature;
      asm volatile("" : "+s"(it));  // (what is derived from it is derived here, not kept)
      int a;
      float lp;
      int lane_here = lane;  // opaque per board: the entries' LDS addresses are computed here,
      asm volatile("" : "+v"(lane_here));  // not once per kernel into registers that get spilled
      wave_sample(
          lane_here, prm.u[b], it, [&](int i) { return lgt[i]; }, [&](int i) { return occ[i] == 0; },
          a, lp);
      if (lane == 0) {
        prm.actions[b] = a;
        if (prm.logprob != nullptr) prm.logprob[b] = lp;
      }
    }
    C6_MARK(20);
  }
}

#ifdef C6_TRACE
extern "C" int c6_debug_trace(long long *host_out) {
  return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(g_trace), sizeof(long long) * 256 * 4 * 64);
}
#endif

// ------------------------------------------------------------------------
// weight repack: PyTorch OIHW fp32 -> MFMA fragment order
// ------------------------------------------------------------------------
template <class P> __device__ __forceinline__ void put_elem(unsigned char *dst, int e, float v) {
  if constexpr (P::EB == 4) {
    reinterpret_cast<float *>(dst)[e] = v;
  } else {
    reinterpret_cast<unsigned short *>(dst)[e] = bits16<P>(v);
  }
}

// part 0: the weight itself (put_elem rounds it to the storage type); part 1 (WLO): what that
// rounding drops, which put_elem rounds in turn
template <class P> __device__ __forceinline__ float weight_part(float v, int part) {
  if constexpr (P::EB == 4) {
    return v;
  } else {
    const float hi = __builtin_bit_cast(float, (unsigned)bits16<P>(v) << 16);
    static_assert(P::WLO == 0 || P::ID != C6_PREC_F16, "the low part is defined for bf16 storage");
    return part ? v - hi : v;
  }
}

// The parameters of weight set `g` of a (possibly stacked) PackParams.
struct GroupView {
  const PackParams &p;
  int g;
  unsigned char *packed;
  const float *pol_w, *pol_b, *val_w, *val_b;
  __device__ GroupView(const PackParams &pp, int group)
      : p(pp), g(group), packed(pp.packed + (size_t)group * pp.packed_stride),
        pol_w(pp.pol_w + (size_t)group * kHeadC), pol_b(pp.pol_b ? pp.pol_b + group : nullptr),
        val_w(pp.val_w ? pp.val_w + (size_t)group * kHeadC : nullptr),
        val_b(pp.val_b ? pp.val_b + group : nullptr) {}
  __device__ const float *conv_w(int l) const {
    const int k = l == 0 ? kK1 : 3;
    return p.conv_w[l] + (size_t)g * kCoutArr[l] * kCinArr[l] * k * k;
  }
  __device__ const float *conv_b(int l) const {
    return p.conv_b[l] ? p.conv_b[l] + (size_t)g * kCoutArr[l] : nullptr;
  }
};

// one thread per (fragment, lane): writes the 16 bytes that lane will load
// (blockIdx.y = weight set: the parameter tensors are stacked [sets, ...], the packed sets lie
// packed_stride bytes apart)
template <class P> __global__ void pack_kernel(const PackParams all) {
  using G = Geo<P>;
  const GroupView prm(all, blockIdx.y);
  const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long nfl = (long long)G::TOTAL_FRAGS * 64;
  if (gid < nfl) {
    const int frag = (int)(gid >> 6), lane = (int)(gid & 63);
    const int m = lane & 31, h = lane >> 5;
    unsigned char *dst = prm.packed + (size_t)gid * 16;
    int l = 0;
    while (l < 8 && frag >= G::frag_offset(l + 1)) ++l;  // frag_offset is monotone
    if (l >= 8) {  // over-read padding, the low-order weight copies behind it, the second first-layer copy
      v4i o = {0, 0, 0, 0};
      if (G::FAST1_FRAGS > 0 && frag >= G::PLANE2_FRAG_OFF && frag < G::PLANE2_FRAG_OFF + G::PLANE2_FRAGS) {
        // the third plane's weights that fall inside the board, summed, as seen from the lane's
        // output square: four channels per lane and fragment
        const int fi = frag - G::PLANE2_FRAG_OFF, wv = fi / 12, j = (fi / 4) % 3, q = fi % 4;
        int p = wv * kPixPerWave + j * 32 + m;
        p = p < kPix ? p : kPix - 1;
        const int r = p / kBoard, c = p % kBoard;
        f32x4 t4;
        for (int e = 0; e < 4; ++e) {
          const float *w = prm.conv_w(0) + (size_t)((8 * q + 4 * h + e) * 3 + 2) * kK1 * kK1;
          float sum = 0.0f;
          for (int ky = 0; ky < kK1; ++ky) {
            const int rr = r + ky - kK1 / 2;
            if (rr < 0 || rr >= kBoard) continue;
            for (int kx = 0; kx < kK1; ++kx) {
              const int cc = c + kx - kK1 / 2;
              if (cc >= 0 && cc < kBoard) sum += w[ky * kK1 + kx];
            }
          }
          t4[e] = sum * act_scale<P>();
        }
        *reinterpret_cast<f32x4 *>(dst) = t4;
        return;
      }
      if (G::FAST1_FRAGS > 0 && frag >= G::FAST1_OFF && frag < G::FAST1_OFF + G::FAST1_STREAM) {
        // k-step (ky, 8 columns); lane half = input plane
        const int part = (frag - G::FAST1_OFF) % G::W;
        const int fi = (frag - G::FAST1_OFF) / G::W, ky = fi / G::CPR, jj = fi % G::CPR;
        const float *w = prm.conv_w(0);
        for (int e = 0; e < G::E; ++e) {
          const int kx = jj * G::E + e;
          put_elem<P>(dst, e, weight_part<P>(kx < kK1 ? w[((m * 3 + h) * kK1 + ky) * kK1 + kx] * act_scale<P>() : 0.0f, part));
        }
        return;
      }
      if constexpr (P::LO6) {
        int ll = 1;
        while (ll < 8 && frag >= G::lo_frag_offset(ll + 1)) ++ll;
        if (frag >= G::HI_FRAGS && ll < 8) {
          const int fi = frag - G::lo_frag_offset(ll);
          const int cin = kCinArr[ll], nt = kCoutArr[ll] / 32, per32 = cin / 32;
          const int c = fi / (nt * 2), t = (fi / 2) % nt, piece = fi & 1;
          const int g = 2 * c + h;
          if (g < G::lo_half_chunks(ll)) {
            const int tap = g / per32, cb = g % per32, co = 32 * t + m;
            const float *w = prm.conv_w(ll);
            const float sc = exp2f((float)reinterpret_cast<const int *>(prm.packed + G::TAIL_OFF)[G::TAIL_SW + ll]);
            // the lane's 32 K slots as e2m3 (the copy approximates the bf16 weights the main pass
            // uses): 24 bytes = piece 0 + piece 1
            f32x16v even, odd;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              even[i] = (float)(__bf16)w[(co * cin + lo6_channel(cb, 2 * i)) * 9 + tap] * sc;
              odd[i] = (float)(__bf16)w[(co * cin + lo6_channel(cb, 2 * i + 1)) * 9 + tap] * sc;
            }
            const u32x6 r = to_fp6_block(even, odd, 1.0f);
            if (piece == 0) {
              o = v4i{(int)r[0], (int)r[1], (int)r[2], (int)r[3]};
            } else {
              o = v4i{(int)r[4], (int)r[5], 0, 0};
            }
          }
        }
      }
      if constexpr (P::LO6) {
        // Second piece of an fp6 fragment: 8 bytes per lane, the lanes' parts packed densely into
        // the fragment's first 512 bytes (WFrags::dense8); the rest of the fragment is zero.
        if (frag >= G::HI_FRAGS && frag < G::lo_frag_offset(8) && ((frag - G::HI_FRAGS) & 1)) {
          unsigned char *fb = prm.packed + (size_t)frag * 1024;
          *reinterpret_cast<v2i *>(fb + lane * 8) = v2i{o[0], o[1]};
          *reinterpret_cast<v2i *>(fb + 512 + lane * 8) = v2i{0, 0};
          return;
        }
      }
      *reinterpret_cast<v4i *>(dst) = o;
      return;
    }
    // (WLO: fragment 2i holds the weights of fragment i of the plain order, fragment 2i + 1 what
    // their rounding dropped)
    const int part = (frag - G::frag_offset(l)) % G::W;
    const int fi = (frag - G::frag_offset(l)) / G::W;
    const int cin = kCinArr[l], cout = kCoutArr[l];
    const int nt = cout / 32;
    const int s = fi / nt, t = fi - s * nt;
    const int co = 32 * t + m;
    const float *w = prm.conv_w(l);
    if (l == 0) {
      const int row = s / G::CPR + kL1RowsHalf * h;  // (ky, plane) row, 69 real + 1 pad
      const int jj = s % G::CPR;
      const int ky = row / 3, ch = row - ky * 3;
      for (int e = 0; e < G::E; ++e) {
        const int kx = jj * G::E + e;
        float v = 0.0f;
        if (row < kK1 * 3 && kx < kK1) v = w[((co * 3 + ch) * kK1 + ky) * kK1 + kx] * act_scale<P>();
        put_elem<P>(dst, e, weight_part<P>(v, part));
      }
    } else {
      // k-step s -> (tap, 16 or 8 input channels): tap-major, or for the pipelined kernel
      // phase-major (a phase = all nine taps of 32 input channels)
      int tap, cbase;
      int tile = t;
      if constexpr (P::PIPE) {
        static_assert(32 / G::KSTEP * 9 == kPhaseSteps, "phase shape");
        const PipeFrag pf = pipe_frag(cin, cout, fi);
        tap = pf.u / 2;
        cbase = 32 * pf.ph + (pf.u % 2) * G::KSTEP;
        tile = pf.t;
      } else {
        const int kc_per_tap = cin / G::KSTEP;
        tap = s / kc_per_tap;
        cbase = (s - tap * kc_per_tap) * G::KSTEP;
      }
      const int cot = 32 * tile + m;
      for (int e = 0; e < G::E; ++e) {
        const int c = cbase + h * G::E + e;
        put_elem<P>(dst, e, weight_part<P>(w[(cot * cin + c) * 9 + tap], part));
      }
    }
    return;
  }
  // fp32 tail: biases, head weights, head biases
  const int ti = (int)(gid - nfl);
  if (ti < G::TAIL_SW) {  // the sw[] words behind it are written by lo_scale_kernel
    float *tail = reinterpret_cast<float *>(prm.packed + G::TAIL_OFF);
    float v = 0.0f;
    if (ti < kBiasTotal) {
      int l = 0;
      while (ti >= bias_offset(l + 1)) ++l;
      v = prm.conv_b(l) ? prm.conv_b(l)[ti - bias_offset(l)] * act_scale<P>() : 0.0f;
    } else if (ti < kBiasTotal + kHeadC) {
      v = prm.pol_w[ti - kBiasTotal] / act_scale<P>();
    } else if (ti < kBiasTotal + 2 * kHeadC) {
      v = prm.val_w ? prm.val_w[ti - kBiasTotal - kHeadC] / act_scale<P>() : 0.0f;
    } else if (ti == kBiasTotal + 2 * kHeadC) {
      v = prm.pol_b ? prm.pol_b[0] : 0.0f;
    } else if (ti == kBiasTotal + 2 * kHeadC + 1) {
      v = prm.val_b ? prm.val_b[0] : 0.0f;
    }
    tail[ti] = v;
  }
}

// sw[l] = largest power of two that keeps 2^sw * max|w_l| inside the range of the low-order
// weight copy's format (one block per layer)
template <class P> __global__ __launch_bounds__(256) void lo_scale_kernel(const PackParams all) {
  using G = Geo<P>;
  const GroupView prm(all, blockIdx.y);
  __shared__ float red[256];
  const int l = blockIdx.x;
  int *sw = reinterpret_cast<int *>(prm.packed + G::TAIL_OFF) + G::TAIL_SW;
  if (l == 0) {
    if (threadIdx.x == 0) sw[0] = 0;
    return;
  }
  const int n = kCoutArr[l] * kCinArr[l] * 9;
  float m = 0.0f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) m = fmaxf(m, fabsf(prm.conv_w(l)[i]));
  red[threadIdx.x] = m;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    int e = 0;
    constexpr float kLargest = 7.5f;  // of e2m3
    if (red[0] > 0.0f && red[0] < INFINITY) e = (int)floorf(log2f(kLargest / red[0]));
    sw[l] = e < -20 ? -20 : (e > 20 ? 20 : e);
  }
}

// ------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------
template <class P> static int launch_pack(const PackParams &pp, hipStream_t st) {
  using G = Geo<P>;
  const long long total = (long long)G::TOTAL_FRAGS * 64 + G::TAIL_FLOATS;
  const int threads = 256;
  const int blocks = (int)((total + threads - 1) / threads);
  const unsigned sets = (unsigned)pp.groups;
  if constexpr (P::LO6) hipLaunchKernelGGL(lo_scale_kernel<P>, dim3(8, sets), dim3(256), 0, st, pp);
  hipLaunchKernelGGL(pack_kernel<P>, dim3(blocks, sets), dim3(threads), 0, st, pp);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("pack_kernel launch failed: %s", hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  return C6_OK;
}

template <class P> static int launch_forward(const FwdParams &fp, hipStream_t st) {
  using G = Geo<P>;
  static_assert(G::LDS_BYTES <= 160 * 1024, "activation tile must fit the 160 KiB LDS of a CU");
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  static thread_local int configured_dev = -1;
  static thread_local int cus = 0;
  const void *kernel;
  if constexpr (P::PIPE) {
    kernel = reinterpret_cast<const void *>(&fused_pipe_kernel<P>);
  } else {
    kernel = reinterpret_cast<const void *>(&fused_forward_kernel<P>);
  }
  if (e == hipSuccess && configured_dev != dev) {
    e = hipFuncSetAttribute(kernel,
                            hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
    int n = 0;
    if (e == hipSuccess) e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess) {
      configured_dev = dev;
      cus = n;
    }
  }
  if (e != hipSuccess) {
    set_error("fused_forward setup failed: %s", hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  long long grid = cus > 0 ? cus : 256;
  if (grid > fp.total_boards) grid = fp.total_boards;
  if constexpr (P::PIPE) {
    hipLaunchKernelGGL(fused_pipe_kernel<P>, dim3((unsigned)grid), dim3(256), G::LDS_BYTES, st, fp);
  } else {
    hipLaunchKernelGGL(fused_forward_kernel<P>, dim3((unsigned)grid), dim3(256), G::LDS_BYTES, st, fp);
  }
  e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("fused_forward launch failed: %s", hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  return C6_OK;
}

int dispatch_pack(int prec, const PackParams &pp, hipStream_t st) {
  if (is_cascade(prec)) {  // both sets of the cascade
    const int rc = launch_pack<PrecBF16>(pp, st);
    if (rc != C6_OK) return rc;
    PackParams second = pp;
    second.packed = pp.packed + kCascadeSecondOffset;
    return prec == C6_PREC_BF16C ? launch_pack<PrecBF16F6W>(second, st) : launch_pack<PrecBF16F6>(second, st);
  }
  switch (prec) {
    case C6_PREC_F32: return launch_pack<PrecF32>(pp, st);
    case C6_PREC_BF16: return launch_pack<PrecBF16>(pp, st);
    case C6_PREC_F16: return launch_pack<PrecF16>(pp, st);
    case C6_PREC_BF16F6: return launch_pack<PrecBF16F6>(pp, st);
    case C6_PREC_BF16F6W: return launch_pack<PrecBF16F6W>(pp, st);
  }
  set_error("unknown precision mode %d", prec);
  return C6_EINVAL;
}

int dispatch_forward(int prec, const FwdParams &fp, hipStream_t st) {
  switch (prec) {
    case C6_PREC_F32: return launch_forward<PrecF32>(fp, st);
    case C6_PREC_BF16: return launch_forward<PrecBF16>(fp, st);
    case C6_PREC_F16: return launch_forward<PrecF16>(fp, st);
    case C6_PREC_BF16F6: return launch_forward<PrecBF16F6>(fp, st);
    case C6_PREC_BF16F6W: return launch_forward<PrecBF16F6W>(fp, st);
  }
  set_error("unknown precision mode %d", prec);
  return C6_EINVAL;
}

// compute units of the current device (the grid of the persistent kernels)
static int device_cus(int &cus) {
  static thread_local int known_dev = -1, known_cus = 0;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess && dev != known_dev) {
    int n = 0;
    e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess) {
      known_dev = dev;
      known_cus = n;
    }
  }
  if (e != hipSuccess) {
    set_error("device query failed: %s", hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  cus = known_cus > 0 ? known_cus : 256;
  return C6_OK;
}

// Cascade: every board through the plain bf16 kernel, whose workgroups list those of their boards
// whose decision margin is below `threshold`; then the listed boards through the kernel that also
// carries the low parts of activations and (C6_PREC_BF16C) weights, which overwrites their
// outputs.  Two launches on the caller's stream, no host synchronisation, no atomic operation and
// nothing to clear: the second kernel reads how many boards each workgroup of the first listed.
int dispatch_cascade(int prec, const FwdParams &fp, float threshold, void *workspace, hipStream_t st) {
  int cus = 0;
  int rc = device_cus(cus);
  if (rc != C6_OK) return rc;
  const long long runs = cus < fp.total_boards ? cus : fp.total_boards;   // = the first kernel's grid
  if (runs > kCascadeMaxRuns) {
    set_error("cascade: %lld workgroups exceed the %d the workspace layout provides for", runs, kCascadeMaxRuns);
    return C6_EINVAL;
  }
  int *ws = static_cast<int *>(workspace);
  FwdParams first = fp;
  first.redo_mode = kRedoDetect;
  first.redo_threshold = threshold;
  first.redo_count = ws;
  first.redo_counts = ws + 4;
  first.redo_list = ws + 4 + kCascadeMaxRuns;
  first.redo_runs = (int)runs;
  first.redo_per = (int)((fp.total_boards + runs - 1) / runs);
  rc = launch_forward<PrecBF16>(first, st);
  if (rc != C6_OK) return rc;
  FwdParams second = first;
  second.packed = fp.packed + kCascadeSecondOffset;
  second.redo_mode = kRedoConsume;
  return prec == C6_PREC_BF16C ? launch_forward<PrecBF16F6W>(second, st) : launch_forward<PrecBF16F6>(second, st);
}

size_t packed_bytes(int prec) {
  if (is_cascade(prec)) return cascade_packed_bytes(prec);
  switch (prec) {
    case C6_PREC_F32: return Geo<PrecF32>::PACKED_BYTES;
    case C6_PREC_BF16: return Geo<PrecBF16>::PACKED_BYTES;
    case C6_PREC_F16: return Geo<PrecF16>::PACKED_BYTES;
    case C6_PREC_BF16F6: return Geo<PrecBF16F6>::PACKED_BYTES;
    case C6_PREC_BF16F6W: return Geo<PrecBF16F6W>::PACKED_BYTES;
  }
  return 0;
}

}  // namespace c6

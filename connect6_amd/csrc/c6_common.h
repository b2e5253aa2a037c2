// Shared definitions of the connect6_amd HIP sources (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/connect6_amd.h"

namespace c6 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// ---- network geometry (default architecture, connect6/model.py:22-24) ----
constexpr int kBoard = 19;
constexpr int kPix = 361;
constexpr int kLayers = 8;
constexpr int kK1 = 23;                                   // first-layer kernel
constexpr int kCinArr[8] = {3, 32, 32, 64, 64, 64, 96, 96};
constexpr int kCoutArr[8] = {32, 32, 64, 64, 64, 96, 96, 96};
constexpr int kBiasTotal = 32 + 32 + 64 + 64 + 64 + 96 + 96 + 96;  // 544
constexpr int kHeadC = 96;

// ---- on-chip activation tile -------------------------------------------
// One board lives in LDS as 421 positions x 96 channel slots, channel-last.
// Position index of square (r,c) is (r+1)*20 + (c+1): rows are 20 apart so a
// single zero column serves as right pad of one row and left pad of the next;
// rows 0 and 20 (+ position 420) are the top/bottom pad.  A 3x3 tap is then
// the constant position offset (ky-1)*20 + (kx-1).
constexpr int kPitch = 20;
constexpr int kPos = 421;
constexpr int kChSlots = 96;

// ---- first layer (23x23 on 3 planes, K = 3*529 lowered densely) -----------
// K is ordered (ky, plane, kx) with kx padded 23 -> 24; the 69 (ky,plane) rows
// are padded to 70 and split in two halves of 35: MFMA lane-half h contracts
// rows [35h, 35h+35).  The zero-padded 41-wide halo is held in E = 16/sizeof(T)
// copies, copy s shifted left by s elements, so that every 16-byte operand
// fragment (E consecutive kx of one row) is 16-byte aligned for every column.
constexpr int kL1RowsHalf = 35;
constexpr int kL1RowPitch = 40;   // elements per halo row in a shifted copy
constexpr int kL1CopyRows = 124;  // 41*3 rows + 1 zero row read by the padded K tail

// MFMA tiling: 256 threads = 4 waves; wave w owns pixels [96w, 96w+96) as three
// 32-pixel column tiles, and all Cout/32 row tiles of output channels.
constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kPixPerWave = 96;

constexpr int kRing = 6;          // weight-fragment prefetch depth (k-steps)
constexpr int kOverreadFrags = 8 * 3;  // zero frags after the last layer (prefetch may over-read)

// precision policies ----------------------------------------------------------
struct PrecF32 {
  static constexpr int WLO = 0;
  static constexpr int PIPE = 0;      // runs the layer-by-layer kernel
  static constexpr int ID = C6_PREC_F32;
  static constexpr int EB = 4;        // bytes per element
  static constexpr int LO6 = 0;
  static constexpr int LO_MASK = 0;
};
struct PrecBF16 {
  static constexpr int WLO = 0;
  static constexpr int PIPE = 1;      // runs the pipelined kernel (weights packed phase-major)
  static constexpr int ID = C6_PREC_BF16;
  static constexpr int EB = 2;
  static constexpr int LO6 = 0;
  static constexpr int LO_MASK = 0;
};
struct PrecF16 {
  static constexpr int WLO = 0;
  static constexpr int PIPE = 1;
  static constexpr int ID = C6_PREC_F16;
  static constexpr int EB = 2;
  static constexpr int LO6 = 0;
  static constexpr int LO_MASK = 0;
};
struct PrecBF16F6 {
  static constexpr int WLO = 0;
  static constexpr int PIPE = 1;
  static constexpr int ID = C6_PREC_BF16F6;
  static constexpr int EB = 2;
  static constexpr int LO6 = 1;       // bf16 plane + what its rounding dropped as block-scaled fp6 (e2m3)
  // Bit l set = 3x3 layer l (0-based) runs a low-order pass over its input.  Every layer does:
  // over 16 weight seeds at B=4096 (kernel against the fp32 kernel, mean argmax agreement with
  // the reference's initialisation / with PyTorch's default one) all layers give 99.23 / 99.55 %,
  // without the last layer 99.17 / 93.3 %, without the last two 99.07 / 93.0 %, without layers 2
  // and 3 99.10 / 99.56 %: flat-logit networks need the late layers, the others every layer.
  // (connect6_amd/profiling.py builds copies with other masks to price the layers one by one)
#ifndef C6_LO_MASK
#define C6_LO_MASK 0xfe
#endif
  static constexpr int LO_MASK = C6_LO_MASK;
};

// bf16 + fp6 + the weights' low part: PrecBF16F6 with every weight fragment of the main pass
// followed by a second fragment holding what the weights' rounding to bf16 dropped, itself
// rounded to bf16 (w = hi + lo to 16 mantissa bits); each activation fragment is contracted with
// both.  Twice the bf16 matrix work of the plain pass; what is left against fp32 arithmetic is
// the e2m3 rounding of the activations' low part (measured 2e-4 relative L2 on the logits).  The
// cascade's second pass.
struct PrecBF16F6W {
  static constexpr int WLO = 1;
  static constexpr int PIPE = 1;
  static constexpr int ID = C6_PREC_BF16F6W;
  static constexpr int EB = 2;
  static constexpr int LO6 = 1;
  static constexpr int LO_MASK = 0xfe;
};

// bf16 + fp6 mode: what rounding an activation to bf16 drops (|lo| <= 2^-9 |a|) is contracted
// with an e2m3 copy of the weights in a second pass of v_mfma_scale_f32_32x32x64_f8f6f4 (K = 64
// per instruction at four times the bf16 rate).  The weight copy of layer l is scaled by 2^sw[l]
// (sw in the packed tail, from max|w|); the instruction's block scales undo the factors.  The 32
// bytes that hold 32 low-order values of a position are 24 bytes of packed 6-bit values, one E8M0
// scale byte (the block's power-of-two scale, taken from the largest of the 32 values) and
// padding; the instruction applies the scale per lane.  A block is the 32 channels of one cout
// tile; which K slot a channel takes follows from which lane holds it after the MFMA
// (lo6_channel).
constexpr int kLoRing = 3;            // low-order weight prefetch ring depth (64-wide K chunks)
__host__ __device__ constexpr int lo6_channel(int block, int slot) {
  // block = cout tile of the producing layer; a lane of that MFMA holds 16 of the tile's channels
  // (register i, lane half hh).  Lane half 0 fills K slots 0-15, lane half 1 slots 16-31; inside
  // a half, slot 2i' holds register i' and slot 2i'+1 register 8 + i' (how the conversion
  // instruction interleaves its two operands).
  const int hh = slot >> 4, s = slot & 15;
  const int i = (s >> 1) + 8 * (s & 1);
  return 32 * block + 8 * (i >> 2) + 4 * hh + (i & 3);
}

template <class P> struct Geo {
  static constexpr int EB = P::EB;
  static constexpr int E = 16 / EB;                 // elements per 16-byte fragment lane
  static constexpr int KSTEP = 2 * E;               // K elements contracted per fragment pair
  static constexpr int W = P::WLO ? 2 : 1;          // weight fragments per (k-step, cout tile): hi, or hi then lo
  static constexpr int PLANE = kChSlots * EB;       // bytes of one precision plane of a position
  static constexpr int LO_OFF = PLANE;              // the fp6 blocks follow the bf16 plane
  static constexpr int RECB = PLANE + (P::LO6 ? kChSlots : 0);  // payload bytes
  // LDS bank conflicts: a ds_read_b128 is served 16 lanes at a time, so 16 consecutive
  // positions must land on 16 different 16-byte bank groups.  192-byte records get there
  // with 16 bytes of padding (stride 208 = 13 x 16); the 384-byte records of fp32 would
  // not fit the LDS padded, so they XOR the 16-byte granule index with (position>>1)&7.
  static constexpr bool PADDED = (EB == 2);
  static constexpr int PIXB = PADDED ? RECB + 16 : RECB;  // bytes per position
  static constexpr int ACT_BYTES = kPos * PIXB;
  static constexpr int CPR = 24 / E;                // fragments per first-layer K row
  static constexpr int STEPS1 = kL1RowsHalf * CPR;  // first-layer k-steps
  static constexpr int COPY_BYTES = kL1CopyRows * kL1RowPitch * EB;
  static constexpr int COPIES_BYTES = E * COPY_BYTES;
  static constexpr int BUF_BYTES = ACT_BYTES > COPIES_BYTES ? ACT_BYTES : COPIES_BYTES;
  // LDS map: [activation tile | first-layer copies] [occupancy 384] [logits 361 f32] [partials]
  static constexpr int OCC_OFF = (BUF_BYTES + 15) & ~15;
  static constexpr int LGT_OFF = OCC_OFF + 384;
  static constexpr int RED_OFF = LGT_OFF + 1456;
  // pipelined kernel: a copy of the weight set's fp32 tail (biases, head weights), so that no
  // layer starts, and the heads do not run, behind the latency of global loads
  static constexpr int TAIL_LDS_OFF = RED_OFF + 64;
  // ... and the next board's input as the loads deliver it, one dword per element: words
  // [0, 1083) the three planes, words 1084 / 1085 side to move / stones left (board-state input),
  // words [1088, 1088 + 361) the legality bytes or the int8 stones.  The loads write LDS
  // directly, so the input never sits in registers (or, under register pressure, in scratch).
  static constexpr int NEXT_IN_OFF = TAIL_LDS_OFF + (kBiasTotal + 2 * kHeadC + 4) * 4;
  static constexpr int NEXT_IN_AUX = 1084, NEXT_IN_BYTES_AT = 1088;
  // ... and, for the cascade's second pass, the running sums of the first pass's per-workgroup
  // counts of listed boards (kCascadeMaxRuns + 1 ints)
  static constexpr int RUNS_OFF = NEXT_IN_OFF + (NEXT_IN_BYTES_AT + 384) * 4;
  static constexpr int LDS_BYTES = P::PIPE ? RUNS_OFF + (1024 + 1 + 3) * 4 : TAIL_LDS_OFF;

  static constexpr int layer_steps(int l) { return l == 0 ? STEPS1 : 9 * kCinArr[l] / KSTEP; }
  static constexpr int layer_frags(int l) { return layer_steps(l) * (kCoutArr[l] / 32) * W; }
  static constexpr int frag_offset(int l) {  // in 1 KiB fragments
    int s = 0;
    for (int i = 0; i < l; ++i) s += layer_frags(i);
    return s;
  }
  static constexpr int HI_FRAGS = frag_offset(8) + kOverreadFrags;
  // fp6 copy of the 3x3 layers' weights (LO6 mode only).  K is cut into half-chunks of 32
  // channels of one tap; a 64-wide chunk is two consecutive half-chunks, one per lane half.
  // A lane's 24 bytes of (chunk, cout tile) are piece 0 = 64 lanes x 16 B and piece 1 = 64 lanes
  // x 8 B, densely packed at the start of a second 1 KiB fragment.
  static constexpr int lo_half_chunks(int l) { return 9 * kCinArr[l] / 32; }
  static constexpr int lo_chunks(int l) { return (lo_half_chunks(l) + 1) / 2; }
  static constexpr int lo_layer_frags(int l) { return l == 0 ? 0 : lo_chunks(l) * (kCoutArr[l] / 32) * 2; }
  static constexpr int lo_frag_offset(int l) {  // in 1 KiB fragments, from the start of the buffer
    int s = HI_FRAGS;
    for (int i = 0; i < l; ++i) s += lo_layer_frags(i);
    return s;
  }
  static constexpr int LO_FRAGS = P::LO6 ? (lo_frag_offset(8) - HI_FRAGS) + kLoRing * 3 * 2 : 0;
  // Pipelined kernel, first layer on a board whose third plane is one constant c (what the
  // reference feeds it: the "last stone of the turn" flag broadcast over the board,
  // connect6/vector_env.py:211-217): that plane's contribution is c * (sum of its weights
  // inside the board, seen from the output square) -- a per-square table, added with the bias --
  // and K shrinks to the other two planes, one per lane half: 23 kernel rows x 3 fragments of
  // 8 columns = 69 k-steps instead of 105.  A second copy of the first layer's weights in that
  // order follows the low-order copies, then the table, laid out as the lanes hold it: fragment
  // ((wave * 3 + pixel tile) * 4 + q) = 64 lanes x four fp32 (channels 8 q + 4 h .. + 3 of the
  // lane's square), one coalesced 16-byte load per lane each.
  static constexpr int FAST1_STEPS = kK1 * CPR;
  static constexpr int FAST1_OFF = HI_FRAGS + LO_FRAGS;  // in 1 KiB fragments
  static constexpr int FAST1_STREAM = FAST1_STEPS * W;   // fragments of that copy
  static constexpr int PLANE2_FRAG_OFF = FAST1_OFF + FAST1_STREAM + 8;  // (8 zero fragments: over-read)
  static constexpr int PLANE2_FRAGS = kWaves * 3 * 4;
  static constexpr int FAST1_FRAGS = (P::PIPE && EB == 2) ? FAST1_STREAM + 8 + PLANE2_FRAGS : 0;
  static constexpr int TOTAL_FRAGS = HI_FRAGS + LO_FRAGS + FAST1_FRAGS;
  static constexpr size_t TAIL_OFF = (size_t)TOTAL_FRAGS * 1024;  // fp32 tail: biases, heads
  // tail words: bias[544] polw[96] valw[96] polb valb pad pad, then 8 ints sw[layer]
  static constexpr int TAIL_SW = kBiasTotal + 2 * kHeadC + 4;
  static constexpr int TAIL_FLOATS = TAIL_SW + 8;
  static constexpr size_t PACKED_BYTES = TAIL_OFF + (size_t)TAIL_FLOATS * 4;
};

// Cascade modes: one packed set = the plain bf16 set, then (256-byte aligned) the set of the same
// parameters for the second pass: bf16 + fp6 + the weights' low part (C6_PREC_BF16C), or, for
// parameters that are exact in bf16 and have no low part, bf16 + fp6 (C6_PREC_BF16C6).
constexpr bool is_cascade(int prec) { return prec == C6_PREC_BF16C || prec == C6_PREC_BF16C6; }
constexpr size_t kCascadeSecondOffset = (Geo<PrecBF16>::PACKED_BYTES + 255) & ~(size_t)255;
constexpr size_t cascade_packed_bytes(int prec) {
  return kCascadeSecondOffset +
         (prec == C6_PREC_BF16C ? Geo<PrecBF16F6W>::PACKED_BYTES : Geo<PrecBF16F6>::PACKED_BYTES);
}
// Its workspace.  Every workgroup of the first pass keeps the list of its own boards that need the
// second pass (it evaluates one contiguous run of boards; its list has room for all of them) and
// writes their number when its run is done: no atomic operation, and nothing to clear before a
// call.  The second pass sums the counts up (every workgroup for itself) and deals the listed boards
// out evenly.  Layout, in int32: [0] boards listed in all (written by the second pass, for the
// caller), [4, 4 + kCascadeMaxRuns) the counts per run, then the lists, `per` entries per run
// (runs x per <= boards + runs).
constexpr int kCascadeMaxRuns = 1024;   // workgroups of the first pass = compute units, at most
constexpr size_t cascade_workspace_bytes(long long boards) {
  return (size_t)(16 + 4 * (long long)kCascadeMaxRuns + 4 * (boards + kCascadeMaxRuns) + 15) & ~(size_t)15;
}

constexpr int bias_offset(int l) {
  int s = 0;
  for (int i = 0; i < l; ++i) s += kCoutArr[i];
  return s;
}

enum : int { kRedoNone = 0, kRedoDetect = 1, kRedoConsume = 2 };

struct FwdParams {
  const void *x;
  int x_dtype;
  long long total_boards;
  long long boards_per_group;
  const unsigned char *packed;
  size_t packed_stride;
  void *logits;               // [boards, 361] of element type logits_dtype (fp32 unless the caller says so)
  int logits_dtype = C6_DT_F32;
  float *value;
  int mask_mode;
  const uint8_t *legal;
  float fill;
  const float *u;
  float inv_temperature;
  long long *actions;
  float *logprob;
  // board-state input (x_dtype == C6_DT_BOARD_I8): x is int8 boards [N,19,19] with +1/-1/0
  const int8_t *player;       // [N] side to move (+1 / -1)
  const int8_t *stones_left;  // [N] stones left in the turn
  const long long *index;     // [B] rows of the state tensors to evaluate, or null for 0..B-1
  long long num_states;       // N: index entries are clamped into [0, N) (no out-of-bounds read)
  int view;                   // D4 view 0..7 applied to the board before evaluation
  // cascade (C6_PREC_BF16C; pipelined kernel only)
  int redo_mode = kRedoNone;      // kRedoDetect: first pass, kRedoConsume: second pass
  float redo_threshold = 0.0f;    // first pass: < 0 = every board goes on the list
  int *redo_count = nullptr;      // boards listed in all (device memory; the second pass writes it)
  int *redo_counts = nullptr;     // boards listed by run r of the first pass
  int *redo_list = nullptr;       // run r's list starts at entry r * redo_per
  int redo_runs = 0;              // workgroups (runs of boards) of the first pass
  int redo_per = 0;               // boards per run of the first pass
};

struct PackParams {
  const float *conv_w[8];     // each tensor stacked over the weight sets: [groups, ...]
  const float *conv_b[8];
  const float *pol_w, *pol_b, *val_w, *val_b;
  unsigned char *packed;
  int groups = 1;             // weight sets (at most 65535: one grid row each)
  size_t packed_stride = 0;   // bytes between consecutive packed sets
};

// state and results of VectorConnect6.step (connect6/vector_env.py:33-53, :8-14 of the reference)
struct EnvParams {
  int8_t *boards;        // [N, n, n]
  int8_t *player;        // [N]
  int8_t *stones_left;   // [N]
  int16_t *empty_count;  // [N]
  int16_t *move_count;   // [N]
  const long long *actions;
  long long num;
  int n, win;
  int view;              // actions are squares of D4 view `view` of the board (0 = the board itself)
  float *reward;
  uint8_t *done;
  int8_t *winner, *sign;
  int16_t *lengths;
};

void set_error(const char *fmt, ...);

}  // namespace c6

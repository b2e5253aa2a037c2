// Batched Connect6 rules on device state for gfx950: one environment step (stone placement,
// local win check, turn bookkeeping) and the canonical network input.  Replaces
// VectorConnect6.step / _check_win_local (connect6/vector_env.py:106-193 of the reference) and
// canonical_network_input (connect6/vector_env.py:196-218), each a chain of a dozen small
// PyTorch launches there.  Both kernels are latency / HBM bound: an environment reads at most
// 8 * (win_length - 1) board bytes and a few state bytes and writes one stone and 9 result bytes.
#include "c6_common.h"
#include "c6_device.h"

namespace c6 {

// one thread per environment
__global__ __launch_bounds__(256) void env_step_kernel(const EnvParams p) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= p.num) return;
  const int n = p.n, cells = n * n;
  long long a = p.actions[i];
  a = a < 0 ? 0 : (a >= cells ? cells - 1 : a);  // never write outside the board
  if (p.view) a = d4_from_view((int)a, p.view, n);  // policy-view square -> board square
  const int row = (int)(a / n), col = (int)(a - (long long)row * n);
  int8_t *board = p.boards + i * cells;
  const int8_t actor = p.player[i];
  board[row * n + col] = actor;
  const int16_t empty = (int16_t)(p.empty_count[i] - 1);
  const int16_t moves = (int16_t)(p.move_count[i] + 1);
  p.empty_count[i] = empty;
  p.move_count[i] = moves;

  // equal stones outward from the new one, at most win - 1 each way, along 4 directions
  bool won = false;
  const int reach = p.win - 1;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int dr = d == 1 ? 0 : 1, dc = d == 0 ? 0 : (d == 3 ? -1 : 1);
    int total = 1;
#pragma unroll
    for (int s = -1; s <= 1; s += 2) {
      int r = row + s * dr, c = col + s * dc;
      for (int k = 0; k < reach; ++k) {
        if (r < 0 || r >= n || c < 0 || c >= n || board[r * n + c] != actor) break;
        ++total;
        r += s * dr;
        c += s * dc;
      }
    }
    won = won || total >= p.win;
  }
  const bool done = won || empty == 0;
  p.reward[i] = won ? 1.0f : 0.0f;
  p.done[i] = done ? 1 : 0;
  p.winner[i] = won ? actor : (int8_t)0;
  p.lengths[i] = moves;
  int8_t sign = 0;
  if (!done) {  // a finished game keeps its side to move and its stones_left
    const int8_t remaining = (int8_t)(p.stones_left[i] - 1);
    if (remaining > 0) {
      p.stones_left[i] = remaining;
      sign = 1;
    } else {
      p.player[i] = (int8_t)-actor;
      p.stones_left[i] = 2;
      sign = -1;
    }
  }
  p.sign[i] = sign;
}

// one thread per board cell: plane 0 = stone of the side to move, 1 = of the other side,
// 2 = this decision is the last stone of the turn.  (A variant with one 16-byte store per thread
// measured slower: its byte loads stop being coalesced.)
__global__ __launch_bounds__(256) void canonical_input_kernel(const int8_t *__restrict__ boards,
                                                              const int8_t *__restrict__ player,
                                                              const int8_t *__restrict__ stones_left,
                                                              long long total, int cells,
                                                              float *__restrict__ out) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long f = (long long)blockIdx.x * blockDim.x + threadIdx.x; f < total; f += stride) {
    const long long b = f / cells;
    const int cell = (int)(f - b * cells);
    const int stone = boards[f], me = player[b];
    float *o = out + b * 3 * cells + cell;
    o[0] = stone == me ? 1.0f : 0.0f;
    o[cells] = stone == -me ? 1.0f : 0.0f;
    o[2 * cells] = stones_left[b] == 1 ? 1.0f : 0.0f;
  }
}

int launch_env_step(const EnvParams &p, hipStream_t st) {
  if (p.num == 0) return C6_OK;
  const long long blocks = (p.num + 255) / 256;
  hipLaunchKernelGGL(env_step_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("env_step_kernel launch failed: %s", hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  return C6_OK;
}

int launch_canonical_input(const int8_t *boards, const int8_t *player, const int8_t *stones_left,
                           long long num, int n, float *out, hipStream_t st) {
  if (num == 0) return C6_OK;
  const int cells = n * n;
  const long long total = num * cells;
  long long blocks = (total + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;  // grid-stride beyond that
  hipLaunchKernelGGL(canonical_input_kernel, dim3((unsigned)blocks), dim3(256), 0, st, boards, player,
                     stones_left, total, cells, out);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("canonical_input_kernel launch failed: %s", hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  return C6_OK;
}

}  // namespace c6

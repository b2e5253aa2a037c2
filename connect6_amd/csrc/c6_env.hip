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

// Plane 0 = stone of the side to move, 1 = of the other side, 2 = this decision is the last
// stone of the turn.  Eight games per workgroup: their int8 boards are staged in LDS with
// coalesced loads, then the 8 x 3 x cells output floats (a whole number of 16-byte units,
// contiguous in memory) are written with 16-byte stores.
// CELLS > 0 fixes the board size at compile time (divisions become multiplications).
constexpr int kCanonGames = 8;
template <int CELLS>
__global__ __launch_bounds__(256) void canonical_input_kernel(const int8_t *__restrict__ boards,
                                                              const int8_t *__restrict__ player,
                                                              const int8_t *__restrict__ stones_left,
                                                              long long num, int cells_arg,
                                                              float *__restrict__ out) {
  const int cells = CELLS > 0 ? CELLS : cells_arg;
  extern __shared__ __attribute__((aligned(16))) int8_t s_board[];  // kCanonGames * cells, + 8 so that word reads may run past the end
  __shared__ int s_me[kCanonGames];
  __shared__ float s_last[kCanonGames];
  const long long g0 = (long long)blockIdx.x * kCanonGames;
  const int ng = (int)(num - g0 < kCanonGames ? num - g0 : kCanonGames);
  const int8_t *src = boards + g0 * cells;
  if (ng == kCanonGames && (reinterpret_cast<uintptr_t>(src) & 7u) == 0) {
    // eight boards = 8 * cells bytes: a whole number of 8-byte units
    for (int i = threadIdx.x; i < cells; i += blockDim.x)
      reinterpret_cast<v2i *>(s_board)[i] = reinterpret_cast<const v2i *>(src)[i];
  } else {
    for (int i = threadIdx.x; i < ng * cells; i += blockDim.x) s_board[i] = src[i];
  }
  if ((int)threadIdx.x < ng) {
    s_me[threadIdx.x] = player[g0 + threadIdx.x];
    s_last[threadIdx.x] = stones_left[g0 + threadIdx.x] == 1 ? 1.0f : 0.0f;
  }
  __syncthreads();
  const int per_game = 3 * cells;
  const int total = ng * per_game;
  float *dst = out + g0 * per_game;
  auto value = [&](int o) {
    const int g = o / per_game, rem = o - g * per_game;
    const int plane = rem / cells, cell = rem - plane * cells;
    const int stone = s_board[g * cells + cell], me = s_me[g];
    return plane == 2 ? s_last[g] : ((plane == 0 ? stone == me : stone == -me) ? 1.0f : 0.0f);
  };
  if ((total & 3) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
    const unsigned *words = reinterpret_cast<const unsigned *>(s_board);
    // (game, offset inside the game) of the thread's first output, then stepped by 4 * blockDim
    // per iteration: no division in the loop
    int g = (4 * (int)threadIdx.x) / per_game, rem = 4 * (int)threadIdx.x - g * per_game;
    const int step = 4 * (int)blockDim.x, step_g = step / per_game, step_rem = step - step_g * per_game;
    for (int q = threadIdx.x; q < total / 4; q += blockDim.x, g += step_g, rem += step_rem) {
      if (rem >= per_game) {
        rem -= per_game;
        ++g;
      }
      int plane = rem >= 2 * cells ? 2 : (rem >= cells ? 1 : 0);
      int cell = rem - plane * cells;
      const int g_first = g;
      f32x4 o;
      if (cell + 3 < cells) {
        // the four squares sit in one plane: fetch their bytes as one (unaligned) word and
        // compare all four with the wanted stone at once
        if (plane == 2) {
          const float l = s_last[g];
          o = f32x4{l, l, l, l};
        } else {
          const int a = g * cells + cell;
          const unsigned w = __builtin_amdgcn_alignbyte(words[(a >> 2) + 1], words[a >> 2], a & 3);
          const int me = s_me[g];
          const unsigned want = (unsigned)((plane == 0 ? me : -me) & 0xff) * 0x01010101u;
          const unsigned x = w ^ want;  // a zero byte = the wanted stone
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = ((x >> (8 * e)) & 0xffu) == 0 ? 1.0f : 0.0f;
        }
      } else {
        int gg = g_first;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int stone = s_board[gg * cells + cell], me = s_me[gg];
          o[e] = plane == 2 ? s_last[gg] : ((plane == 0 ? stone == me : stone == -me) ? 1.0f : 0.0f);
          if (++cell == cells) {
            cell = 0;
            if (++plane == 3) {
              plane = 0;
              gg = gg + 1 < ng ? gg + 1 : gg;
            }
          }
        }
      }
      reinterpret_cast<f32x4 *>(dst)[q] = o;
    }
  } else {
    for (int o = threadIdx.x; o < total; o += blockDim.x) dst[o] = value(o);
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
  const long long blocks = (num + kCanonGames - 1) / kCanonGames;
  if (n == kBoard) {
    hipLaunchKernelGGL(canonical_input_kernel<kPix>, dim3((unsigned)blocks), dim3(256),
                       (size_t)kCanonGames * cells + 8, st, boards, player, stones_left, num, cells, out);
  } else {
    hipLaunchKernelGGL(canonical_input_kernel<0>, dim3((unsigned)blocks), dim3(256),
                       (size_t)kCanonGames * cells + 8, st, boards, player, stones_left, num, cells, out);
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("canonical_input_kernel launch failed: %s", hipGetErrorString(e));
    return C6_ELAUNCH;
  }
  return C6_OK;
}

}  // namespace c6

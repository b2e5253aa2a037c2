/* connect6_amd -- C ABI of the MI355X (gfx950) Connect6 policy/value forward path.
 *
 * One shared library, plain pointers and sizes only.  Every pointer named
 * "device" is a HIP device pointer owned by the caller (PyTorch in the shipped
 * host code); the library never allocates, frees or keeps device memory, and
 * every call only enqueues work on the caller's stream (no synchronisation).
 * All functions return C6_OK (0) or a negative C6_E* code; c6_last_error()
 * gives the message of the calling thread's last failure.
 *
 * The reference implementation is pure Python on PyTorch, so it has no FFI of
 * its own; each entry point below names the reference call it replaces.
 */
#ifndef CONNECT6_AMD_H
#define CONNECT6_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define C6_BOARD 19
#define C6_ACTIONS 361
#define C6_LAYERS 8

/* return codes */
#define C6_OK 0
#define C6_EINVAL (-1)   /* bad shape / dtype / null pointer / alignment */
#define C6_ELAUNCH (-2)  /* HIP reported an error at launch */
#define C6_EARCH (-3)    /* device is not gfx950 or architecture not the default one */

/* arithmetic modes of the network ("prec") */
#define C6_PREC_F32 0    /* fp32 operands, fp32 MFMA                                        */
#define C6_PREC_BF16 1   /* bf16 operands, bf16 MFMA, fp32 accumulate, bf16 layer boundaries */
#define C6_PREC_F16 2    /* fp16 operands, fp16 MFMA, fp32 accumulate, fp16 layer boundaries */
#define C6_PREC_BF16F6 3 /* bf16 MFMA + a second pass on what the bf16 rounding of each activation
                            dropped, held as block-scaled fp6 (e2m3, one power-of-two scale per 32
                            channels), on the fp6 MFMA at four times the bf16 rate */
#define C6_PREC_BF16C 4  /* cascade: every board in C6_PREC_BF16, then the boards whose decision
                            is closer than the rounding noise again in C6_PREC_BF16F6W; needs a
                            workspace: c6_forward_cascade / c6_forward_boards_cascade */
#define C6_PREC_BF16C6 6  /* the cascade for parameters that are exact in bf16 (an ensemble or a
                            module held in bf16): the weights have no low part, so the second
                            pass is C6_PREC_BF16F6 */
#define C6_PREC_BF16F6W 5 /* C6_PREC_BF16F6 plus, in the main pass, what the rounding of the
                            weights to bf16 dropped (a second bf16 weight fragment per fragment,
                            twice the bf16 matrix work): within 3e-4 relative L2 of fp32 */

/* element types of caller tensors */
#define C6_DT_F32 0
#define C6_DT_BF16 1
#define C6_DT_F16 2
#define C6_DT_BOARD_I8 3 /* int8 board states (+1 / -1 / 0), only through c6_forward_boards */

/* masking of occupied squares in the policy logits */
#define C6_MASK_NONE 0   /* logits as the network produced them (PolicyValueNet.forward)    */
#define C6_MASK_INPUT 1  /* square occupied iff x[b,0,r,c] != 0 or x[b,1,r,c] != 0           */
#define C6_MASK_LEGAL 2  /* square occupied iff legal[b,a] == 0 (uint8 / torch.bool tensor)  */

int c6_version(void);
const char *c6_last_error(void);

/* Size in bytes of one packed weight set for arithmetic mode `prec`. */
int c6_packed_bytes(int prec, size_t *bytes);

/* Repack one checkpoint's parameters for the kernels.
 * Replaces: the parameter tensors nn.Conv2d holds in PolicyValueNet.__init__
 * (connect6/model.py:52-75) and the per-key stacking of
 * HistoricalPolicyEnsemble._stack (connect6/history.py:224-240).
 * conv_w[i] / conv_b[i]: device fp32, PyTorch layouts [Cout,Cin,k,k] / [Cout]
 * for the default architecture (kernels 23,3x7; channels 32,32,64,64,64,96,96,96);
 * conv_b[i] may be NULL (no bias).  pol_* / val_*: device fp32 [1,96,1,1] / [1];
 * val_w / val_b may be NULL (history checkpoints need no value head).
 * `conv_w` and `conv_b` themselves are HOST arrays of 8 device pointers.
 * `packed`: device buffer of c6_packed_bytes(prec) bytes, 16-byte aligned. */
int c6_pack_weights(const float *const *conv_w, const float *const *conv_b,
                    const float *pol_w, const float *pol_b, const float *val_w,
                    const float *val_b, int prec, void *packed, void *stream);

/* The same for `groups` checkpoints in one call (two launches whatever their number): every
 * parameter tensor is the checkpoints' tensors stacked along a new first dimension, as
 * HistoricalPolicyEnsemble._stack builds them (connect6/history.py:224-240): conv_w[i] device fp32
 * [groups,Cout,Cin,k,k], conv_b[i] [groups,Cout], pol_w / val_w [groups,1,96,1,1], pol_b / val_b
 * [groups,1].  Set g is written at packed + g * packed_stride (a multiple of 16 bytes, at least
 * c6_packed_bytes(prec)); 1 <= groups <= 65535. */
int c6_pack_weights_grouped(const float *const *conv_w, const float *const *conv_b,
                            const float *pol_w, const float *pol_b, const float *val_w,
                            const float *val_b, int64_t groups, int prec, void *packed,
                            size_t packed_stride, void *stream);

/* Batched forward of G weight sets, each applied to T boards, in one launch.
 * Replaces: PolicyValueNet.forward (connect6/model.py:96-111) with G = 1, and
 * HistoricalPolicyEnsemble.forward_grouped (connect6/history.py:276-303) with
 * G = number of checkpoints (value == NULL there: policy only).
 *   x       device [G*T,3,19,19] contiguous, element type x_dtype
 *   packed  device, G weight sets, consecutive sets `packed_stride` bytes apart
 *   logits  device fp32 [G*T,361] (may be NULL)
 *   value   device fp32 [G*T] (may be NULL)
 *   mask_mode / legal / fill: see C6_MASK_*; `fill` is stored bit-exactly in
 *           every masked logit (connect6/model.py:123-125 uses finfo.min).
 * Optional fused sampling (connect6/train.py:195-213, _sample_actions): when
 * `actions` is not NULL, each board also draws an action by inverse CDF on
 * u[b] in [0,1) from softmax(masked_logits / max(temperature,1e-4)) (masking
 * as selected by mask_mode, always with fill = lowest float) and writes
 * actions[b] (int64) and, if not NULL, logprob[b] (fp32). */
int c6_forward(const void *x, int x_dtype, int64_t groups, int64_t boards_per_group,
               const void *packed, size_t packed_stride, int prec, float *logits,
               float *value, int mask_mode, const uint8_t *legal, float fill,
               const float *u, float temperature, int64_t *actions, float *logprob,
               void *stream);

/* The same forward, fed directly from the environment's state tensors instead of float planes.
 * Replaces, in one launch, the collector's per-step chain (connect6/train.py:730-748,
 * :791-799): _transform_boards(boards, view) -> canonical_network_input (connect6/
 * vector_env.py:196-218: plane 0 = boards == player, plane 1 = boards == -player, plane 2 =
 * stones_left == 1) -> optional row gather (network_input[index]) -> forward -> mask_logits
 * with legal = view_boards == 0 -> optional sampling.
 *   boards       device int8 [N,19,19], values +1 / -1 / 0
 *   player       device int8 [N], side to move (+1 / -1)
 *   stones_left  device int8 [N]
 *   num_states   N
 *   index        device int64 [B] rows of the state tensors to evaluate (entries outside [0,N)
 *                are clamped into range), or NULL (rows 0..B-1, B <= N)
 *   view         D4 view 0..7 (numbering of _symmetry_for_phase); outputs are in view coordinates
 *   mask_mode    C6_MASK_NONE or C6_MASK_INPUT (occupied squares of the viewed board)
 * Remaining arguments as c6_forward with groups = 1. */
int c6_forward_boards(const int8_t *boards, const int8_t *player, const int8_t *stones_left,
                      int64_t num_states, const int64_t *index, int view, int64_t batch,
                      const void *packed,
                      int prec, float *logits, float *value, int mask_mode, float fill,
                      const float *u, float temperature, int64_t *actions, float *logprob,
                      void *stream);

/* c6_forward / c6_forward_boards in a cascade mode (`prec` = C6_PREC_BF16C, or C6_PREC_BF16C6 for
 * parameters that are exact in bf16; `packed` holds sets packed for that mode).  Replaces the same
 * reference calls as they do (connect6/model.py:96-111, connect6/history.py:276-303,
 * connect6/train.py:730-748, :791-799).
 * First every board is evaluated with plain bf16 layer boundaries.  A board is evaluated again,
 * with the corrections of C6_PREC_BF16F6W, when the rounding of the plain pass can change
 * the move that an argmax picks (reference callers: connect6/benchmark.py:32,44,
 * connect6/evaluate.py:54, connect6/gui_cnn.py:43): when its largest logit among the free squares
 * (free as C6_MASK_LEGAL or the input planes say, whatever mask_mode writes) leads the second
 * largest by less than `threshold` standard deviations of the free squares' logits, or when two
 * other free squares lie within twice that of the largest.  Its logits, value and draw replace
 * the first ones.  threshold = 0 evaluates no board twice (results of C6_PREC_BF16), threshold < 0
 * every board (results of C6_PREC_BF16F6W; with C6_PREC_BF16C6, whose second pass leaves the
 * weights' low part out because there is none, of C6_PREC_BF16F6).  The plain pass's error on a
 * difference of two logits is about 0.01 standard deviations of the logits; with threshold 0.02
 * about 6 % of the boards of a random network are evaluated twice and the argmax agrees with
 * fp32's on 99.9 % of the boards (reference initialisation, 32 networks; worst network 99.7 %).
 * A board's results do not depend on the other boards of the batch.
 *   logits     device [boards,361] of element type logits_dtype (C6_DT_F32, C6_DT_BF16 or
 *              C6_DT_F16; may be NULL): a bf16 / fp16 ensemble gets its logits rounded once (to
 *              nearest even, as Tensor.to does) by the kernel instead of by a cast behind it;
 *              `fill` is converted the same way
 *   workspace  device, c6_cascade_workspace_bytes(boards) bytes, 16-byte aligned, contents
 *              arbitrary (nothing has to be cleared: every workgroup of the first pass lists its
 *              own boards and writes how many, the second pass adds the counts up); after the
 *              call its first int32 holds the number of boards that were evaluated twice
 * Two launches on `stream`, no synchronisation with the host, no atomic operation. */
int c6_cascade_workspace_bytes(int64_t boards, size_t *bytes);
int c6_forward_cascade(const void *x, int x_dtype, int64_t groups, int64_t boards_per_group,
                       const void *packed, size_t packed_stride, int prec, void *logits,
                       int logits_dtype, float *value, int mask_mode, const uint8_t *legal, float fill, const float *u,
                       float temperature, int64_t *actions, float *logprob, float threshold,
                       void *workspace, size_t workspace_bytes, void *stream);
int c6_forward_boards_cascade(const int8_t *boards, const int8_t *player,
                              const int8_t *stones_left, int64_t num_states,
                              const int64_t *index, int view, int64_t batch, const void *packed,
                              int prec, void *logits, int logits_dtype, float *value, int mask_mode,
                              float fill,
                              const float *u, float temperature, int64_t *actions,
                              float *logprob, float threshold, void *workspace,
                              size_t workspace_bytes, void *stream);

/* Forward of ONE weight set for any architecture the reference's PolicyValueNet accepts
 * (connect6/model.py:26-77: any board size, odd kernels, positive channel counts), layer by
 * layer through a caller-provided workspace.  Compatibility path for non-default
 * architectures (the reference's own tests use board 5, kernels 3,3,3, channels 8,8,16);
 * the default architecture should use c6_forward.
 *   x        device [B,3,n,n] of element type x_dtype
 *   kernels, channels: HOST arrays of `layers` ints
 *   conv_w / conv_b:   HOST arrays of `layers` device fp32 pointers (PyTorch layouts)
 *   workspace: device, c6_generic_workspace_bytes(...) bytes, 16-byte aligned
 *   logits fp32 [B,n*n] (may be NULL), value fp32 [B] (may be NULL; val_w may then be NULL) */
int c6_generic_workspace_bytes(int64_t batch, int board, int layers, const int *channels,
                               size_t *bytes);
int c6_forward_generic(const void *x, int x_dtype, int64_t batch, int board, int layers,
                       const int *kernels, const int *channels, const float *const *conv_w,
                       const float *const *conv_b, const float *pol_w, const float *pol_b,
                       const float *val_w, const float *val_b, int prec, void *workspace,
                       size_t workspace_bytes, float *logits, float *value, int mask_mode,
                       const uint8_t *legal, float fill, void *stream);

/* c6_forward_generic for `groups` weight sets at once: one launch per layer for the whole
 * ensemble.  Replaces: the non-default-architecture case of
 * HistoricalPolicyEnsemble.forward_grouped (connect6/history.py:263-273: one grouped convolution
 * per layer over the stacked parameters).
 *   x        device [groups*boards_per_group,3,n,n]; board b uses weight set b / boards_per_group
 *   conv_w[l] device fp32 [groups,Cout,Cin,k,k], conv_b[l] [groups,Cout] (the reference's stacked
 *            layouts, connect6/history.py:224-240); pol_w [groups,C], pol_b [groups],
 *            val_w [groups,C], val_b [groups]
 *   workspace: c6_generic_workspace_bytes(groups*boards_per_group, ...) bytes
 * Everything else as c6_forward_generic. */
int c6_forward_generic_grouped(const void *x, int x_dtype, int64_t groups,
                               int64_t boards_per_group, int board, int layers,
                               const int *kernels, const int *channels,
                               const float *const *conv_w, const float *const *conv_b,
                               const float *pol_w, const float *pol_b, const float *val_w,
                               const float *val_b, int prec, void *workspace,
                               size_t workspace_bytes, float *logits, float *value, int mask_mode,
                               const uint8_t *legal, float fill, void *stream);

/* c6_forward_generic without a workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference.  The layer-boundary activations go through a 16 MiB
 * array that lives in the library's device image (one copy per GPU, held until the process
 * ends); a batch whose c6_generic_workspace_bytes() exceeds that returns C6_EINVAL.  The call
 * allocates and frees nothing.  All calls on one GPU share that array: calls that overlap in
 * time on one GPU (different streams or threads) race; calls on one stream are safe back to
 * back.  The first call on a device looks the array's address up (hipGetSymbolAddress, which
 * may load the code object and take the memory): a caller under graph capture makes one call
 * per device outside the capture first; every later call only enqueues kernels.  Arguments and
 * results as c6_forward_generic. */
int c6_forward_generic_static(const void *x, int x_dtype, int64_t batch, int board, int layers,
                              const int *kernels, const int *channels,
                              const float *const *conv_w, const float *const *conv_b,
                              const float *pol_w, const float *pol_b, const float *val_w,
                              const float *val_b, int prec, float *logits, float *value,
                              int mask_mode, const uint8_t *legal, float fill, void *stream);

/* Out-of-place occupied-square masking of existing logits.
 * Replaces: mask_logits (connect6/model.py:123-125).
 * logits/out: device [B,361] of element type dtype; legal: device uint8 [B,361];
 * fill_bits: the fill value's bit pattern in that element type.  Operands that are 16-byte
 * (legal: 8-byte) aligned take the vector kernels; anything else that is element-aligned, such
 * as a row slice of a larger tensor, takes an element-wise kernel. */
int c6_mask_logits(const void *logits, const uint8_t *legal, int dtype, int64_t batch,
                   uint32_t fill_bits, void *out, void *stream);

/* Masked softmax + inverse-CDF categorical sampling of existing logits.
 * Replaces: _sample_actions / _sample_actions_only (connect6/train.py:195-213).
 * logits fp32 [B,361]; legal uint8 [B,361] or NULL; u fp32 [B] in [0,1);
 * actions int64 [B]; logprob fp32 [B] or NULL. */
int c6_softmax_sample(const float *logits, const uint8_t *legal, const float *u,
                      float temperature, int64_t batch, int64_t *actions, float *logprob,
                      void *stream);

/* Eight D4 views of network inputs, in the order of _symmetry_for_phase
 * (connect6/train.py:216-219); view p is _transform_boards(x, p%4, p>=4)
 * (connect6/train.py:222-230).  x: device [B,3,19,19]; out: [8,B,3,19,19];
 * both of element type dtype. */
int c6_d4_expand(const void *x, int dtype, int64_t batch, void *out, void *stream);

/* Map the eight views' logits back with _transform_actions
 * (connect6/train.py:233-253) and average logits and values over the views.
 * view_logits fp32 [8,B,361], view_values fp32 [8,B] (may be NULL with values);
 * logits fp32 [B,361]; values fp32 [B]. */
int c6_d4_reduce(const float *view_logits, const float *view_values, int64_t batch,
                 float *logits, float *values, void *stream);

/* One step of N Connect6 games held as device tensors.
 * Replaces: VectorConnect6.step and _check_win_local (connect6/vector_env.py:106-193).
 * State, updated in place (layouts of connect6/vector_env.py:33-53):
 *   boards int8 [N,n,n] (+1 / -1 / 0), current_player int8 [N], stones_left int8 [N],
 *   empty_count int16 [N], move_count int16 [N]
 * actions int64 [N]: square row*n + col each game plays (values outside [0, n*n) are clamped;
 *   like the reference without debug_checks, an occupied square is overwritten).
 * view: 0, or the D4 view 1..7 (numbering of _symmetry_for_phase) the actions are expressed
 *   in; they are mapped back as _inverse_transform_actions does (connect6/train.py:256-277,
 *   :854-862) before the stone is placed.
 * Results (connect6/vector_env.py:8-14, StepBatch): reward fp32 [N] (1 if the move made a line
 * of win_length or more), done uint8/bool [N] (win, or board full), winner int8 [N],
 * transition_sign int8 [N] (+1 same side moves again, -1 side changed, 0 game over),
 * game_lengths int16 [N] (= move_count after the move).  A finished game keeps its side to
 * move and stones_left; the caller resets it. */
int c6_env_step(int8_t *boards, int8_t *current_player, int8_t *stones_left, int16_t *empty_count,
                int16_t *move_count, const int64_t *actions, int view, int64_t num_envs,
                int board_size, int win_length, float *reward, uint8_t *done, int8_t *winner,
                int8_t *transition_sign, int16_t *game_lengths, void *stream);

/* Network input planes of N games.
 * Replaces: canonical_network_input (connect6/vector_env.py:196-218).
 * out fp32 [N,3,n,n]: plane 0 = boards == current_player, plane 1 = boards == -current_player,
 * plane 2 = stones_left == 1 (broadcast over the board). */
int c6_canonical_input(const int8_t *boards, const int8_t *current_player,
                       const int8_t *stones_left, int64_t num_envs, int board_size, float *out,
                       void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CONNECT6_AMD_H */

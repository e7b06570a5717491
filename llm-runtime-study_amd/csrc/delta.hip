// Linear-recurrent mixers whose state per head is a matrix S [dim, vdim] in float32: the gated delta rule (with one
// decay a head, or one a head and key channel) and the selective state space recurrence (at the end of this file).
//
// For every token, with q and k unit vectors of the head's key group, v the head's value, beta in (0, 1) the
// step size and g in (0, 1) the decay:
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// so the read-out sees the token's own write.  Everything here is float32 whatever the run's dtype: only the
// projections that feed it and the output that leaves it may be bfloat16.
//
// Three kernels serve a step of any shape (prompt portions and single tokens side by side):
//   delta_prepare   per (token, head): the short causal convolution over time of the q, k and v channels
//                   (taps before the step's first token come from the request's state), silu, unit norm of
//                   q and k, and the two gates of the recurrence;
//   delta_conv_keep per (request, channel): the last taps-1 inputs of the convolution, for the next step;
//   delta_scan      per (request, head, 16 columns of S): walks the request's tokens in order with its part of S in
//                   registers, a column shared by the 16 lanes of a row of lanes;
//   delta_gate      per (token, head): the read-out divided by its root mean square over vdim, times the norm's
//                   weight, times silu of the output gate.
// A request's state row holds S for every head and then the convolution's inputs:
//   S of head h at h * rows * vdim * 16 floats, element (i, j) at ((i % rows) * vdim + j) * 16 + i / rows with
//   rows = 4, 8 or 16 (dim over the 16 lanes of a column, padded): the order in which the scan's threads hold it,
//   so that loading and storing it are whole lines; then [taps - 1, channels], oldest first.
#include "common.h"

namespace {

constexpr int SPLIT = 16;     // lanes that share a column of S (one row of lanes: their sums need no LDS)
constexpr int COLUMNS = 16;   // columns of S a workgroup of 256 threads owns
// tokens whose inputs are staged in LDS at a time: 16, or 8 for the widest keys (two buffers stay within 64 KB)

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }

template <typename TP>
__global__ void delta_prepare_kernel(const TP* __restrict__ proj, int ld, const int* __restrict__ token_request,
                                     const int* __restrict__ cu, const int* __restrict__ slot_ids,
                                     float* __restrict__ state, int64_t state_stride, int64_t conv_offset,
                                     const float* __restrict__ conv_w, int taps, int G, int H, int d, int dv,
                                     const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                     float* __restrict__ qkv, float* __restrict__ gates, int keep_inside, int beta_at, int decay_at,
                                     int decay_rank, const float* __restrict__ decay_up, float* __restrict__ decays) {
  // beta_at, decay_at: the columns of proj that hold the step sizes (H) and the decay inputs: H of them, or, with
  // decay_rank > 0, decay_rank values that decay_up [decay_rank, H * d] carries to one input per head and key channel
  // (dt_bias then holds H * d values and decays [tokens, H * d] receives the decays; gates' second half is left alone);
  // decay_rank < 0: decays holds those H * d inputs of every token already (a product made them) and is turned into the decays in place
  // keep_inside: every request brings one token, so this wave alone reads and writes its channels' kept inputs of its
  // request: it moves them on itself (no delta_conv_keep launch)
  const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  const int channels = 2 * G * d + H * dv;
  const int r = token_request[t], start = cu[r], at = t - start;
  float* kept = state + (int64_t)slot_ids[r] * state_stride + conv_offset;
  const bool is_v = unit >= 2 * G;
  const int c0 = is_v ? 2 * G * d + (unit - 2 * G) * dv : unit * d, n = is_v ? dv : d;
  float* out = qkv + (int64_t)t * channels + c0;
  float ss = 0.f;
  for (int i = lane; i < n; i += WAVE) {
    const int c = c0 + i;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int s = at - (taps - 1 - j);
      const float x = s >= 0 ? to_float(proj[(int64_t)(start + s) * ld + c]) : kept[(int64_t)(taps - 1 + s) * channels + c];
      acc = fmaf(conv_w[(int64_t)c * taps + j], x, acc);
      if (keep_inside && j > 0) kept[(int64_t)(j - 1) * channels + c] = x;      // input j of this token's window is entry j - 1 of the next one's
    }
    const float y = silu_f(acc);
    out[i] = y;
    ss = fmaf(y, y, ss);
  }
  if (!is_v) {
    ss = wave_sum(ss);
    // unit vectors; the queries also carry the 1 / sqrt(dim) of the scores
    const float scale = (unit < G ? 1.0f / sqrtf((float)d) : 1.0f) / sqrtf(ss + 1e-6f);
    for (int i = lane; i < n; i += WAVE) out[i] *= scale;
  } else {
    const int h = unit - 2 * G;
    const int64_t row = (int64_t)t * ld;
    if (lane == 0) gates[(int64_t)t * 2 * H + h] = 1.f / (1.f + expf(-to_float(proj[row + beta_at + h])));
    if (decay_rank != 0) {
      const float rate = expf(a_log[h]);
      for (int i = lane; i < d; i += WAVE) {
        float a = dt_bias[h * d + i];
        if (decay_rank < 0) a += decays[(int64_t)t * H * d + h * d + i];
        for (int r = 0; r < decay_rank; ++r) a = fmaf(to_float(proj[row + decay_at + r]), decay_up[(int64_t)r * H * d + h * d + i], a);
        const float softplus = a > 20.f ? a : log1pf(expf(a));
        decays[(int64_t)t * H * d + h * d + i] = expf(-rate * softplus);
      }
    } else if (lane == 0) {
      const float a = to_float(proj[row + decay_at + h]) + dt_bias[h];
      const float softplus = a > 20.f ? a : log1pf(expf(a));
      gates[(int64_t)t * 2 * H + H + h] = expf(-expf(a_log[h]) * softplus);
    }
  }
}

template <typename TP>
__global__ void delta_conv_keep_kernel(const TP* __restrict__ proj, int ld, const int* __restrict__ cu,
                                       const int* __restrict__ slot_ids, float* __restrict__ state, int64_t state_stride,
                                       int64_t conv_offset, int taps, int channels, int first_column) {
  // first_column: where the convolution's channels begin in a row of proj
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int start = cu[r], n = cu[r + 1] - start;
  float* kept = state + (int64_t)slot_ids[r] * state_stride + conv_offset;
  // entry j becomes the input n - (taps - 1) + j of this step, or the old entry j + n: read from further on only
  for (int j = 0; j < taps - 1; ++j) {
    const int s = n - (taps - 1) + j;
    kept[(int64_t)j * channels + c] = s >= 0 ? to_float(proj[(int64_t)(start + s) * ld + first_column + c]) : kept[(int64_t)(taps - 1 + s) * channels + c];
  }
}

// A 16-lane sum that every lane of the row gets: four adds whose second operand comes through the lanes' crossbar
// (quad swaps, then the row mirrored by halves and whole), no LDS.
template <int CTRL>
__device__ __forceinline__ float from_lane(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row_sum16(float v) {
  v += from_lane<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  v += from_lane<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  v += from_lane<0x141>(v);    // row_half_mirror
  v += from_lane<0x140>(v);    // row_mirror
  return v;
}

// One workgroup of 256 threads owns 16 columns of one head's matrix for one request: thread (column c, part s) holds
// the ROWS rows s * rows .. of column c in registers, so a token costs each thread 4 * rows multiply-adds and two
// 16-lane sums, and a head of 128 columns is spread over eight compute units.  Both products with the old matrix are
// taken in one pass (the read-out of the new one follows from them: S'^T q = g S^T q + u (k . q)), then the matrix is
// updated.  The inputs of CHUNK tokens are staged in LDS, the next chunk's on their way into registers meanwhile.
//
// RULE says which recurrence: RULE_DELTA as above; RULE_PLAIN without the correction (u = v: S <- g S + k v^T, what a
// state space layer does with k = B, q = C, v = dt x); RULE_DELTA_CHANNELS with a decay per key channel (decays
// [tokens, H * d]: row i of S is multiplied by its own decay first, then the rule runs with g = 1).
enum { RULE_DELTA = 0, RULE_PLAIN = 1, RULE_DELTA_CHANNELS = 2 };

template <int ROWS, int CHUNK, int RULE>
__global__ __launch_bounds__(256) void delta_scan_kernel(const float* __restrict__ qkv, const float* __restrict__ gates,
                                                         const int* __restrict__ cu, const int* __restrict__ slot_ids,
                                                         float* __restrict__ state, int64_t state_stride, int G, int H, int d,
                                                         int dv, float* __restrict__ raw_out, const float* __restrict__ decays) {
  constexpr int VECTORS = RULE == RULE_DELTA_CHANNELS ? 3 : 2;    // arrays of CHUNK x dpad values a buffer holds: k, q (, decays)
  constexpr int K4 = ROWS / 4;                 // float4 pieces of a thread's slice of a key
  constexpr int rows = ROWS;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int r = blockIdx.x, h = blockIdx.y, block = blockIdx.z, tid = threadIdx.x;
  const int dpad = rows * SPLIT, channels = 2 * G * d + H * dv, hk = h / (H / G);
  const int per_buffer = CHUNK * (VECTORS * dpad + COLUMNS + 4);
  const int c = tid / SPLIT, s = tid % SPLIT, column = block * COLUMNS + c;
  const bool mine = column < dv;
  const int start = cu[r], n = cu[r + 1] - start;
  float* st = state + (int64_t)slot_ids[r] * state_stride + (int64_t)h * rows * dv * SPLIT + (int64_t)block * COLUMNS * SPLIT;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) S[i] = mine ? st[(int64_t)i * dv * SPLIT + tid] : 0.f;

  // what a thread brings in of a chunk: pieces of four values of the keys and queries (CHUNK * dpad / 4 pieces each,
  // at most KQ of them a thread), one value of the 16 columns' v, and the scalars of a token (step, decay, k . q)
  constexpr int KQ = (CHUNK * ROWS * SPLIT / 4 + 255) / 256;
  float4 k_reg[KQ], q_reg[KQ], g_reg[RULE == RULE_DELTA_CHANNELS ? KQ : 1];
  float v_reg = 0.f, scalar_reg = 0.f;
  const int pieces = CHUNK * dpad / 4, row_pieces = dpad / 4;
  const bool d_whole = d % 4 == 0 && channels % 4 == 0;     // every piece of four is 16 bytes aligned
  auto fetch = [&](int c0) {
    const int count = min(CHUNK, n - c0);
#pragma unroll
    for (int p = 0; p < KQ; ++p) {
      const int e = tid + p * 256, tt = e / row_pieces, i = (e % row_pieces) * 4;
      k_reg[p] = q_reg[p] = make_float4(0.f, 0.f, 0.f, 0.f);
      if constexpr (RULE == RULE_DELTA_CHANNELS) {
        g_reg[p] = make_float4(1.f, 1.f, 1.f, 1.f);
        if (e < pieces && tt < count) {
          const float* grow = decays + (int64_t)(start + c0 + tt) * H * d + h * d + i;
          if (d % 4 == 0 && i + 4 <= d) {
            g_reg[p] = *(const float4*)grow;
          } else {
            float gg[4] = {1.f, 1.f, 1.f, 1.f};
            for (int x = 0; x < 4; ++x)
              if (i + x < d) gg[x] = grow[x];
            g_reg[p] = make_float4(gg[0], gg[1], gg[2], gg[3]);
          }
        }
      }
      if (e < pieces && tt < count) {
        const float* row = qkv + (int64_t)(start + c0 + tt) * channels + hk * d + i;
        if (d_whole && i + 4 <= d) {
          q_reg[p] = *(const float4*)row;
          k_reg[p] = *(const float4*)(row + G * d);
        } else {
          float kq[8] = {};
          for (int x = 0; x < 4; ++x)
            if (i + x < d) {
              kq[x] = row[x];
              kq[4 + x] = row[G * d + x];
            }
          q_reg[p] = make_float4(kq[0], kq[1], kq[2], kq[3]);
          k_reg[p] = make_float4(kq[4], kq[5], kq[6], kq[7]);
        }
      }
    }
    const int tt = tid / COLUMNS, cc = tid % COLUMNS;
    v_reg = (tt < CHUNK && tt < count && block * COLUMNS + cc < dv) ? qkv[(int64_t)(start + c0 + tt) * channels + 2 * G * d + h * dv + block * COLUMNS + cc] : 0.f;
    scalar_reg = 0.f;
    if (tid < 2 * CHUNK && tid / 2 < count) scalar_reg = gates[(int64_t)(start + c0 + tid / 2) * 2 * H + (tid % 2) * H + h];
  };
  auto stage = [&](float* buf) {
    float* k_l = buf;
    float* q_l = buf + CHUNK * dpad;
#pragma unroll
    for (int p = 0; p < KQ; ++p) {
      const int e = tid + p * 256;
      if (e < pieces) {
        *(float4*)(k_l + e * 4) = k_reg[p];
        *(float4*)(q_l + e * 4) = q_reg[p];
        if constexpr (RULE == RULE_DELTA_CHANNELS) *(float4*)(buf + 2 * CHUNK * dpad + e * 4) = g_reg[p];
      }
    }
    if (tid < CHUNK * COLUMNS) buf[VECTORS * CHUNK * dpad + tid] = v_reg;      // [CHUNK][COLUMNS]
    if (tid < 2 * CHUNK) buf[VECTORS * CHUNK * dpad + CHUNK * COLUMNS + (tid / 2) * 4 + tid % 2] = scalar_reg;
  };
  fetch(0);
  int turn = 0;
  for (int c0 = 0; c0 < n; c0 += CHUNK, turn ^= 1) {
    float* buf = lds + turn * per_buffer;
    stage(buf);
    __syncthreads();
    if (c0 + CHUNK < n) fetch(c0 + CHUNK);
    const int count = min(CHUNK, n - c0);
    const float* k_l = buf + s * rows;
    const float* q_l = buf + CHUNK * dpad + s * rows;
    const float* d_l = buf + 2 * CHUNK * dpad + s * rows;       // the channels' decays, where the rule has them
    const float* v_l = buf + VECTORS * CHUNK * dpad;
    const float* g_l = v_l + CHUNK * COLUMNS;
    for (int tt = 0; tt < count; ++tt) {
      float kk[ROWS], qq[ROWS];
#pragma unroll
      for (int p = 0; p < K4; ++p) {
        const float4 a = *(const float4*)(k_l + tt * dpad + 4 * p), b = *(const float4*)(q_l + tt * dpad + 4 * p);
        kk[4 * p] = a.x, kk[4 * p + 1] = a.y, kk[4 * p + 2] = a.z, kk[4 * p + 3] = a.w;
        qq[4 * p] = b.x, qq[4 * p + 1] = b.y, qq[4 * p + 2] = b.z, qq[4 * p + 3] = b.w;
        if constexpr (RULE == RULE_DELTA_CHANNELS) {
          const float4 e = *(const float4*)(d_l + tt * dpad + 4 * p);
          S[4 * p] *= e.x, S[4 * p + 1] *= e.y, S[4 * p + 2] *= e.z, S[4 * p + 3] *= e.w;
        }
      }
      float dk = 0.f, dq = 0.f, kq = 0.f;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        dk = fmaf(S[i], kk[i], dk);
        dq = fmaf(S[i], qq[i], dq);
        kq = fmaf(kk[i], qq[i], kq);
      }
      if constexpr (RULE != RULE_PLAIN) dk = row_sum16(dk);
      dq = row_sum16(dq);
      kq = row_sum16(kq);
      const float beta = g_l[4 * tt], g = RULE == RULE_DELTA_CHANNELS ? 1.f : g_l[4 * tt + 1];
      const float u = RULE == RULE_PLAIN ? v_l[tt * COLUMNS + c] : beta * (v_l[tt * COLUMNS + c] - g * dk);
#pragma unroll
      for (int i = 0; i < ROWS; ++i) S[i] = fmaf(kk[i], u, g * S[i]);
      if (s == 0 && mine) raw_out[(int64_t)(start + c0 + tt) * H * dv + h * dv + column] = fmaf(u, kq, g * dq);
    }
    // the other buffer is written next; this one again only after the barrier of the turn between
  }
  if (mine) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) st[(int64_t)i * dv * SPLIT + tid] = S[i];
  }
}

// The same for steps in which every request brings one token: nothing is staged, a thread reads its slices of the key
// and the query where the preparation left them, and as many workgroups as fit run side by side (no LDS holds them back).
template <int ROWS, int RULE>
__global__ __launch_bounds__(256) void delta_scan_single_kernel(const float* __restrict__ qkv, const float* __restrict__ gates,
                                                                const int* __restrict__ slot_ids, float* __restrict__ state,
                                                                int64_t state_stride, int G, int H, int d, int dv, float* __restrict__ raw_out,
                                                                const float* __restrict__ decays) {
  const int r = blockIdx.x, h = blockIdx.y, block = blockIdx.z, tid = threadIdx.x;
  const int channels = 2 * G * d + H * dv, hk = h / (H / G);
  const int c = tid / SPLIT, s = tid % SPLIT, column = block * COLUMNS + c;
  if (column >= dv) return;
  float* st = state + (int64_t)slot_ids[r] * state_stride + (int64_t)h * ROWS * dv * SPLIT + (int64_t)block * COLUMNS * SPLIT;
  const float* row = qkv + (int64_t)r * channels;
  float S[ROWS], kk[ROWS], qq[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) S[i] = st[(int64_t)i * dv * SPLIT + tid];
  if (d % 4 == 0 && channels % 4 == 0) {          // every piece of four values is 16 bytes aligned
#pragma unroll
    for (int p = 0; p < ROWS / 4; ++p) {
      const int at = s * ROWS + 4 * p;
      const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
      const float4 a = at < d ? *(const float4*)(row + hk * d + at) : zero, b = at < d ? *(const float4*)(row + G * d + hk * d + at) : zero;
      qq[4 * p] = a.x, qq[4 * p + 1] = a.y, qq[4 * p + 2] = a.z, qq[4 * p + 3] = a.w;
      kk[4 * p] = b.x, kk[4 * p + 1] = b.y, kk[4 * p + 2] = b.z, kk[4 * p + 3] = b.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int at = s * ROWS + i;
      qq[i] = at < d ? row[hk * d + at] : 0.f;
      kk[i] = at < d ? row[G * d + hk * d + at] : 0.f;
    }
  }
  const float v = row[2 * G * d + h * dv + column];
  const float beta = gates[(int64_t)r * 2 * H + h], g = RULE == RULE_DELTA_CHANNELS ? 1.f : gates[(int64_t)r * 2 * H + H + h];
  if constexpr (RULE == RULE_DELTA_CHANNELS) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int at = s * ROWS + i;
      if (at < d) S[i] *= decays[(int64_t)r * H * d + h * d + at];
    }
  }
  float dk = 0.f, dq = 0.f, kq = 0.f;
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    dk = fmaf(S[i], kk[i], dk);
    dq = fmaf(S[i], qq[i], dq);
    kq = fmaf(kk[i], qq[i], kq);
  }
  dk = row_sum16(dk);
  dq = row_sum16(dq);
  kq = row_sum16(kq);
  const float u = RULE == RULE_PLAIN ? v : beta * (v - g * dk);
#pragma unroll
  for (int i = 0; i < ROWS; ++i) st[(int64_t)i * dv * SPLIT + tid] = fmaf(kk[i], u, g * S[i]);
  if (s == 0) raw_out[(int64_t)r * H * dv + h * dv + column] = fmaf(u, kq, g * dq);
}

// The head's read-out divided by its root mean square over vdim, times the norm's weight, times silu(gate): a wave a
// (token, head).  gate_rank > 0: the gate is sigmoid instead, of the gate_rank values at gate_at carried to H * dv
// inputs by gate_up [gate_rank, H * dv]; gate_rank < 0: gate_up holds those H * dv inputs of every token already, [tokens, H * dv].
template <typename TP, typename TO>
__global__ __launch_bounds__(256) void delta_gate_kernel(const float* __restrict__ raw_out, const TP* __restrict__ proj, int ld,
                                                         int gate_at, const float* __restrict__ norm_w, float eps, int tokens, int H,
                                                         int dv, TO* __restrict__ out, int gate_rank, const float* __restrict__ gate_up) {
  const int64_t pair = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (pair >= (int64_t)tokens * H) return;
  const int64_t token = pair / H;
  const int h = (int)(pair % H);
  const float* o = raw_out + token * H * dv + (int64_t)h * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += WAVE) ss = fmaf(o[i], o[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += WAVE) {
    float factor;
    if (gate_rank < 0) {
      factor = 1.f / (1.f + expf(-gate_up[token * H * dv + (int64_t)h * dv + i]));
    } else if (gate_rank > 0) {
      float gate = 0.f;
      for (int r = 0; r < gate_rank; ++r) gate = fmaf(to_float(proj[token * ld + gate_at + r]), gate_up[(int64_t)r * H * dv + h * dv + i], gate);
      factor = 1.f / (1.f + expf(-gate));
    } else {
      factor = silu_f(to_float(proj[token * ld + gate_at + h * dv + i]));
    }
    out[token * H * dv + (int64_t)h * dv + i] = from_float<TO>(o[i] * inv * norm_w[i] * factor);
  }
}

// ------------------------------------------------------------------ selective state space recurrence
// Per head h (group h / (H / G)) with N = the state size: S <- exp(-exp(A_log_h) dt) S + dt B x^T (S [N, dv]),
// y = S^T C + D_h x, which is the scan above under RULE_PLAIN with k = B, q = C, v = dt x and g the decay.
//   ssm_prepare  per (token, unit), unit = a C group, a B group or an x head: the causal convolution with bias of the unit's
//                channels (taps before the step's first token from the request's state), silu; for x heads also the step
//                size dt = softplus(dt_in + dt_bias), the decay, v = dt x and the skip term D x;
//   ssm_gate     per (token, norm part): (read-out + skip) * silu(z), divided by the part's root mean square, times the weight.
// proj columns: z (H*dv) | x (H*dv) | B (G*N) | C (G*N) | dt (H); the convolution's channels are x | B | C in this order,
// and so are its kept inputs in the state row; the scan's scratch row is C | B | v.
template <typename TP>
__global__ void ssm_prepare_kernel(const TP* __restrict__ proj, int ld, const int* __restrict__ token_request,
                                   const int* __restrict__ cu, const int* __restrict__ slot_ids, float* __restrict__ state,
                                   int64_t state_stride, int64_t conv_offset, const float* __restrict__ conv_w,
                                   const float* __restrict__ conv_b, int taps, int G, int H, int N, int dv,
                                   const float* __restrict__ a_log, const float* __restrict__ dt_bias, const float* __restrict__ skip_w,
                                   float* __restrict__ qkv, float* __restrict__ gates, float* __restrict__ skip, int keep_inside) {
  const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  const int inner = H * dv, channels = inner + 2 * G * N;
  const int r = token_request[t], start = cu[r], at = t - start;
  float* kept = state + (int64_t)slot_ids[r] * state_stride + conv_offset;
  const bool is_x = unit >= 2 * G;
  // where the unit's channels lie among the convolution's (x | B | C) and in the scan's row (C | B | v)
  const int n = is_x ? dv : N;
  const int c_in = is_x ? (unit - 2 * G) * dv : unit < G ? inner + G * N + unit * N : inner + (unit - G) * N;
  const int c_out = is_x ? 2 * G * N + (unit - 2 * G) * dv : unit * N;
  float dt = 0.f, skip_factor = 0.f;
  if (is_x) {
    const int h = unit - 2 * G;
    const float a = to_float(proj[(int64_t)t * ld + inner + channels + h]) + dt_bias[h];
    dt = a > 20.f ? a : log1pf(expf(a));
    skip_factor = skip_w[h];
    if (lane == 0) {
      gates[(int64_t)t * 2 * H + h] = 1.f;
      gates[(int64_t)t * 2 * H + H + h] = expf(-expf(a_log[h]) * dt);
    }
  }
  for (int i = lane; i < n; i += WAVE) {
    const int c = c_in + i;
    float acc = conv_b ? conv_b[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int s = at - (taps - 1 - j);
      const float x = s >= 0 ? to_float(proj[(int64_t)(start + s) * ld + inner + c]) : kept[(int64_t)(taps - 1 + s) * channels + c];
      acc = fmaf(conv_w[(int64_t)c * taps + j], x, acc);
      if (keep_inside && j > 0) kept[(int64_t)(j - 1) * channels + c] = x;
    }
    const float y = silu_f(acc);
    if (is_x) {
      qkv[(int64_t)t * channels + c_out + i] = dt * y;
      skip[(int64_t)t * inner + (unit - 2 * G) * dv + i] = skip_factor * y;
    } else {
      qkv[(int64_t)t * channels + c_out + i] = y;
    }
  }
}

template <typename TP, typename TO>
__global__ __launch_bounds__(256) void ssm_gate_kernel(const float* __restrict__ raw_out, const float* __restrict__ skip,
                                                       const TP* __restrict__ proj, int ld, const float* __restrict__ norm_w, float eps,
                                                       int tokens, int parts, int part_size, TO* __restrict__ out) {
  const int64_t pair = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (pair >= (int64_t)tokens * parts) return;
  const int64_t token = pair / parts;
  const int64_t first = (pair % parts) * part_size, inner = (int64_t)parts * part_size;
  float ss = 0.f;
  constexpr int HELD = 16;                 // parts of up to 1,024 values stay in registers between the sum and the norm
  if (part_size <= HELD * WAVE) {
    float r[HELD], k[HELD], z[HELD];
#pragma unroll
    for (int n = 0; n < HELD; ++n) {       // every load is on its way before the first exponential
      const int i = lane + n * WAVE;
      if (i < part_size) {
        r[n] = raw_out[token * inner + first + i];
        k[n] = skip[token * inner + first + i];
        z[n] = to_float(proj[token * ld + first + i]);
      }
    }
#pragma unroll
    for (int n = 0; n < HELD; ++n) {
      if (lane + n * WAVE < part_size) {
        r[n] = (r[n] + k[n]) * silu_f(z[n]);
        ss = fmaf(r[n], r[n], ss);
      }
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)part_size + eps);
#pragma unroll
    for (int n = 0; n < HELD; ++n) {
      const int i = lane + n * WAVE;
      if (i < part_size) out[token * inner + first + i] = from_float<TO>(r[n] * inv * norm_w[first + i]);
    }
    return;
  }
  for (int i = lane; i < part_size; i += WAVE) {
    const float y = (raw_out[token * inner + first + i] + skip[token * inner + first + i]) * silu_f(to_float(proj[token * ld + first + i]));
    ss = fmaf(y, y, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)part_size + eps);
  for (int i = lane; i < part_size; i += WAVE) {
    const float y = (raw_out[token * inner + first + i] + skip[token * inner + first + i]) * silu_f(to_float(proj[token * ld + first + i]));
    out[token * inner + first + i] = from_float<TO>(y * inv * norm_w[first + i]);
  }
}

template <int RULE>
void launch_scan(int rows, bool single, dim3 grid, hipStream_t s, const float* qkv, const float* gates, const int* cu, const int* slot_ids,
                 float* state, int64_t state_stride, int G, int H, int d, int dv, float* raw, const float* decays) {
  const int chunk = rows == 16 ? 8 : 16, vectors = RULE == RULE_DELTA_CHANNELS ? 3 : 2;
  const size_t lds = (size_t)2 * chunk * (vectors * rows * SPLIT + COLUMNS + 4) * sizeof(float);
  if (single) {        // one token each: token r is request r's
    if (rows == 4) delta_scan_single_kernel<4, RULE><<<grid, 256, 0, s>>>(qkv, gates, slot_ids, state, state_stride, G, H, d, dv, raw, decays);
    else if (rows == 8) delta_scan_single_kernel<8, RULE><<<grid, 256, 0, s>>>(qkv, gates, slot_ids, state, state_stride, G, H, d, dv, raw, decays);
    else delta_scan_single_kernel<16, RULE><<<grid, 256, 0, s>>>(qkv, gates, slot_ids, state, state_stride, G, H, d, dv, raw, decays);
  } else if (rows == 4) delta_scan_kernel<4, 16, RULE><<<grid, 256, lds, s>>>(qkv, gates, cu, slot_ids, state, state_stride, G, H, d, dv, raw, decays);
  else if (rows == 8) delta_scan_kernel<8, 16, RULE><<<grid, 256, lds, s>>>(qkv, gates, cu, slot_ids, state, state_stride, G, H, d, dv, raw, decays);
  else delta_scan_kernel<16, 8, RULE><<<grid, 256, lds, s>>>(qkv, gates, cu, slot_ids, state, state_stride, G, H, d, dv, raw, decays);
}

}  // namespace

// Rows of a head's matrix that one lane holds: the key size over the 16 lanes of a column, to the next of 4, 8, 16.
LRS_API int lrs_delta_state_rows(int d) { return d <= 64 ? 4 : d <= 128 ? 8 : 16; }

namespace {

// The gated delta rule's kernels for one step.  gate_at, beta_at, decay_at: columns of proj.  decay_rank > 0: a decay per
// head and key channel from decay_rank values (decay_up [decay_rank, H*d], dt_bias [H*d], decays [tokens, H*d] scratch);
// gate_rank > 0: a sigmoid gate from gate_rank values (gate_up [gate_rank, H*dv]); 0: silu of H*dv columns.  A rank below 0:
// the inputs were made by a product of the caller's: decays [tokens, H*d] holds the decays' inputs, gate_up [tokens, H*dv] the gate's.
int delta_launch(void* out, int out_dtype, const void* proj, int proj_dtype, int ld, int tokens, int requests,
                 const int* token_request, const int* cu, const int* slot_ids, float* state, int64_t state_stride,
                 const float* conv_w, int taps, int G, int H, int d, int dv, const float* a_log, const float* dt_bias,
                 const float* norm_w, float eps, float* qkv, float* gates, float* raw, int gate_at, int beta_at, int decay_at,
                 int decay_rank, const float* decay_up, float* decays, int gate_rank, const float* gate_up, void* stream) {
  LRS_REQUIRE(tokens > 0 && requests > 0 && requests <= tokens, "delta_rule: bad sizes tokens=%d requests=%d", tokens, requests);
  LRS_REQUIRE(G > 0 && H > 0 && H % G == 0 && d > 0 && dv > 0 && taps >= 1, "delta_rule: bad sizes G=%d H=%d d=%d dv=%d taps=%d", G, H, d, dv, taps);
  LRS_REQUIRE(d <= 256, "delta_rule: takes keys of up to 256 values, got %d", d);
  const int rows = lrs_delta_state_rows(d), channels = 2 * G * d + H * dv;
  const int gate_end = gate_rank < 0 ? 0 : gate_at + (gate_rank > 0 ? gate_rank : H * dv);
  const int decay_end = decay_rank < 0 ? 0 : decay_at + (decay_rank > 0 ? decay_rank : H);
  const int last = gate_end > decay_end ? gate_end : decay_end;
  LRS_REQUIRE(ld >= channels && ld >= last && ld >= beta_at + H, "delta_rule: projection rows of %d hold fewer than the columns needed", ld);
  const int64_t conv_offset = (int64_t)H * rows * SPLIT * dv;
  LRS_REQUIRE(state_stride >= conv_offset + (int64_t)(taps - 1) * channels, "delta_rule: a state row of %lld floats is too short", (long long)state_stride);
  LRS_REQUIRE(eps > 0.f, "delta_rule: eps must be positive");
  LRS_REQUIRE(((uintptr_t)qkv % 16) == 0 && ((uintptr_t)decays % 16) == 0, "delta_rule: the scratch rows must be 16 bytes aligned");
  LRS_REQUIRE(decay_rank == 0 || ((decay_up || decay_rank < 0) && decays), "delta_rule: decays per channel need their matrix and scratch rows");
  LRS_REQUIRE(gate_rank == 0 || gate_up, "delta_rule: a gate of low rank needs its matrix or its inputs");
  hipStream_t s = (hipStream_t)stream;
  dim3 pgrid(tokens, 2 * G + H), kgrid(requests, (channels + 255) / 256), sgrid(requests, H, (dv + COLUMNS - 1) / COLUMNS);
  const int64_t pairs = (int64_t)tokens * H;
  const bool single = tokens == requests;
#define ALL(TP, TO)                                                                                                           \
  do {                                                                                                                        \
    delta_prepare_kernel<TP><<<pgrid, WAVE, 0, s>>>((const TP*)proj, ld, token_request, cu, slot_ids, state, state_stride,    \
                                                    conv_offset, conv_w, taps, G, H, d, dv, a_log, dt_bias, qkv, gates,       \
                                                    single, beta_at, decay_at, decay_rank, decay_up, decays);                 \
    if (taps > 1 && !single)                                                                                                  \
      delta_conv_keep_kernel<TP><<<kgrid, 256, 0, s>>>((const TP*)proj, ld, cu, slot_ids, state, state_stride, conv_offset,  \
                                                       taps, channels, 0);                                                    \
    if (decay_rank != 0) launch_scan<RULE_DELTA_CHANNELS>(rows, single, sgrid, s, qkv, gates, cu, slot_ids, state, state_stride, G, H, d, dv, raw, decays); \
    else launch_scan<RULE_DELTA>(rows, single, sgrid, s, qkv, gates, cu, slot_ids, state, state_stride, G, H, d, dv, raw, nullptr);                    \
    delta_gate_kernel<TP, TO><<<(unsigned)((pairs + 3) / 4), 256, 0, s>>>(raw, (const TP*)proj, ld, gate_at, norm_w, eps, tokens, H, dv, (TO*)out, \
                                                                          gate_rank, gate_up);                                \
  } while (0)
  if (proj_dtype == LRS_F32 && out_dtype == LRS_F32) ALL(float, float);
  else if (proj_dtype == LRS_F32 && out_dtype == LRS_BF16) ALL(float, bf16);
  else if (proj_dtype == LRS_BF16 && out_dtype == LRS_BF16) ALL(bf16, bf16);
  else return lrs_fail("delta_rule: projections in dtype %d with outputs in dtype %d are not served", proj_dtype, out_dtype);
#undef ALL
  return lrs_check_launch("delta_rule");
}

}  // namespace

// proj [tokens, ld]: columns q (G*d) | k (G*d) | v (H*dv) | output gate (H*dv) | step size (H) | decay input (H).
// qkv [tokens, 2*G*d + H*dv], gates [tokens, 2*H] and raw [tokens, H*dv] are float32 scratch; out [tokens, H*dv] in out_dtype.
LRS_API int lrs_delta_rule(void* out, int out_dtype, const void* proj, int proj_dtype, int ld, int tokens, int requests,
                           const int* token_request, const int* cu, const int* slot_ids, float* state, int64_t state_stride,
                           const float* conv_w, int taps, int G, int H, int d, int dv, const float* a_log,
                           const float* dt_bias, const float* norm_w, float eps, float* qkv, float* gates, float* raw, void* stream) {
  const int channels = 2 * G * d + H * dv;
  return delta_launch(out, out_dtype, proj, proj_dtype, ld, tokens, requests, token_request, cu, slot_ids, state, state_stride, conv_w, taps,
                      G, H, d, dv, a_log, dt_bias, norm_w, eps, qkv, gates, raw, channels, channels + H * dv, channels + H * dv + H, 0, nullptr,
                      nullptr, 0, nullptr, stream);
}

// The rule with a decay per head and key channel and a sigmoid gate, both from inputs of low rank.  proj columns:
// q (G*d) | k (G*d) | v (H*dv) | step size (H) | decay input (decay_rank) | gate input (gate_rank); decay_up [decay_rank, H*d],
// dt_bias [H*d], gate_up [gate_rank, H*dv], decays [tokens, H*d] float32 scratch.  Both ranks -1: the caller has applied the
// second matrices itself; proj ends with the step sizes, decays holds W_a2 (W_a1 x) and gate_up W_g2 (W_g1 x), [tokens, H*d] and [tokens, H*dv].
LRS_API int lrs_delta_rule_channels(void* out, int out_dtype, const void* proj, int proj_dtype, int ld, int tokens, int requests,
                                    const int* token_request, const int* cu, const int* slot_ids, float* state, int64_t state_stride,
                                    const float* conv_w, int taps, int G, int H, int d, int dv, const float* a_log,
                                    const float* dt_bias, const float* norm_w, float eps, float* qkv, float* gates, float* raw,
                                    int decay_rank, const float* decay_up, float* decays, int gate_rank, const float* gate_up, void* stream) {
  LRS_REQUIRE((decay_rank > 0 && gate_rank > 0) || (decay_rank == -1 && gate_rank == -1),
              "delta_rule_channels: ranks must both be positive, or both -1 for inputs that are given, got %d and %d", decay_rank, gate_rank);
  const int channels = 2 * G * d + H * dv;
  return delta_launch(out, out_dtype, proj, proj_dtype, ld, tokens, requests, token_request, cu, slot_ids, state, state_stride, conv_w, taps,
                      G, H, d, dv, a_log, dt_bias, norm_w, eps, qkv, gates, raw, channels + H + decay_rank, channels, channels + H, decay_rank,
                      decay_up, decays, gate_rank, gate_up, stream);
}

// One step of the state space recurrence for a ragged batch.  proj [tokens, ld]: z (H*dv) | x (H*dv) | B (G*N) | C (G*N) | dt (H).
// conv_w [H*dv + 2*G*N, taps], conv_b the same many or null; state rows as the delta rule's with d = N: every head's S, then
// the convolution's last taps - 1 inputs.  qkv [tokens, 2*G*N + H*dv], gates [tokens, 2*H], raw and skip [tokens, H*dv]
// float32 scratch; the output is normalised in `parts` equal parts of H*dv; out [tokens, H*dv] in out_dtype.
LRS_API int lrs_ssm(void* out, int out_dtype, const void* proj, int proj_dtype, int ld, int tokens, int requests,
                    const int* token_request, const int* cu, const int* slot_ids, float* state, int64_t state_stride,
                    const float* conv_w, const float* conv_b, int taps, int G, int H, int N, int dv, const float* a_log,
                    const float* dt_bias, const float* skip_w, const float* norm_w, int parts, float eps, float* qkv, float* gates,
                    float* raw, float* skip, void* stream) {
  LRS_REQUIRE(tokens > 0 && requests > 0 && requests <= tokens, "ssm: bad sizes tokens=%d requests=%d", tokens, requests);
  LRS_REQUIRE(G > 0 && H > 0 && H % G == 0 && N > 0 && dv > 0 && taps >= 1, "ssm: bad sizes G=%d H=%d N=%d dv=%d taps=%d", G, H, N, dv, taps);
  LRS_REQUIRE(N <= 256, "ssm: takes states of up to 256 values a column, got %d", N);
  LRS_REQUIRE(parts > 0 && (H * dv) % parts == 0, "ssm: %d values do not divide into %d parts", H * dv, parts);
  const int rows = lrs_delta_state_rows(N), inner = H * dv, channels = inner + 2 * G * N;
  LRS_REQUIRE(ld >= inner + channels + H, "ssm: projection rows of %d hold fewer than the %d columns needed", ld, inner + channels + H);
  const int64_t conv_offset = (int64_t)H * rows * SPLIT * dv;
  LRS_REQUIRE(state_stride >= conv_offset + (int64_t)(taps - 1) * channels, "ssm: a state row of %lld floats is too short", (long long)state_stride);
  LRS_REQUIRE(eps > 0.f, "ssm: eps must be positive");
  LRS_REQUIRE(((uintptr_t)qkv % 16) == 0, "ssm: the scratch rows must be 16 bytes aligned");
  hipStream_t s = (hipStream_t)stream;
  dim3 pgrid(tokens, 2 * G + H), kgrid(requests, (channels + 255) / 256), sgrid(requests, H, (dv + COLUMNS - 1) / COLUMNS);
  const int64_t pairs = (int64_t)tokens * parts;
  const bool single = tokens == requests;
#define ALL(TP, TO)                                                                                                           \
  do {                                                                                                                        \
    ssm_prepare_kernel<TP><<<pgrid, WAVE, 0, s>>>((const TP*)proj, ld, token_request, cu, slot_ids, state, state_stride,      \
                                                  conv_offset, conv_w, conv_b, taps, G, H, N, dv, a_log, dt_bias, skip_w, qkv, \
                                                  gates, skip, single);                                                       \
    if (taps > 1 && !single)                                                                                                  \
      delta_conv_keep_kernel<TP><<<kgrid, 256, 0, s>>>((const TP*)proj, ld, cu, slot_ids, state, state_stride, conv_offset,  \
                                                       taps, channels, inner);                                                \
    launch_scan<RULE_PLAIN>(rows, single, sgrid, s, qkv, gates, cu, slot_ids, state, state_stride, G, H, N, dv, raw, nullptr);   \
    ssm_gate_kernel<TP, TO><<<(unsigned)((pairs + 3) / 4), 256, 0, s>>>(raw, skip, (const TP*)proj, ld, norm_w, eps, tokens,  \
                                                                        parts, inner / parts, (TO*)out);                      \
  } while (0)
  if (proj_dtype == LRS_F32 && out_dtype == LRS_F32) ALL(float, float);
  else if (proj_dtype == LRS_F32 && out_dtype == LRS_BF16) ALL(float, bf16);
  else if (proj_dtype == LRS_BF16 && out_dtype == LRS_BF16) ALL(bf16, bf16);
  else return lrs_fail("ssm: projections in dtype %d with outputs in dtype %d are not served", proj_dtype, out_dtype);
#undef ALL
  return lrs_check_launch("ssm");
}

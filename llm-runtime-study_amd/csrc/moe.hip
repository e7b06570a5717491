// Routed experts: every token runs `top` of `experts` small feed-forward layers and adds their outputs up,
// weighted by a softmax over the chosen router logits.
//
//   moe_route     per token: the `top` largest of (router logits + bias), lowest index first among equals, and
//                 the softmax over those alone (float32);
//   moe_align     one workgroup: sorts the step's (token, choice) pairs by expert into runs padded to whole row
//                 tiles, so that every tile of the two products below belongs to one expert.  The number of tiles
//                 a launch is sized for follows from the step's shape alone (pairs / tile + experts at most), so a
//                 step can be recorded or captured; tiles beyond the ones in use leave at once;
//   moe_experts   the grouped product: rows gathered through the sorted list, an expert's matrix per tile, and
//                 optionally the activation (the square of relu) on the way out.  A float32 / any-shape form on
//                 the vector units, whose sums over K run in one order whatever else is in the step, and a
//                 bfloat16 form on the matrix cores;
//   moe_combine   per token: the weighted sum of its experts' rows in the order of its choices, and, when a norm
//                 weight is given, the RMS norm of that sum added into the residual stream.
#include "common.h"

LRS_API int lrs_compute_units();

namespace {

constexpr int ROUTE_MAX_PER_LANE = 8;     // experts up to 64 * 8

// One token by one wave.
__device__ __forceinline__ void route_token(const float* __restrict__ logits, int ld, const float* __restrict__ bias,
                                            int* ids, float* __restrict__ weights, int t, int experts, int top, int lane) {
  float v[ROUTE_MAX_PER_LANE];
#pragma unroll
  for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) {
    const int e = lane + WAVE * c;
    v[c] = e < experts ? logits[(int64_t)t * ld + e] + (bias ? bias[e] : 0.f) : -INFINITY;
  }
  float first = 0.f, mine = 0.f, total = 0.f;
  int chosen = 0;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
#pragma unroll
    for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) best = fmaxf(best, v[c]);
    best = wave_max(best);
    int where = 1 << 30;
#pragma unroll
    for (int c = ROUTE_MAX_PER_LANE - 1; c >= 0; --c)
      if (v[c] == best) where = lane + WAVE * c;
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) where = min(where, __shfl_xor(where, off, WAVE));
    if (where >= experts) where = k;    // logits that are not numbers: any expert, never an index outside the table
#pragma unroll
    for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c)
      if (lane + WAVE * c == where) v[c] = -INFINITY;
    if (k == 0) first = best;
    const float w = expf(best - first);
    total += w;
    if (lane == k % WAVE && k / WAVE == 0) {
      mine = w;
      chosen = where;
    }
    if (k >= WAVE) {                    // more choices than lanes: written as they come, scaled below
      if (lane == 0) {
        ids[(int64_t)t * top + k] = where;
        weights[(int64_t)t * top + k] = w;
      }
    }
  }
  if (lane < top && lane < WAVE) {
    ids[(int64_t)t * top + lane] = chosen;
    weights[(int64_t)t * top + lane] = mine / total;
  }
  if (top > WAVE && lane == 0)
    for (int k = WAVE; k < top; ++k) weights[(int64_t)t * top + k] /= total;
}

// How a token's experts are chosen and weighted.
//   ROUTE_SOFTMAX_CHOSEN  the largest (logit + bias); weights: the softmax over the chosen (logit + bias) alone
//   ROUTE_SIGMOID         scores s = sigmoid(logit); the largest (s + bias) are chosen, the bias taking part in the
//                         choice only; weights: the chosen s divided by their sum (+ 1e-20), times `scale`.  With
//                         groups > 0 the experts form that many equal groups of neighbours, a group's score is the sum of
//                         its two largest (s + bias), and only experts of the `keep` best groups can be chosen.
//   ROUTE_SIGMOID_SCORES  chosen as under ROUTE_SIGMOID; weights: the chosen s themselves, times `scale` (not divided by their sum)
enum { ROUTE_SOFTMAX_CHOSEN = 0, ROUTE_SIGMOID = 1, ROUTE_SIGMOID_SCORES = 2 };
struct RouteRule {
  int kind, groups, keep;
  float scale;
};

// The lowest index among the lanes' elements that equal `best` (1 << 30 if none).
__device__ __forceinline__ int route_where(const float (&v)[ROUTE_MAX_PER_LANE], float best, int lane) {
  int where = 1 << 30;
#pragma unroll
  for (int c = ROUTE_MAX_PER_LANE - 1; c >= 0; --c)
    if (v[c] == best) where = lane + WAVE * c;
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) where = min(where, __shfl_xor(where, off, WAVE));
  return where;
}
__device__ __forceinline__ float route_max(const float (&v)[ROUTE_MAX_PER_LANE]) {
  float best = -INFINITY;
#pragma unroll
  for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) best = fmaxf(best, v[c]);
  return wave_max(best);
}

// One token by one wave, ROUTE_SIGMOID.
__device__ __forceinline__ void route_token_sigmoid(const float* __restrict__ logits, int ld, const float* __restrict__ bias,
                                                    int* ids, float* __restrict__ weights, int t, int experts, int top, int lane,
                                                    const RouteRule rule) {
  float s[ROUTE_MAX_PER_LANE], v[ROUTE_MAX_PER_LANE];
#pragma unroll
  for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) {
    const int e = lane + WAVE * c;
    const float z = e < experts ? logits[(int64_t)t * ld + e] : 0.f;
    s[c] = e < experts ? 1.0f / (1.0f + expf(-z)) : 0.f;
    // without a bias and without groups the order of the scores is the order of the logits, which does not run out of
    // digits where the sigmoid nears one (logits of 17 and of 30 both give 1.0f)
    v[c] = e < experts ? (bias || rule.groups > 0 ? s[c] + (bias ? bias[e] : 0.f) : z) : -INFINITY;
  }
  if (rule.groups > 0 && rule.keep < rule.groups) {
    const int per = experts / rule.groups;
    float score[ROUTE_MAX_PER_LANE];       // of group lane + WAVE * c
#pragma unroll
    for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) score[c] = -INFINITY;
    for (int g = 0; g < rule.groups; ++g) {
      float mine[ROUTE_MAX_PER_LANE];
#pragma unroll
      for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) mine[c] = (lane + WAVE * c) / per == g ? v[c] : -INFINITY;
      const float first = route_max(mine);
      float sum = first;
      if (per > 1) {
        const int where = route_where(mine, first, lane);
#pragma unroll
        for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c)
          if (lane + WAVE * c == where) mine[c] = -INFINITY;
        sum = first + route_max(mine);
      }
#pragma unroll
      for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c)
        if (lane + WAVE * c == g) score[c] = sum;
    }
    bool kept[ROUTE_MAX_PER_LANE];
#pragma unroll
    for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) kept[c] = false;
    for (int k = 0; k < rule.keep; ++k) {
      const float best = route_max(score);
      int where = route_where(score, best, lane);
      if (where >= rule.groups) where = k;   // scores that are not numbers: any group
#pragma unroll
      for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c) {
        if (lane + WAVE * c == where) score[c] = -INFINITY;
        if ((lane + WAVE * c) / per == where) kept[c] = true;
      }
    }
#pragma unroll
    for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c)
      if (!kept[c]) v[c] = -INFINITY;
  }
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    const float best = route_max(v);
    int where = route_where(v, best, lane);
    if (where >= experts) where = k;    // scores that are not numbers: any expert, never an index outside the table
    float own = 0.f;
#pragma unroll
    for (int c = 0; c < ROUTE_MAX_PER_LANE; ++c)
      if (lane + WAVE * c == where) {
        v[c] = -INFINITY;
        own = s[c];
      }
    const float w = __shfl(own, where % WAVE, WAVE);
    total += w;
    if (lane == 0) {
      ids[(int64_t)t * top + k] = where;
      weights[(int64_t)t * top + k] = w;
    }
  }
  // the same lane wrote them: it reads its own stores
  if (lane == 0 && rule.kind == ROUTE_SIGMOID_SCORES) {
    if (rule.scale != 1.f)
      for (int k = 0; k < top; ++k) weights[(int64_t)t * top + k] *= rule.scale;
  } else if (lane == 0) {
    for (int k = 0; k < top; ++k) weights[(int64_t)t * top + k] = weights[(int64_t)t * top + k] / (total + 1e-20f) * rule.scale;
  }
}

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ bias,
                                                        int* __restrict__ ids, float* __restrict__ weights, int tokens,
                                                        int experts, int top, const RouteRule rule) {
  const int t = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (t >= tokens) return;
  if (rule.kind != ROUTE_SOFTMAX_CHOSEN) route_token_sigmoid(logits, ld, bias, ids, weights, t, experts, top, threadIdx.x % WAVE, rule);
  else route_token(logits, ld, bias, ids, weights, t, experts, top, threadIdx.x % WAVE);
}

// sorted [capacity]: the pair (token * top + choice) at each row of the sorted order, -1 for the rows that pad an
// expert's run to whole tiles; place [pairs]: the row of each pair; tile_expert [max_tiles]: the expert of each
// tile of `tile` rows, -1 for tiles not in use.
__device__ __forceinline__ void align_pairs(const int* ids, int pairs, int experts, int tile, int* __restrict__ sorted,
                                            int capacity, int* __restrict__ place, int* __restrict__ tile_expert, int max_tiles,
                                            int* shared) {
  int* count = shared;                  // [experts]
  int* first = count + experts;         // [experts + 1]: first row of each expert's run
  int* cursor = first + experts + 1;    // [experts]
  const int tid = threadIdx.x;
  for (int e = tid; e < experts; e += blockDim.x) count[e] = cursor[e] = 0;
  for (int i = tid; i < capacity; i += blockDim.x) sorted[i] = -1;
  for (int i = tid; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  for (int i = tid; i < pairs; i += blockDim.x) atomicAdd(&count[min((unsigned)ids[i], (unsigned)experts - 1)], 1);
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = at;
      at += (count[e] + tile - 1) / tile * tile;
    }
    first[experts] = at;
  }
  __syncthreads();
  for (int e = tid; e < experts; e += blockDim.x)
    for (int i = first[e] / tile; i < first[e + 1] / tile; ++i) tile_expert[i] = e;
  for (int i = tid; i < pairs; i += blockDim.x) {
    const int e = min((unsigned)ids[i], (unsigned)experts - 1), row = first[e] + atomicAdd(&cursor[e], 1);
    sorted[row] = i;
    place[i] = row;
  }
}

__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, int pairs, int experts, int tile,
                                                         int* __restrict__ sorted, int capacity, int* __restrict__ place,
                                                         int* __restrict__ tile_expert, int max_tiles) {
  extern __shared__ int shared[];
  align_pairs(ids, pairs, experts, tile, sorted, capacity, place, tile_expert, max_tiles, shared);
}

// Both in one workgroup, for steps of few tokens (single tokens above all), where a launch costs more than either does.
__global__ __launch_bounds__(1024) void moe_route_align_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ bias,
                                                               int* ids, float* __restrict__ weights, int tokens, int experts,
                                                               int top, int tile, int* __restrict__ sorted, int capacity,
                                                               int* __restrict__ place, int* __restrict__ tile_expert, int max_tiles,
                                                               const RouteRule rule) {
  extern __shared__ int shared[];
  for (int t = threadIdx.x / WAVE; t < tokens; t += blockDim.x / WAVE) {
    if (rule.kind != ROUTE_SOFTMAX_CHOSEN) route_token_sigmoid(logits, ld, bias, ids, weights, t, experts, top, threadIdx.x % WAVE, rule);
    else route_token(logits, ld, bias, ids, weights, t, experts, top, threadIdx.x % WAVE);
  }
  __syncthreads();          // the choices are in memory for every thread of the workgroup
  align_pairs(ids, tokens * top, experts, tile, sorted, capacity, place, tile_expert, max_tiles, shared);
}

// ACT_SILU_PAIRS: the matrix holds, for every feature j, a gate row 2j and an up row 2j + 1; the output has half as many columns,
// out[:, j] = silu(gate_j) * up_j.  Every kernel below leaves a lane four neighbouring columns, so a lane holds whole pairs.
// ACT_CLAMPED_PAIRS: the same rows; out[:, j] = g * sigmoid(alpha * g) * (u + 1) with g = min(w * gate_j, limit) and
// u = clamp(w * up_j, -limit, limit), w the weight of the row's (token, choice) pair where a list of them is given: the
// expert then runs on w times its input, the products being linear in it.
enum { ACT_NONE = 0, ACT_RELU_SQUARED = 1, ACT_SILU_PAIRS = 2, ACT_CLAMPED_PAIRS = 3 };
struct PairAct {
  const float* pair_weights;   // [pairs], or null for 1
  float alpha, limit;
};
__device__ __forceinline__ float silu_times(float gate, float up) { return gate / (1.0f + expf(-gate)) * up; }
__device__ __forceinline__ float clamped_times(float gate, float up, float w, const PairAct& pa) {
  const float g = fminf(w * gate, pa.limit), u = fminf(fmaxf(w * up, -pa.limit), pa.limit);
  return g / (1.0f + expf(-pa.alpha * g)) * (u + 1.0f);
}
__device__ __forceinline__ float pair_times(int act, float gate, float up, float w, const PairAct& pa) {
  return act == ACT_SILU_PAIRS ? silu_times(gate, up) : clamped_times(gate, up, w, pa);
}
__device__ __forceinline__ float weight_of_row(const PairAct& pa, const int* __restrict__ sorted, int row) {
  return pa.pair_weights ? pa.pair_weights[sorted[row]] : 1.f;
}

// Any dtype, any shape: a 32 x 64 tile of outputs per workgroup of 256 threads, a thread 2 x 4 of them, each the
// sum of its products in the order of k.
template <typename T, typename TO>
__global__ __launch_bounds__(256) void moe_experts_kernel(TO* __restrict__ out, int ldc, const T* __restrict__ a, int lda,
                                                          const T* __restrict__ w, int n, int k, const int* __restrict__ sorted,
                                                          const int* __restrict__ tile_expert, int top, int gather, int act, int sub,
                                                          const PairAct pa) {
  constexpr int TM = 32, TN = 64, TK = 16;
  const int expert = tile_expert[blockIdx.x / sub];       // sub: runs of 32 rows in a tile of the sorted list
  if (expert < 0) return;
  __shared__ float a_s[TK][TM + 1];
  __shared__ float b_s[TK][TN + 1];
  __shared__ int row_of[TM];
  const int tid = threadIdx.x, row0 = blockIdx.x * TM, col0 = blockIdx.y * TN;
  if (tid < TM) {
    const int pair = sorted[row0 + tid];
    row_of[tid] = pair < 0 ? -1 : (gather ? pair / top : row0 + tid);
  }
  __syncthreads();
  const T* we = w + (int64_t)expert * n * k;
  const int ty = tid / 16, tx = tid % 16;
  float acc[2][4] = {};
  for (int k0 = 0; k0 < k; k0 += TK) {
    for (int e = tid; e < TM * TK; e += 256) {
      const int m = e / TK, kk = e % TK, src = row_of[m];
      a_s[kk][m] = (src >= 0 && k0 + kk < k) ? to_float(a[(int64_t)src * lda + k0 + kk]) : 0.f;
    }
    for (int e = tid; e < TN * TK; e += 256) {
      const int c = e / TK, kk = e % TK;
      b_s[kk][c] = (col0 + c < n && k0 + kk < k) ? to_float(we[(int64_t)(col0 + c) * k + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float av[2], bv[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) av[i] = a_s[kk][ty * 2 + i];
#pragma unroll
      for (int i = 0; i < 4; ++i) bv[i] = b_s[kk][tx * 4 + i];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) acc[i][jj] = fmaf(av[i], bv[jj], acc[i][jj]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = ty * 2 + i;
    if (row_of[m] < 0) continue;
    const float pw = act == ACT_CLAMPED_PAIRS ? weight_of_row(pa, sorted, row0 + m) : 1.f;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int c = col0 + tx * 4 + jj;
      if (c >= n) continue;
      float v = acc[i][jj];
      if (act >= ACT_SILU_PAIRS) {
        if (jj % 2 == 0) out[(int64_t)(row0 + m) * ldc + c / 2] = from_float<TO>(pair_times(act, v, acc[i][jj + 1], pw, pa));
        continue;
      }
      if (act == ACT_RELU_SQUARED) v = v > 0.f ? v * v : 0.f;
      out[(int64_t)(row0 + m) * ldc + c] = from_float<TO>(v);
    }
  }
}

// bfloat16 on the matrix cores: a workgroup of four waves makes 32 rows x 128 columns of one expert, a wave 32 x 32
// as two by two products of 16 x 16 x 32; K in slices of 64 through LDS, rows padded by 8 values so that the
// 16-byte fragment reads of a wave fall on different banks; the next slice is read into registers while one is
// multiplied.
constexpr int GM = 32, GN = 128, GK = 64, GPAD = 8;

// NT: columns per workgroup, 128 (a wave 32 of them) or 64 (a wave 16: twice the workgroups, for steps of so few rows
// that 128 columns each would leave compute units without any).
template <typename TO, int NT>
__global__ __launch_bounds__(256) void moe_experts_bf16_kernel(TO* __restrict__ out, int ldc, const bf16* __restrict__ a, int lda,
                                                               const bf16* __restrict__ w, int n, int k, const int* __restrict__ sorted,
                                                               const int* __restrict__ tile_expert, int top, int gather, int act, const PairAct pa) {
  const int expert = tile_expert[blockIdx.x];
  if (expert < 0) return;
  __shared__ __attribute__((aligned(16))) bf16 a_s[GM][GK + GPAD];
  __shared__ __attribute__((aligned(16))) bf16 b_s[NT][GK + GPAD];
  __shared__ int row_of[GM];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  constexpr int WN = NT / 64;                 // products of 16 columns a wave makes side by side
  const int row0 = blockIdx.x * GM, col0 = blockIdx.y * NT;
  if (tid < GM) {
    const int pair = sorted[row0 + tid];
    row_of[tid] = pair < 0 ? -1 : (gather ? pair / top : row0 + tid);
  }
  __syncthreads();
  const bf16* we = w + (int64_t)expert * n * k;
  // a thread brings 8 values (16 bytes) of one row of the slice: 32 x 64 of the rows is one piece each, 128 x 64 of the
  // weights four
  const int a_row = tid / 8, a_col = (tid % 8) * 8;
  const int a_src = row_of[a_row];
  const bf16* a_ptr = a_src >= 0 ? a + (int64_t)a_src * lda + a_col : nullptr;
  bf16x8 a_reg, b_reg[NT / 32];
  const bf16x8 zero = {};
  auto fetch = [&](int k0) {
    a_reg = a_ptr ? *(const bf16x8*)(a_ptr + k0) : zero;
#pragma unroll
    for (int p = 0; p < NT / 32; ++p) {
      const int r = p * 32 + a_row;
      b_reg[p] = col0 + r < n ? *(const bf16x8*)(we + (int64_t)(col0 + r) * k + k0 + a_col) : zero;
    }
  };
  floatx4 acc[2][WN] = {};
  fetch(0);
  const int frag_row = lane % 16, frag_k = (lane / 16) * 8;
  for (int k0 = 0; k0 < k; k0 += GK) {
    *(bf16x8*)&a_s[a_row][a_col] = a_reg;
#pragma unroll
    for (int p = 0; p < NT / 32; ++p) *(bf16x8*)&b_s[p * 32 + a_row][a_col] = b_reg[p];
    __syncthreads();
    if (k0 + GK < k) fetch(k0 + GK);
#pragma unroll
    for (int kk = 0; kk < GK; kk += 32) {
      bf16x8 af[2], bfr[WN];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = *(const bf16x8*)&a_s[i * 16 + frag_row][kk + frag_k];
#pragma unroll
      for (int i = 0; i < WN; ++i) bfr[i] = *(const bf16x8*)&b_s[wave * 16 * WN + i * 16 + frag_row][kk + frag_k];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int jj = 0; jj < WN; ++jj)
          // the weights as the first operand: a lane then holds four consecutive columns of one output row
          acc[i][jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[jj], af[i], acc[i][jj], 0, 0, 0);
    }
    __syncthreads();
  }
  // lane l of a product holds output row (l % 16) and columns (l / 16) * 4 .. + 4 of its 16 x 16
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = i * 16 + lane % 16;
    if (row_of[m] < 0) continue;
    const float pw = act == ACT_CLAMPED_PAIRS ? weight_of_row(pa, sorted, row0 + m) : 1.f;
#pragma unroll
    for (int jj = 0; jj < WN; ++jj) {
      const int c = col0 + wave * 16 * WN + jj * 16 + (lane / 16) * 4;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        if (c + x >= n) continue;
        float v = acc[i][jj][x];
        if (act >= ACT_SILU_PAIRS) {
          if (x % 2 == 0) out[(int64_t)(row0 + m) * ldc + (c + x) / 2] = from_float<TO>(pair_times(act, v, acc[i][jj][x + 1], pw, pa));
          continue;
        }
        if (act == ACT_RELU_SQUARED) v = v > 0.f ? v * v : 0.f;
        out[(int64_t)(row0 + m) * ldc + c + x] = from_float<TO>(v);
      }
    }
  }
}

// The same for steps that bring an expert a hundred rows and more: 128 rows x 128 columns per workgroup, a wave
// 64 x 64 as four by four products, so that a slice of K is fetched once for four times the work.
constexpr int WM = 128;

template <typename TO>
__global__ __launch_bounds__(256) void moe_experts_bf16_wide_kernel(TO* __restrict__ out, int ldc, const bf16* __restrict__ a, int lda,
                                                                    const bf16* __restrict__ w, int n, int k, const int* __restrict__ sorted,
                                                                    const int* __restrict__ tile_expert, int top, int gather, int act, const PairAct pa) {
  // Workgroups are dealt to the chip's eight dies in turn, each with an L2 of its own: number the tiles so that a die
  // gets neighbours (row tiles of one expert under one column tile, which share the weights).
  const int total = gridDim.x * gridDim.y, flat = blockIdx.y * gridDim.x + blockIdx.x;
  const int logical = total % 8 == 0 ? (flat % 8) * (total / 8) + flat / 8 : flat;
  const int tile_x = logical % gridDim.x, tile_y = logical / gridDim.x;
  const int expert = tile_expert[tile_x];
  if (expert < 0) return;
  __shared__ __attribute__((aligned(16))) bf16 a_s[WM][GK + GPAD];
  __shared__ __attribute__((aligned(16))) bf16 b_s[GN][GK + GPAD];
  __shared__ int row_of[WM];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int row0 = tile_x * WM, col0 = tile_y * GN;
  if (tid < WM) {
    const int pair = sorted[row0 + tid];
    row_of[tid] = pair < 0 ? -1 : (gather ? pair / top : row0 + tid);
  }
  __syncthreads();
  const bf16* we = w + (int64_t)expert * n * k;
  const int l_row = tid / 8, l_col = (tid % 8) * 8;          // a thread brings 16 bytes of rows l_row, + 32, + 64, + 96
  const bf16* a_ptr[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int src = row_of[p * 32 + l_row];
    a_ptr[p] = src >= 0 ? a + (int64_t)src * lda + l_col : nullptr;
  }
  bf16x8 a_reg[4], b_reg[4];
  const bf16x8 zero = {};
  auto fetch = [&](int k0) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      a_reg[p] = a_ptr[p] ? *(const bf16x8*)(a_ptr[p] + k0) : zero;
      const int r = p * 32 + l_row;
      b_reg[p] = col0 + r < n ? *(const bf16x8*)(we + (int64_t)(col0 + r) * k + k0 + l_col) : zero;
    }
  };
  floatx4 acc[4][4] = {};
  fetch(0);
  const int wm = wave / 2, wn = wave % 2, frag_row = lane % 16, frag_k = (lane / 16) * 8;
  for (int k0 = 0; k0 < k; k0 += GK) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      *(bf16x8*)&a_s[p * 32 + l_row][l_col] = a_reg[p];
      *(bf16x8*)&b_s[p * 32 + l_row][l_col] = b_reg[p];
    }
    __syncthreads();
    if (k0 + GK < k) fetch(k0 + GK);
#pragma unroll
    for (int kk = 0; kk < GK; kk += 32) {
      bf16x8 af[4], bfr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) af[i] = *(const bf16x8*)&a_s[wm * 64 + i * 16 + frag_row][kk + frag_k];
#pragma unroll
      for (int i = 0; i < 4; ++i) bfr[i] = *(const bf16x8*)&b_s[wn * 64 + i * 16 + frag_row][kk + frag_k];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
          acc[i][jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[jj], af[i], acc[i][jj], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = wm * 64 + i * 16 + lane % 16;
    if (row_of[m] < 0) continue;
    const float pw = act == ACT_CLAMPED_PAIRS ? weight_of_row(pa, sorted, row0 + m) : 1.f;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int c = col0 + wn * 64 + jj * 16 + (lane / 16) * 4;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        if (c + x >= n) continue;
        float v = acc[i][jj][x];
        if (act >= ACT_SILU_PAIRS) {
          if (x % 2 == 0) out[(int64_t)(row0 + m) * ldc + (c + x) / 2] = from_float<TO>(pair_times(act, v, acc[i][jj][x + 1], pw, pa));
          continue;
        }
        if (act == ACT_RELU_SQUARED) v = v > 0.f ? v * v : 0.f;
        out[(int64_t)(row0 + m) * ldc + c + x] = from_float<TO>(v);
      }
    }
  }
}

// The grouped product for large steps the way this package's many-rows product is made (gemm_bf16_wide in gemm.hip):
// 128 sorted rows x 256 columns of one expert per workgroup of four waves, a wave 64 rows x 128 columns; memory writes
// slices of 32 of K straight into LDS (fetch_to_lds), three stages, in a layout whose rows swap places and whose chunks
// are turned round by the row number so that every fragment read touches every bank once; no registers hold a slice on
// its way.  What differs from the dense kernel: a row's address comes from the sorted list (the token of the pair, or
// the sorted row itself), the weights are the tile's expert's, rows that pad an expert's run are fetched from the tile's
// first row and never written, and the epilogue may square the positive part.
template <typename TO>
__global__ __launch_bounds__(256, 2) void moe_experts_bf16_fetch_kernel(TO* __restrict__ out, int ldc, const bf16* __restrict__ x, int lda,
                                                                        const bf16* __restrict__ w, int n, int k, const int* __restrict__ sorted,
                                                                        const int* __restrict__ tile_expert, int tiles_m, int tiles_n, int top,
                                                                        int gather, int act, const PairAct pa) {
  constexpr int BM = 128, BN = 256, BK = 32, STAGES = 3;
  constexpr int XL = BM / 16 / 4, WL = BN / 16 / 4;
  constexpr int STAGE_ELEMENTS = (BM + BN) * BK;
  __shared__ __attribute__((aligned(64))) bf16 slices[STAGES * STAGE_ELEMENTS];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int r = lane & 15, g = lane >> 4;
  int id = blockIdx.x;
  const int tiles = tiles_m * tiles_n;
  if (tiles % 8 == 0) id = (id % 8) * (tiles / 8) + id / 8;        // consecutive workgroups go to different dies
  const int band = id / (4 * tiles_n), within = id % (4 * tiles_n);
  const int band_rows = tiles_m - band * 4 < 4 ? tiles_m - band * 4 : 4;
  const int tile_m = band * 4 + within % band_rows;
  const int expert = tile_expert[tile_m];
  if (expert < 0) return;
  const int m0 = tile_m * BM, n0 = (within / band_rows) * BN;
  const bf16* we = w + (int64_t)expert * n * k;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 128;
  const int place_row = (lane >> 2) ^ ((lane >> 5) & 1);
  const int place_chunk = (lane & 3) ^ ((place_row >> 1) & 3);
  const int first_pair = sorted[m0];                                 // a tile in use begins with a row in use
  const int fallback = gather ? first_pair / top : m0;
  unsigned xoff[XL], woff[WL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int at = m0 + 16 * (wave + 4 * i) + place_row, pair = sorted[at];
    const int row = pair < 0 ? fallback : (gather ? pair / top : at);
    xoff[i] = (unsigned)((row * lda + place_chunk * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int row = n0 + 16 * (wave + 4 * i) + place_row;
    woff[i] = (unsigned)(((row < n ? row : n - 1) * k + place_chunk * 8) * 2);
  }
  const int frag = ((r ^ ((r >> 3) & 1)) * 4 + (g ^ ((r >> 1) & 3))) * 8;
  floatx4 acc[8][4];
#pragma unroll
  for (int it = 0; it < 8; ++it)
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) acc[it][jt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int steps = k / BK;
  const unsigned slices_address = (unsigned)(uintptr_t)(__attribute__((address_space(3))) bf16*)slices;
  auto fetch = [&](int kt, int stage) {
    const int at = (kt < steps ? kt : steps - 1) * BK * 2;
    const unsigned to = slices_address + (unsigned)(stage * STAGE_ELEMENTS * 2 + wave * 1024);
#pragma unroll
    for (int i = 0; i < XL; ++i) fetch_to_lds((const char*)x + at, xoff[i], to + (unsigned)(i * 4096));
#pragma unroll
    for (int i = 0; i < WL; ++i) fetch_to_lds((const char*)we + at, woff[i], to + (unsigned)(BM * BK * 2 + i * 4096));
  };
  auto multiply = [&](int stage) {
    const bf16* xs = slices + stage * STAGE_ELEMENTS;
    const bf16* ws = xs + BM * BK;
    bf16x8 xf[4];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) xf[jt] = *(const bf16x8*)(xs + frag + (wm + jt * 16) * BK);
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const bf16x8 wf = *(const bf16x8*)(ws + frag + (wn + it * 16) * BK);
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) acc[it][jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[jt], acc[it][jt], 0, 0, 0);
    }
  };
  int m0_opaque = m0;
  fetch(0, 0);
  fetch(1, 1);
  fetched_then_barrier<6>();
  int stage = 0;
  for (int kt = 0; kt < steps; ++kt) {
    fetch(kt + 2, stage == 0 ? 2 : stage - 1);
    multiply(stage);
    fetched_then_barrier<6>();
    stage = stage == STAGES - 1 ? 0 : stage + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");               // the fetches past K that nobody reads
  asm volatile("" : "+s"(ldc), "+s"(m0_opaque));
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) {
    const int at = m0_opaque + wm + jt * 16 + r;
    const bool in_use = sorted[at] >= 0;
    const float pw = in_use && act == ACT_CLAMPED_PAIRS ? weight_of_row(pa, sorted, at) : 1.f;
    const int64_t row_at = (int64_t)at * ldc;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int row0 = n0 + wn + it * 16 + 4 * g;                  // this lane's four weight rows = output columns
      if (in_use && row0 < n) {
        floatx4 v = acc[it][jt];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __shfl(v[i], lane, WAVE);      // keeps the loop above free of spills, as in the dense kernel
        if (act == ACT_RELU_SQUARED) {
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = v[i] > 0.f ? v[i] * v[i] : 0.f;
        }
        if (act >= ACT_SILU_PAIRS) {
          const float first = pair_times(act, v[0], v[1], pw, pa), second = pair_times(act, v[2], v[3], pw, pa);
          if constexpr (sizeof(TO) == 2) *(bf16x2*)((bf16*)out + row_at + row0 / 2) = bf16x2{(bf16)first, (bf16)second};
          else ((float*)out)[row_at + row0 / 2] = first, ((float*)out)[row_at + row0 / 2 + 1] = second;
        } else if constexpr (sizeof(TO) == 2) *(bf16x4*)((bf16*)out + row_at + row0) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
        else *(floatx4*)((float*)out + row_at + row0) = v;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// What becomes of a token's weighted sum y of its experts' rows:
//   COMBINE_ADD        residual += y
//   COMBINE_ADD_RMS    residual += w * y * rsqrt(mean(y^2) + eps)                       (a layer that normalises what a sublayer gives out)
//   COMBINE_LAYERNORM  residual = w * (z - mean z) / sqrt(variance of z + eps), z = alpha * residual + y   (one that normalises the sum)
enum { COMBINE_ADD = 0, COMBINE_ADD_RMS = 1, COMBINE_LAYERNORM = 2 };

template <typename TW>
__global__ __launch_bounds__(1024) void moe_combine_kernel(float* __restrict__ residual, const float* __restrict__ rows, int hidden,
                                                           const int* __restrict__ place, const float* __restrict__ weights, int top,
                                                           const TW* __restrict__ norm_w, float eps, bf16* __restrict__ rounded, int kind,
                                                           float alpha, const float* __restrict__ extra) {
  extern __shared__ float sum[];        // [hidden], 16 floats for the reduction, then the token's rows and weights [top] each
  float* share = sum + hidden + 16;
  int* where = (int*)(share + top);
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < top; c += blockDim.x) {
    share[c] = weights ? weights[(int64_t)t * top + c] : 1.f;
    where[c] = place[(int64_t)t * top + c];
  }
  __syncthreads();
  float* out = residual + (int64_t)t * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float acc = 0.f;
    for (int c = 0; c < top; ++c) acc = fmaf(share[c], rows[(int64_t)where[c] * hidden + i], acc);
    if (extra) acc += extra[(int64_t)t * hidden + i];          // what a part that runs for every token gave out
    if (kind == COMBINE_LAYERNORM) {
      acc = fmaf(alpha, out[i], acc);
      ss += acc;                        // the sum of the row, for its mean
    } else {
      ss = fmaf(acc, acc, ss);
    }
    sum[i] = acc;
  }
  if (kind == COMBINE_LAYERNORM) {
    const float mean = block_sum(ss, sum + hidden) / (float)hidden;
    float sq = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float d = sum[i] - mean;    // written by this thread
      sq = fmaf(d, d, sq);
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, sum + hidden) / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float v = (sum[i] - mean) * inv * to_float(norm_w[i]);
      out[i] = v;
      if (rounded) rounded[(int64_t)t * hidden + i] = (bf16)v;
    }
    return;
  }
  float inv = 1.f;
  if (kind == COMBINE_ADD_RMS) {
    ss = block_sum(ss, sum + hidden);
    inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  }
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = out[i] + (kind == COMBINE_ADD_RMS ? sum[i] * inv * to_float(norm_w[i]) : sum[i]);
    out[i] = v;
    if (rounded) rounded[(int64_t)t * hidden + i] = (bf16)v;       // the stream as the next sublayer reads it
  }
}

}  // namespace

// Rows of a tile of the grouped products: 32, or 128 once the step brings every expert 48 rows and more on average: what
// a step of a few dozen rows an expert pays for is how often an expert's weights are fetched, once a tile, and not
// the matrix instructions on rows that only pad (8 layers at the 8B sizes, a prompt of 512 tokens, 128 rows an expert:
// 6.9 ms with tiles of 128, 9.8 ms with tiles of 32).  Follows from the step's shape alone, so that recorded and captured
// steps keep it.
LRS_API int lrs_moe_tile_rows(int pairs, int experts) { return (int64_t)pairs >= (int64_t)48 * experts ? WM : GM; }

// The most tiles that `pairs` (token, choice) pairs of `experts` experts can fill: every expert in use ends in at
// most one tile that is not full.
LRS_API int lrs_moe_max_tiles(int pairs, int experts) {
  const int padded = pairs / lrs_moe_tile_rows(pairs, experts) + experts;
  return pairs < padded ? pairs : padded;
}

static int check_rule(const char* who, int kind, int groups, int keep, float scale, int experts, int top) {
  LRS_REQUIRE(kind >= ROUTE_SOFTMAX_CHOSEN && kind <= ROUTE_SIGMOID_SCORES, "%s: unknown routing rule %d", who, kind);
  if (kind == ROUTE_SOFTMAX_CHOSEN) {
    LRS_REQUIRE(groups == 0, "%s: groups of experts come with the sigmoid rule only", who);
    return 0;
  }
  LRS_REQUIRE(scale > 0.f, "%s: the weights' scale must be positive", who);
  if (groups > 0) {
    LRS_REQUIRE(experts % groups == 0 && keep > 0 && keep <= groups, "%s: %d experts do not form %d equal groups of which %d are kept", who, experts, groups, keep);
    LRS_REQUIRE((int64_t)keep * (experts / groups) >= top, "%s: %d groups of %d experts hold fewer than the %d to choose", who, keep, experts / groups, top);
  }
  return 0;
}

// rule, groups, keep, scale: see RouteRule (0, 0, 0, 1 for the softmax over the chosen logits).
LRS_API int lrs_moe_route(const float* logits, int ld, const float* bias, int* ids, float* weights, int tokens, int experts,
                          int top, int rule, int groups, int keep, float scale, void* stream) {
  if (int rc = check_rule("moe_route", rule, groups, keep, scale, experts, top)) return rc;
  LRS_REQUIRE(tokens > 0 && experts > 0 && top > 0 && top <= experts, "moe_route: bad sizes tokens=%d experts=%d top=%d", tokens, experts, top);
  LRS_REQUIRE(experts <= WAVE * ROUTE_MAX_PER_LANE, "moe_route: at most %d experts, got %d", WAVE * ROUTE_MAX_PER_LANE, experts);
  LRS_REQUIRE(ld >= experts, "moe_route: rows of %d logits hold fewer than %d experts", ld, experts);
  moe_route_kernel<<<(tokens + 3) / 4, 256, 0, (hipStream_t)stream>>>(logits, ld, bias, ids, weights, tokens, experts, top, RouteRule{rule, groups, keep, scale});
  return lrs_check_launch("moe_route");
}

LRS_API int lrs_moe_align(const int* ids, int pairs, int experts, int* sorted, int capacity, int* place, int* tile_expert,
                          int max_tiles, void* stream) {
  LRS_REQUIRE(pairs > 0 && experts > 0, "moe_align: bad sizes pairs=%d experts=%d", pairs, experts);
  const int tile = lrs_moe_tile_rows(pairs, experts);
  LRS_REQUIRE(max_tiles >= lrs_moe_max_tiles(pairs, experts), "moe_align: %d tiles may not hold %d pairs of %d experts", max_tiles, pairs, experts);
  LRS_REQUIRE(capacity >= max_tiles * tile, "moe_align: the sorted list holds %d rows, %d tiles need %d", capacity, max_tiles, max_tiles * tile);
  const size_t lds = (size_t)(3 * experts + 1) * sizeof(int);
  LRS_REQUIRE(lds <= 48 * 1024, "moe_align: %d experts are too many", experts);
  moe_align_kernel<<<1, 1024, lds, (hipStream_t)stream>>>(ids, pairs, experts, tile, sorted, capacity, place, tile_expert, max_tiles);
  return lrs_check_launch("moe_align");
}

LRS_API int lrs_moe_route_align(const float* logits, int ld, const float* bias, int* ids, float* weights, int tokens, int experts,
                                int top, int* sorted, int capacity, int* place, int* tile_expert, int max_tiles, int rule, int groups, int keep,
                                float scale, void* stream) {
  if (int rc = check_rule("moe_route_align", rule, groups, keep, scale, experts, top)) return rc;
  LRS_REQUIRE(tokens > 0 && tokens <= 256 && experts > 0 && top > 0 && top <= experts, "moe_route_align: bad sizes tokens=%d experts=%d top=%d", tokens, experts, top);
  LRS_REQUIRE(experts <= WAVE * ROUTE_MAX_PER_LANE && ld >= experts, "moe_route_align: at most %d experts in rows of at least as many logits", WAVE * ROUTE_MAX_PER_LANE);
  const int pairs = tokens * top, tile = lrs_moe_tile_rows(pairs, experts);
  LRS_REQUIRE(max_tiles >= lrs_moe_max_tiles(pairs, experts), "moe_route_align: %d tiles may not hold %d pairs of %d experts", max_tiles, pairs, experts);
  LRS_REQUIRE(capacity >= max_tiles * tile, "moe_route_align: the sorted list holds %d rows, %d tiles need %d", capacity, max_tiles, max_tiles * tile);
  const size_t lds = (size_t)(3 * experts + 1) * sizeof(int);
  moe_route_align_kernel<<<1, 1024, lds, (hipStream_t)stream>>>(logits, ld, bias, ids, weights, tokens, experts, top, tile, sorted, capacity, place,
                                                                tile_expert, max_tiles, RouteRule{rule, groups, keep, scale});
  return lrs_check_launch("moe_route_align");
}

// out [max_tiles * tile, n] = rows of `a` (row pair / top of the sorted list if `gather`, else the sorted row
// itself) times the tile's expert matrix w[expert] [n, k], transposed; act 1: the square of relu; act 2: see ACT_SILU_PAIRS (out has n / 2 columns).
LRS_API int lrs_moe_experts(void* out, int out_dtype, int ldc, const void* a, const void* w, int dtype, int lda, int n, int k,
                            const int* sorted, const int* tile_expert, int max_tiles, int tile, int top, int gather, int act,
                            const float* pair_weights, float act_alpha, float act_limit, void* stream) {
  const PairAct pa{pair_weights, act_alpha, act_limit};
  LRS_REQUIRE(tile == GM || tile == WM, "moe_experts: tiles have %d or %d rows, got %d", GM, WM, tile);
  LRS_REQUIRE(max_tiles > 0 && n > 0 && k > 0 && top > 0, "moe_experts: bad sizes tiles=%d n=%d k=%d top=%d", max_tiles, n, k, top);
  LRS_REQUIRE(act >= ACT_NONE && act <= ACT_CLAMPED_PAIRS, "moe_experts: unknown activation %d", act);
  LRS_REQUIRE(act != ACT_CLAMPED_PAIRS || act_limit > 0.f, "moe_experts: the clamp's limit must be positive, got %g", (double)act_limit);
  LRS_REQUIRE(act == ACT_CLAMPED_PAIRS || pair_weights == nullptr, "moe_experts: weights on the inputs come with the clamped activation");
  LRS_REQUIRE(lda >= k && ldc >= (act >= ACT_SILU_PAIRS ? n / 2 : n), "moe_experts: strides lda=%d ldc=%d too small for k=%d n=%d", lda, ldc, k, n);
  LRS_REQUIRE(act < ACT_SILU_PAIRS || n % 4 == 0, "moe_experts: pairs of gate and up rows come four rows at a time, got %d rows", n);
  hipStream_t s = (hipStream_t)stream;
  const bool cores = dtype == LRS_BF16 && k % GK == 0 && lda % 8 == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0;
  // large steps of shapes the fetching kernel takes: whole slices of 32 of K, rows of the output 16 bytes aligned, offsets
  // that fit 32 bits
  const bool fetching = cores && tile == WM && k % 32 == 0 && n % 4 == 0 && ldc % 4 == 0 && ((uintptr_t)out % 16) == 0 && k >= 64 &&
                        (int64_t)n * k < (1ll << 30) && (gather ? (int64_t)max_tiles * tile / top + 1 : (int64_t)max_tiles * tile) * lda < (1ll << 30);
  if (fetching) {
    const int tiles_n = (n + 255) / 256;
    if (out_dtype == LRS_BF16)
      moe_experts_bf16_fetch_kernel<bf16><<<max_tiles * tiles_n, 256, 0, s>>>((bf16*)out, ldc, (const bf16*)a, lda, (const bf16*)w, n, k, sorted, tile_expert, max_tiles, tiles_n, top, gather, act, pa);
    else if (out_dtype == LRS_F32)
      moe_experts_bf16_fetch_kernel<float><<<max_tiles * tiles_n, 256, 0, s>>>((float*)out, ldc, (const bf16*)a, lda, (const bf16*)w, n, k, sorted, tile_expert, max_tiles, tiles_n, top, gather, act, pa);
    else
      return lrs_fail("moe_experts: unknown output dtype %d", out_dtype);
    return lrs_check_launch("moe_experts");
  }
  if (cores && tile == WM) {
    dim3 grid(max_tiles, (n + GN - 1) / GN);
    if (out_dtype == LRS_BF16)
      moe_experts_bf16_wide_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)out, ldc, (const bf16*)a, lda, (const bf16*)w, n, k, sorted, tile_expert, top, gather, act, pa);
    else if (out_dtype == LRS_F32)
      moe_experts_bf16_wide_kernel<float><<<grid, 256, 0, s>>>((float*)out, ldc, (const bf16*)a, lda, (const bf16*)w, n, k, sorted, tile_expert, top, gather, act, pa);
    else
      return lrs_fail("moe_experts: unknown output dtype %d", out_dtype);
    return lrs_check_launch("moe_experts");
  }
  if (cores) {
    // few tiles (single tokens, short portions): 64 columns a workgroup, so that twice as many stream the weights
    const bool narrow = (int64_t)max_tiles * ((n + GN - 1) / GN) < 4 * lrs_compute_units();
    dim3 grid(max_tiles, narrow ? (n + 63) / 64 : (n + GN - 1) / GN);
#define CORES(TO, NT) moe_experts_bf16_kernel<TO, NT><<<grid, 256, 0, s>>>((TO*)out, ldc, (const bf16*)a, lda, (const bf16*)w, n, k, sorted, tile_expert, top, gather, act, pa)
    if (out_dtype == LRS_BF16) { if (narrow) CORES(bf16, 64); else CORES(bf16, 128); }
    else if (out_dtype == LRS_F32) { if (narrow) CORES(float, 64); else CORES(float, 128); }
    else return lrs_fail("moe_experts: unknown output dtype %d", out_dtype);
#undef CORES
    return lrs_check_launch("moe_experts");
  }
  dim3 grid(max_tiles * (tile / GM), (n + 63) / 64);       // the any-shape form walks a tile of 128 rows as four of 32
#define RUN(T, TO) moe_experts_kernel<T, TO><<<grid, 256, 0, s>>>((TO*)out, ldc, (const T*)a, lda, (const T*)w, n, k, sorted, tile_expert, top, gather, act, tile / GM, pa)
  if (dtype == LRS_F32 && out_dtype == LRS_F32) RUN(float, float);
  else if (dtype == LRS_BF16 && out_dtype == LRS_BF16) RUN(bf16, bf16);
  else if (dtype == LRS_BF16 && out_dtype == LRS_F32) RUN(bf16, float);
  else return lrs_fail("moe_experts: inputs of dtype %d with outputs of dtype %d are not served", dtype, out_dtype);
#undef RUN
  return lrs_check_launch("moe_experts");
}

// residual [tokens, hidden] += (norm of) sum_c weights[t, c] * rows[place[t, c]]; norm_w null: the plain sum; rounded:
// where the updated rows are left in bfloat16 as well, or null.  weights null: every choice counts once.  extra [tokens, hidden]
// (or null): rows added to the sum before the norm.
LRS_API int lrs_moe_combine(float* residual, const float* rows, int tokens, int hidden, const int* place, const float* weights,
                            int top, const void* norm_w, int norm_dtype, float eps, void* rounded, int layer_norm, float alpha,
                            const float* extra, void* stream) {
  // layer_norm (with a norm weight): the stream becomes the layer norm of alpha * stream + sum, instead of taking the sum's RMS norm on top
  LRS_REQUIRE(tokens > 0 && hidden > 0 && top > 0, "moe_combine: bad sizes tokens=%d hidden=%d top=%d", tokens, hidden, top);
  LRS_REQUIRE(!norm_w || eps > 0.f, "moe_combine: eps must be positive");
  LRS_REQUIRE(!layer_norm || norm_w, "moe_combine: a layer norm needs its weight");
  const int kind = !norm_w ? COMBINE_ADD : layer_norm ? COMBINE_LAYERNORM : COMBINE_ADD_RMS;
  const size_t lds = (size_t)(hidden + 16 + 2 * top) * sizeof(float);
  LRS_REQUIRE(lds <= 64 * 1024, "moe_combine: a width of %d with %d choices is too much", hidden, top);
  hipStream_t s = (hipStream_t)stream;
  const int threads = hidden >= 2048 ? 1024 : 256;
  if (norm_w && norm_dtype == LRS_BF16)
    moe_combine_kernel<bf16><<<tokens, threads, lds, s>>>(residual, rows, hidden, place, weights, top, (const bf16*)norm_w, eps, (bf16*)rounded, kind, alpha, extra);
  else
    moe_combine_kernel<float><<<tokens, threads, lds, s>>>(residual, rows, hidden, place, weights, top, (const float*)norm_w, eps, (bf16*)rounded, kind, alpha, extra);
  return lrs_check_launch("moe_combine");
}

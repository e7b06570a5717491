// Attention heads that are rotated first and normalised afterwards, and small kernels of layers built around them.
//
//   rotate_unit_prep   per token of the fused projection row [q: nq*d | k: nkv*d | v: nkv*dv | ...]: a bias per column is added
//                      (where the layer has one: the product before this kernel then leaves it out), the first 2*rot_half dims
//                      of every q and k head are turned by the token's angles (pairs (j, j + rot_half), or neighbours
//                      (2j, 2j + 1)), then the head is divided by its own root mean square over all d dims (no weight); q
//                      written back in place, k into the key pages [page, kv_head, slot, d], v into the value pages
//                      [page, kv_head, dv, slot];
//   gated_clamped      out[t, j] = g * sigmoid(alpha * g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit),
//                      for rows [gate: inter | up: inter];
//   add_gathered       out[t, :] += table[ids[t], :] over float32 rows (a learned position vector added to the stream);
//   scale_values       x *= factor over float32 values (logits times a constant).
#include "common.h"

namespace {

// One pair or single dim of a head, rotated: item j < rot_half is a pair, item j >= rot_half the single dim j + rot_half.
struct Item {
  int first, second;      // dims; second < 0: a single dim
  float a, b;
};

template <typename T>
__device__ __forceinline__ Item rotated_item(const T* __restrict__ src, const float* __restrict__ bias, int j, int rot_half, int neighbours,
                                             const float* __restrict__ cosrow, const float* __restrict__ sinrow) {
  Item it;
  if (j < rot_half) {
    it.first = neighbours ? 2 * j : j;
    it.second = neighbours ? 2 * j + 1 : j + rot_half;
    const float u = to_float(src[it.first]) + (bias ? bias[it.first] : 0.f), v = to_float(src[it.second]) + (bias ? bias[it.second] : 0.f);
    const float c = cosrow[j], s = sinrow[j];
    it.a = u * c - v * s;
    it.b = v * c + u * s;
  } else {
    it.first = j + rot_half;
    it.second = -1;
    it.a = to_float(src[it.first]) + (bias ? bias[it.first] : 0.f);
    it.b = 0.f;
  }
  return it;
}

// A workgroup four heads of a token, a wave a head (blockIdx.y counts the groups of four).  The rotated values are made twice, once for the sum of squares and once
// for the write, by the same operations (the same bits); every value is read and written by one lane only, so q can be
// written where it was read.
template <typename T>
__global__ __launch_bounds__(256) void rotate_unit_prep_kernel(T* __restrict__ qkv, int row_stride, int nq, int nkv, int d, int dv, float eps,
                                                               int unit, const float* __restrict__ cosv, const float* __restrict__ sinv,
                                                               int rot_half, int neighbours, T* __restrict__ k_pages,
                                                               T* __restrict__ v_pages, const int* __restrict__ slots, int page_size,
                                                               const float* __restrict__ bias) {
  const int token = blockIdx.x, tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  T* row = qkv + (int64_t)token * row_stride;
  const int slot = slots ? slots[token] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const float* cosrow = cosv + (int64_t)token * rot_half;
  const float* sinrow = sinv + (int64_t)token * rot_half;
  const int items = d - rot_half;
  const int head = blockIdx.y * 4 + wave;
  if (head < nq + nkv) {
    const bool is_q = head < nq;
    const T* src = row + (int64_t)head * d;
    const float* hb = bias ? bias + (int64_t)head * d : nullptr;
    float ss = 0.f;
    if (unit && (is_q || slot >= 0)) {
      for (int j = lane; j < items; j += WAVE) {
        const Item it = rotated_item(src, hb, j, rot_half, neighbours, cosrow, sinrow);
        ss = fmaf(it.a, it.a, ss);
        ss = fmaf(it.b, it.b, ss);
      }
      ss = wave_sum(ss);
    }
    const float inv = unit ? 1.0f / sqrtf(ss / (float)d + eps) : 1.f;
    T* dst = is_q ? row + (int64_t)head * d : k_pages + ((page * nkv + (head - nq)) * page_size + off) * d;
    if (is_q || slot >= 0) {
      for (int j = lane; j < items; j += WAVE) {
        const Item it = rotated_item(src, hb, j, rot_half, neighbours, cosrow, sinrow);
        dst[it.first] = from_float<T>(it.a * inv);
        if (it.second >= 0) dst[it.second] = from_float<T>(it.b * inv);
      }
    }
  }
  if (slot >= 0 && v_pages) {           // the values, dealt out over the token's workgroups (null: values_in_runs_kernel stores them)
    const int qn = nq * d, kn = nkv * d, vn = nkv * dv;
    for (int e = blockIdx.y * 256 + tid; e < vn; e += 256 * gridDim.y) {
      const int kvh = e / dv, i = e % dv;
      const float v = to_float(row[qn + kn + e]) + (bias ? bias[qn + kn + e] : 0.f);
      v_pages[((page * nkv + kvh) * dv + i) * page_size + off] = from_float<T>(v);
    }
  }
}

// The same for bfloat16 heads whose size and rotated part are multiples of eight (sixteen for neighbouring pairs): 16 bytes a
// load, a lane holds runs of eight dims (a run and its partner run where the pairs lie rot_half apart; one run of four pairs
// where they are neighbours), which stay in registers between the sum of squares and the write.  A head of up to 512 dims.
// A head of few items shares its wave with others: `lanes` (a power of two, at least the head's items, 64 at most) lanes a head,
// 64 / lanes heads a wave, and the sum of squares goes round those lanes only (a head of 128 dims is 12 or 16 items: four heads
// a wave, where a wave a head left three lanes in four idle).
constexpr int RUNS = 4;      // work items a lane holds: 64 lanes x 4 items x up to 16 dims

__host__ __device__ inline int lanes_of_head(int items) {
  int lanes = 1;
  while (lanes < items && lanes < WAVE) lanes *= 2;
  return lanes;
}

__global__ __launch_bounds__(256) void rotate_unit_prep_vec_kernel(bf16* __restrict__ qkv, int row_stride, int nq, int nkv, int d, int dv,
                                                                   float eps, int unit, const float* __restrict__ cosv,
                                                                   const float* __restrict__ sinv, int rot_half, int neighbours,
                                                                   bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                                                                   const int* __restrict__ slots, int page_size, const float* __restrict__ bias) {
  const int token = blockIdx.x, tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  bf16* row = qkv + (int64_t)token * row_stride;
  const int slot = slots ? slots[token] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const float* cosrow = cosv + (int64_t)token * rot_half;
  const float* sinrow = sinv + (int64_t)token * rot_half;
  // items of a head: with pairs rot_half apart, item j < rot_half / 8 is the runs (8j, 8j + rot_half), the rest single runs
  // behind the rotated part; with neighbours, item j < rot_half / 4 is the run 8j (four pairs), the rest single runs
  const int paired = neighbours ? rot_half / 4 : rot_half / 8;
  const int items = neighbours ? d / 8 : (d - rot_half) / 8;
  const int lanes = lanes_of_head(items), per_wave = WAVE / lanes, own = lane % lanes;
  const int head = (blockIdx.y * 4 + wave) * per_wave + lane / lanes;
  // eight values of a run with their biases added
  auto run_of = [&](const bf16* at, const float* b, float (&out)[8]) {
    const bf16x8 x = *(const bf16x8*)at;
    floatx4 b0 = {0.f, 0.f, 0.f, 0.f}, b1 = b0;
    if (b) b0 = *(const floatx4*)b, b1 = *(const floatx4*)(b + 4);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = (float)x[i] + (i < 4 ? b0[i] : b1[i - 4]);
  };
  if (head < nq + nkv && (head < nq || slot >= 0)) {
    const bool is_q = head < nq;
    const bf16* src = row + (int64_t)head * d;
    const float* hb = bias ? bias + (int64_t)head * d : nullptr;
    float va[RUNS][8], vb[RUNS][8];
    float ss = 0.f;
#pragma unroll
    for (int n = 0; n < RUNS; ++n) {
      const int j = own + n * lanes;
      if (j >= items) continue;
      if (j < paired && !neighbours) {
        float lo[8], hi[8];
        run_of(src + j * 8, hb ? hb + j * 8 : nullptr, lo);
        run_of(src + j * 8 + rot_half, hb ? hb + j * 8 + rot_half : nullptr, hi);
        floatx4 c4[2], s4[2];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          c4[half] = *(const floatx4*)(cosrow + j * 8 + half * 4);
          s4[half] = *(const floatx4*)(sinrow + j * 8 + half * 4);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float u = lo[i], v = hi[i], c = c4[i / 4][i % 4], s = s4[i / 4][i % 4];
          va[n][i] = u * c - v * s;
          vb[n][i] = v * c + u * s;
          ss = fmaf(va[n][i], va[n][i], ss);
          ss = fmaf(vb[n][i], vb[n][i], ss);
        }
      } else if (j < paired) {
        float x[8];
        run_of(src + j * 8, hb ? hb + j * 8 : nullptr, x);
        const floatx4 c4 = *(const floatx4*)(cosrow + j * 4), s4 = *(const floatx4*)(sinrow + j * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float u = x[2 * i], v = x[2 * i + 1];
          va[n][2 * i] = u * c4[i] - v * s4[i];
          va[n][2 * i + 1] = v * c4[i] + u * s4[i];
          ss = fmaf(va[n][2 * i], va[n][2 * i], ss);
          ss = fmaf(va[n][2 * i + 1], va[n][2 * i + 1], ss);
        }
      } else {
        const int at = neighbours ? j * 8 : j * 8 + rot_half;
        run_of(src + at, hb ? hb + at : nullptr, va[n]);
#pragma unroll
        for (int i = 0; i < 8; ++i) ss = fmaf(va[n][i], va[n][i], ss);
      }
    }
    for (int step = lanes / 2; step > 0; step /= 2) ss += __shfl_xor(ss, step, WAVE);      // among the head's own lanes
    const float inv = unit ? 1.0f / sqrtf(ss / (float)d + eps) : 1.f;
    bf16* dst = is_q ? row + (int64_t)head * d : k_pages + ((page * nkv + (head - nq)) * page_size + off) * d;
#pragma unroll
    for (int n = 0; n < RUNS; ++n) {
      const int j = own + n * lanes;
      if (j >= items) continue;
      bf16x8 first;
#pragma unroll
      for (int i = 0; i < 8; ++i) first[i] = (bf16)(va[n][i] * inv);
      if (j < paired && !neighbours) {
        bf16x8 second;
#pragma unroll
        for (int i = 0; i < 8; ++i) second[i] = (bf16)(vb[n][i] * inv);
        *(bf16x8*)(dst + j * 8) = first;
        *(bf16x8*)(dst + j * 8 + rot_half) = second;
      } else {
        *(bf16x8*)(dst + (neighbours || j < paired ? j * 8 : j * 8 + rot_half)) = first;
      }
    }
  }
  if (slot >= 0 && v_pages) {           // the values, dealt out over the token's workgroups (null: values_in_runs_kernel stores them)
    const int qn = nq * d, kn = nkv * d, vn = nkv * dv;
    for (int e = blockIdx.y * 256 + tid; e < vn; e += 256 * gridDim.y) {
      const int kvh = e / dv, i = e % dv;
      const float v = (float)row[qn + kn + e] + (bias ? bias[qn + kn + e] : 0.f);
      v_pages[((page * nkv + kvh) * dv + i) * page_size + off] = (bf16)v;
    }
  }
}

// The values of 16 consecutive tokens of the step and one kv head into the value pages [page, kv_head, dv, slot], for steps of
// many tokens: tokens that follow each other inside a page lie side by side there, so a thread gathers one dim of 16 / sizeof(T)
// such tokens (neighbouring lanes read neighbouring dims of one token), adds the dim's bias and writes one 16-byte store; where
// a run is broken (a page's edge, another request, a slot that is not stored) it stores one by one.
template <typename T>
__global__ __launch_bounds__(256) void values_in_runs_kernel(const T* __restrict__ qkv, int row_stride, int v_offset, int tokens, int nkv, int dv,
                                                             T* __restrict__ v_pages, const int* __restrict__ slots, int page_size,
                                                             const float* __restrict__ bias) {
  constexpr int RUN = 16 / sizeof(T);
  typedef T vec __attribute__((ext_vector_type(RUN)));
  __shared__ int slot_of[16];
  const int tid = threadIdx.x, token0 = blockIdx.x * 16, kvh = blockIdx.y;
  if (tid < 16) slot_of[tid] = token0 + tid < tokens ? slots[token0 + tid] : -1;
  __syncthreads();
  for (int e = tid; e < dv * (16 / RUN); e += 256) {
    const int dim = e % dv, first = (e / dv) * RUN;
    const int slot0 = slot_of[first];
    bool run = slot0 >= 0 && slot0 % RUN == 0 && slot0 % page_size + RUN <= page_size;
#pragma unroll
    for (int i = 1; i < RUN; ++i) run = run && slot_of[first + i] == slot0 + i;
    const int column = v_offset + kvh * dv + dim;
    const float b = bias ? bias[column] : 0.f;
    const T* src = qkv + (int64_t)(token0 + first) * row_stride + column;
    if (run) {
      vec v;
#pragma unroll
      for (int i = 0; i < RUN; ++i) v[i] = from_float<T>(to_float(src[(int64_t)i * row_stride]) + b);
      const int64_t page = slot0 / page_size, off = slot0 % page_size;
      *(vec*)(v_pages + ((page * nkv + kvh) * dv + dim) * page_size + off) = v;
    } else {
#pragma unroll
      for (int i = 0; i < RUN; ++i) {
        const int slot = slot_of[first + i];
        if (slot < 0) continue;
        const int64_t page = slot / page_size, off = slot % page_size;
        v_pages[((page * nkv + kvh) * dv + dim) * page_size + off] = from_float<T>(to_float(src[(int64_t)i * row_stride]) + b);
      }
    }
  }
}

template <typename T>
__global__ void gated_clamped_kernel(T* __restrict__ out, const T* __restrict__ gu, int64_t count, int inter, float alpha, float limit) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= count) return;
  const int64_t t = e / inter, j = e % inter;
  const float g = fminf(to_float(gu[t * 2 * inter + j]), limit);
  const float u = fminf(fmaxf(to_float(gu[t * 2 * inter + inter + j]), -limit), limit);
  out[e] = from_float<T>(g / (1.f + expf(-alpha * g)) * (u + 1.f));
}

template <typename T>
__global__ void add_gathered_kernel(float* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids, int64_t count, int cols) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= count) return;
  const int64_t t = e / cols, c = e % cols;
  out[e] += to_float(table[(int64_t)ids[t] * cols + c]);
}

__global__ void scale_values_kernel(float* __restrict__ x, int64_t count, float factor) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e < count) x[e] *= factor;
}

}  // namespace

// qkv [tokens, row_stride] in dtype: q (nq*d) | k (nkv*d) | v (nkv*dv) | anything else.  cos, sin [tokens, rot_half] float32
// (rot_half 0: no rotation).  neighbours: the pairs are dims (2j, 2j + 1) instead of (j, j + rot_half).  unit: every head is
// divided by sqrt(mean of its squares + eps) after the rotation.  slots[t] = page * page_size + offset (negative: the token's
// key and value are not stored).  bias (float32 [nq*d + nkv*d + nkv*dv], or null): added to q, k and v as they are read.
LRS_API int lrs_rotate_unit_prep(void* qkv, int dtype, int tokens, int row_stride, int nq, int nkv, int d, int dv, float eps, int unit,
                                 const float* cosv, const float* sinv, int rot_half, int neighbours, void* k_pages, void* v_pages,
                                 const int* slots, int page_size, const float* bias, void* stream) {
  LRS_REQUIRE(tokens > 0 && nq > 0 && nkv > 0 && d > 0 && dv > 0, "rotate_unit_prep: bad sizes tokens=%d nq=%d nkv=%d d=%d dv=%d", tokens, nq, nkv, d, dv);
  LRS_REQUIRE(row_stride >= nq * d + nkv * d + nkv * dv, "rotate_unit_prep: rows of %d hold fewer than q, k and v", row_stride);
  LRS_REQUIRE(rot_half >= 0 && 2 * rot_half <= d, "rotate_unit_prep: rotary width %d exceeds head_dim %d", 2 * rot_half, d);
  LRS_REQUIRE(rot_half == 0 || (cosv && sinv), "rotate_unit_prep: rotation asked for without tables");
  LRS_REQUIRE(!unit || eps > 0.f, "rotate_unit_prep: eps must be positive");
  LRS_REQUIRE(k_pages && v_pages && slots && page_size > 0, "rotate_unit_prep: cache write needs pages, slots and a page size");
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(tokens, (nq + nkv + 3) / 4);
  // steps of many tokens: the values as runs of slots, 16 bytes a store, by workgroups of their own (token by token they are
  // 2-byte writes a page row apart)
  if (tokens >= 64 && page_size % (dtype == LRS_F32 ? 4 : 8) == 0 && (uintptr_t)v_pages % 16 == 0) {
    const dim3 vgrid((tokens + 15) / 16, nkv);
    if (dtype == LRS_F32)
      values_in_runs_kernel<float><<<vgrid, 256, 0, s>>>((const float*)qkv, row_stride, (nq + nkv) * d, tokens, nkv, dv, (float*)v_pages, slots, page_size, bias);
    else if (dtype == LRS_BF16)
      values_in_runs_kernel<bf16><<<vgrid, 256, 0, s>>>((const bf16*)qkv, row_stride, (nq + nkv) * d, tokens, nkv, dv, (bf16*)v_pages, slots, page_size, bias);
    else return lrs_fail("rotate_unit_prep: unknown dtype %d", dtype);
    if (lrs_check_launch("values_in_runs")) return 1;
    v_pages = nullptr;
  }
  if (dtype == LRS_F32)
    rotate_unit_prep_kernel<float><<<grid, 256, 0, s>>>((float*)qkv, row_stride, nq, nkv, d, dv, eps, unit, cosv, sinv, rot_half, neighbours,
                                                        (float*)k_pages, (float*)v_pages, slots, page_size, bias);
  else if (dtype == LRS_BF16 && d % 8 == 0 && d <= 8 * WAVE * RUNS && rot_half % (neighbours ? 4 : 8) == 0 && row_stride % 8 == 0 &&
           ((uintptr_t)qkv | (uintptr_t)cosv | (uintptr_t)sinv | (uintptr_t)k_pages | (uintptr_t)bias) % 16 == 0) {
    const int per_block = 4 * (WAVE / lanes_of_head(neighbours ? d / 8 : (d - rot_half) / 8));       // heads a workgroup takes
    grid.y = (nq + nkv + per_block - 1) / per_block;
    rotate_unit_prep_vec_kernel<<<grid, 256, 0, s>>>((bf16*)qkv, row_stride, nq, nkv, d, dv, eps, unit, cosv, sinv, rot_half, neighbours,
                                                     (bf16*)k_pages, (bf16*)v_pages, slots, page_size, bias);
  } else if (dtype == LRS_BF16)
    rotate_unit_prep_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)qkv, row_stride, nq, nkv, d, dv, eps, unit, cosv, sinv, rot_half, neighbours,
                                                       (bf16*)k_pages, (bf16*)v_pages, slots, page_size, bias);
  else return lrs_fail("rotate_unit_prep: unknown dtype %d", dtype);
  return lrs_check_launch("rotate_unit_prep");
}

// out [tokens, inter] from gate_up [tokens, 2 * inter] (gate columns, then up columns), both contiguous, of one dtype.
LRS_API int lrs_gated_clamped(void* out, const void* gate_up, int dtype, int tokens, int inter, float alpha, float limit, void* stream) {
  LRS_REQUIRE(tokens > 0 && inter > 0 && limit > 0.f, "gated_clamped: bad arguments tokens=%d inter=%d limit=%g", tokens, inter, (double)limit);
  const int64_t count = (int64_t)tokens * inter;
  const unsigned blocks = (unsigned)((count + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_F32) gated_clamped_kernel<float><<<blocks, 256, 0, s>>>((float*)out, (const float*)gate_up, count, inter, alpha, limit);
  else if (dtype == LRS_BF16) gated_clamped_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)out, (const bf16*)gate_up, count, inter, alpha, limit);
  else return lrs_fail("gated_clamped: unknown dtype %d", dtype);
  return lrs_check_launch("gated_clamped");
}

// out [tokens, cols] float32 += table[ids[t]] (table [rows, cols] in dtype; the caller answers for ids within the table).
LRS_API int lrs_add_gathered(float* out, const void* table, int dtype, const int* ids, int tokens, int cols, void* stream) {
  LRS_REQUIRE(tokens > 0 && cols > 0, "add_gathered: bad sizes tokens=%d cols=%d", tokens, cols);
  const int64_t count = (int64_t)tokens * cols;
  const unsigned blocks = (unsigned)((count + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_F32) add_gathered_kernel<float><<<blocks, 256, 0, s>>>(out, (const float*)table, ids, count, cols);
  else if (dtype == LRS_BF16) add_gathered_kernel<bf16><<<blocks, 256, 0, s>>>(out, (const bf16*)table, ids, count, cols);
  else return lrs_fail("add_gathered: unknown dtype %d", dtype);
  return lrs_check_launch("add_gathered");
}

LRS_API int lrs_scale_values(float* x, int64_t count, float factor, void* stream) {
  LRS_REQUIRE(count > 0, "scale_values: nothing to scale");
  scale_values_kernel<<<(unsigned)((count + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, count, factor);
  return lrs_check_launch("scale_values");
}

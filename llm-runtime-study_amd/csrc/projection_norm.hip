// Attention heads whose q and k are normalised over the whole projection (all heads of a token at once), and the
// small elementwise kernels of layers that run their sublayers side by side.
//
//   qkv_norm_prep   per token of the fused projection row [q: nq*d | k: nkv*d | v: nkv*dv | ...]: the RMS norm of the
//                   whole q part and of the whole k part (one sum of squares each, a weight per column), the half-split
//                   rotation of the first 2*rot_half dims of every q and k head, q written back in place, k into the
//                   key pages [page, kv_head, slot, d], v into the value pages [page, kv_head, dv, slot];
//   sigmoid_gate    out[t, c] *= sigmoid(gate[t, c / group]): the output gate of the heads, a value a column or one a head;
//   axpby           out = alpha * a + beta * b over float32 rows: sums of sublayer outputs and the scaled residual add,
//                   optionally followed by the RMS norm of the new rows (the next layer's input) in the same pass;
//   activation      out = act(x) elementwise: exact (erf) gelu, tanh gelu, silu, relu.
#include "common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void qkv_norm_prep_kernel(T* __restrict__ qkv, int row_stride, int nq, int nkv, int d, int dv,
                                                            const float* __restrict__ q_weight, const float* __restrict__ k_weight,
                                                            float eps, const float* __restrict__ cosv, const float* __restrict__ sinv,
                                                            int rot_half, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                            const int* __restrict__ slots, int page_size) {
  __shared__ float scratch[16];
  const int token = blockIdx.x, tid = threadIdx.x;
  T* row = qkv + (int64_t)token * row_stride;
  const int qn = nq * d, kn = nkv * d, vn = nkv * dv;
  float ssq = 0.f, ssk = 0.f;
  for (int e = tid; e < qn; e += 256) {
    const float x = to_float(row[e]);
    ssq = fmaf(x, x, ssq);
  }
  for (int e = tid; e < kn; e += 256) {
    const float x = to_float(row[qn + e]);
    ssk = fmaf(x, x, ssk);
  }
  ssq = block_sum(ssq, scratch);
  ssk = block_sum(ssk, scratch);
  const float inv_q = q_weight ? 1.0f / sqrtf(ssq / (float)qn + eps) : 1.f;
  const float inv_k = k_weight ? 1.0f / sqrtf(ssk / (float)kn + eps) : 1.f;
  const int slot = slots ? slots[token] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const float* cosrow = cosv + (int64_t)token * rot_half;
  const float* sinrow = sinv + (int64_t)token * rot_half;
  // a head's work items: item j < rot_half is the pair (j, j + rot_half), item j >= rot_half the single dim j + rot_half;
  // no two items touch the same value, so q can be written where it was read
  const int items = d - rot_half;
  for (int w = tid; w < (nq + nkv) * items; w += 256) {
    const int head = w / items, j = w % items;
    const bool is_q = head < nq;
    if (!is_q && slot < 0) continue;
    const T* src = row + (int64_t)head * d;
    const float* weight = is_q ? q_weight : k_weight;
    const int wbase = (is_q ? head : head - nq) * d;
    const float inv = is_q ? inv_q : inv_k;
    T* dst = is_q ? row + (int64_t)head * d : k_pages + ((page * nkv + (head - nq)) * page_size + off) * d;
    if (j < rot_half) {
      float a = to_float(src[j]) * inv, b = to_float(src[j + rot_half]) * inv;
      if (weight) {
        a *= weight[wbase + j];
        b *= weight[wbase + j + rot_half];
      }
      const float c = cosrow[j], s = sinrow[j];
      dst[j] = from_float<T>(a * c - b * s);
      dst[j + rot_half] = from_float<T>(b * c + a * s);
    } else {
      const int i = j + rot_half;
      float a = to_float(src[i]) * inv;
      if (weight) a *= weight[wbase + i];
      dst[i] = from_float<T>(a);
    }
  }
  if (slot >= 0) {
    for (int e = tid; e < vn; e += 256) {
      const int kvh = e / dv, i = e % dv;
      v_pages[((page * nkv + kvh) * dv + i) * page_size + off] = row[qn + kn + e];
    }
  }
}

// The same in bfloat16 for heads whose size and rotated half are multiples of eight and rows of q and k of up to 8,192 values:
// 16 bytes a load, a work item is a run of eight dims (with its partner eight of the other half where the head is rotated
// there), and the rows stay in registers between the sums of squares and the norms.
constexpr int PREP_ITEMS = 4;       // work items a thread holds

__global__ __launch_bounds__(256) void qkv_norm_prep_vec_kernel(bf16* __restrict__ qkv, int row_stride, int nq, int nkv, int d, int dv,
                                                                const float* __restrict__ q_weight, const float* __restrict__ k_weight,
                                                                float eps, const float* __restrict__ cosv, const float* __restrict__ sinv,
                                                                int rot_half, bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                                                                const int* __restrict__ slots, int page_size) {
  __shared__ float scratch[16];
  const int token = blockIdx.x, tid = threadIdx.x;
  bf16* row = qkv + (int64_t)token * row_stride;
  const int qn = nq * d, kn = nkv * d, vn = nkv * dv;
  const int rot8 = rot_half / 8, items = (d - rot_half) / 8, total = (nq + nkv) * items;
  bf16x8 lo[PREP_ITEMS], hi[PREP_ITEMS];
  float ssq = 0.f, ssk = 0.f;
#pragma unroll
  for (int n = 0; n < PREP_ITEMS; ++n) {
    const int w = tid + n * 256;
    if (w < total) {
      const int head = w / items, j = w % items;
      const bf16* src = row + (int64_t)head * d;
      const bool paired = j < rot8;
      lo[n] = *(const bf16x8*)(src + (paired ? j * 8 : j * 8 + rot_half));
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) ss = fmaf((float)lo[n][i], (float)lo[n][i], ss);
      if (paired) {
        hi[n] = *(const bf16x8*)(src + j * 8 + rot_half);
#pragma unroll
        for (int i = 0; i < 8; ++i) ss = fmaf((float)hi[n][i], (float)hi[n][i], ss);
      }
      if (head < nq) ssq += ss;
      else ssk += ss;
    }
  }
  ssq = block_sum(ssq, scratch);
  ssk = block_sum(ssk, scratch);
  const float inv_q = q_weight ? 1.0f / sqrtf(ssq / (float)qn + eps) : 1.f;
  const float inv_k = k_weight ? 1.0f / sqrtf(ssk / (float)kn + eps) : 1.f;
  const int slot = slots ? slots[token] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const float* cosrow = cosv + (int64_t)token * rot_half;
  const float* sinrow = sinv + (int64_t)token * rot_half;
#pragma unroll
  for (int n = 0; n < PREP_ITEMS; ++n) {
    const int w = tid + n * 256;
    if (w >= total) continue;
    const int head = w / items, j = w % items;
    const bool is_q = head < nq;
    if (!is_q && slot < 0) continue;
    const float* weight = is_q ? q_weight : k_weight;
    const int wbase = (is_q ? head : head - nq) * d;
    const float inv = is_q ? inv_q : inv_k;
    bf16* dst = is_q ? row + (int64_t)head * d : k_pages + ((page * nkv + (head - nq)) * page_size + off) * d;
    const floatx4 one4 = {1.f, 1.f, 1.f, 1.f};
    if (j < rot8) {
      // weights and angles of the eight pairs, 16 bytes a load, all asked for before any is used
      floatx4 wa[2], wb[2], c4[2], s4[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        wa[half] = weight ? *(const floatx4*)(weight + wbase + j * 8 + half * 4) : one4;
        wb[half] = weight ? *(const floatx4*)(weight + wbase + j * 8 + rot_half + half * 4) : one4;
        c4[half] = *(const floatx4*)(cosrow + j * 8 + half * 4);
        s4[half] = *(const floatx4*)(sinrow + j * 8 + half * 4);
      }
      bf16x8 first, second;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float a = (float)lo[n][i] * inv * wa[i / 4][i % 4], b = (float)hi[n][i] * inv * wb[i / 4][i % 4];
        const float c = c4[i / 4][i % 4], sn = s4[i / 4][i % 4];
        first[i] = (bf16)(a * c - b * sn);
        second[i] = (bf16)(b * c + a * sn);
      }
      *(bf16x8*)(dst + j * 8) = first;
      *(bf16x8*)(dst + j * 8 + rot_half) = second;
    } else {
      const int at = j * 8 + rot_half;
      floatx4 wa[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) wa[half] = weight ? *(const floatx4*)(weight + wbase + at + half * 4) : one4;
      bf16x8 only;
#pragma unroll
      for (int i = 0; i < 8; ++i) only[i] = (bf16)((float)lo[n][i] * inv * wa[i / 4][i % 4]);
      *(bf16x8*)(dst + at) = only;
    }
  }
  if (slot >= 0) {
    for (int e = tid; e < vn; e += 256) {
      const int kvh = e / dv, i = e % dv;
      v_pages[((page * nkv + kvh) * dv + i) * page_size + off] = row[qn + kn + e];
    }
  }
}

template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ out, int out_stride, const T* __restrict__ gate, int gate_stride, int rows, int cols,
                                    int group) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (int64_t)rows * cols) return;
  const int64_t r = e / cols, c = e % cols;
  const float g = to_float(gate[r * gate_stride + c / group]);     // one gate value for every `group` neighbouring columns
  T* o = out + r * out_stride + c;
  *o = from_float<T>(to_float(*o) / (1.f + expf(-g)));
}

__global__ void axpby_kernel(float* __restrict__ out, const float* __restrict__ a, float alpha, const float* __restrict__ b, float beta,
                             int64_t count) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e < count) out[e] = alpha * a[e] + beta * b[e];
}

// out = alpha * a + beta * b for one row a workgroup, and the row's RMS norm times a weight beside it.
template <typename TN>
__global__ __launch_bounds__(256) void axpby_norm_kernel(float* __restrict__ out, const float* __restrict__ a, float alpha,
                                                         const float* __restrict__ b, float beta, int cols,
                                                         const float* __restrict__ norm_weight, float eps, TN* __restrict__ normed) {
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * cols;
  float ss = 0.f;
  for (int c = threadIdx.x; c < cols; c += 256) {
    const float v = alpha * a[base + c] + beta * b[base + c];
    out[base + c] = v;
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)cols + eps);
  for (int c = threadIdx.x; c < cols; c += 256) normed[base + c] = from_float<TN>(out[base + c] * inv * norm_weight[c]);
}

// The same for rows of up to 8,192 values, a multiple of four: 16 bytes a load, the row stays in registers between the sum of
// squares and the norm, and every load is on its way before the first is used.
template <typename TN>
__global__ __launch_bounds__(256) void axpby_norm_vec_kernel(float* __restrict__ out, const float* __restrict__ a, float alpha,
                                                             const float* __restrict__ b, float beta, int cols,
                                                             const float* __restrict__ norm_weight, float eps, TN* __restrict__ normed) {
  constexpr int PER = 8;
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * cols;
  const int quads = cols / 4;
  floatx4 va[PER], vb[PER], w[PER];
#pragma unroll
  for (int n = 0; n < PER; ++n) {
    const int q = threadIdx.x + n * 256;
    if (q < quads) {
      va[n] = *(const floatx4*)(a + base + 4 * q);
      vb[n] = *(const floatx4*)(b + base + 4 * q);
      w[n] = *(const floatx4*)(norm_weight + 4 * q);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int n = 0; n < PER; ++n) {
    const int q = threadIdx.x + n * 256;
    if (q < quads) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        va[n][i] = alpha * va[n][i] + beta * vb[n][i];
        ss = fmaf(va[n][i], va[n][i], ss);
      }
      *(floatx4*)(out + base + 4 * q) = va[n];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)cols + eps);
#pragma unroll
  for (int n = 0; n < PER; ++n) {
    const int q = threadIdx.x + n * 256;
    if (q < quads) {
      TN packed[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) packed[i] = from_float<TN>(va[n][i] * inv * w[n][i]);
      if constexpr (sizeof(TN) == 4) *(floatx4*)(normed + base + 4 * q) = *(const floatx4*)packed;
      else *(uint64_t*)(normed + base + 4 * q) = *(const uint64_t*)packed;
    }
  }
}

enum { ACT_GELU_ERF = 0, ACT_GELU_TANH = 1, ACT_SILU = 2, ACT_RELU = 3 };

__device__ __forceinline__ float activate(float x, int kind) {
  switch (kind) {
    case ACT_GELU_ERF: return 0.5f * x * (1.f + erff(x * 0.70710678118654752f));
    case ACT_GELU_TANH: return 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
    case ACT_SILU: return x / (1.f + expf(-x));
    default: return fmaxf(x, 0.f);
  }
}

template <typename T>
__global__ void activation_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t count, int kind) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e < count) out[e] = from_float<T>(activate(to_float(x[e]), kind));
}

}  // namespace

// qkv [tokens, row_stride] in dtype: q (nq*d) | k (nkv*d) | v (nkv*dv) | anything else.  q_weight [nq*d], k_weight [nkv*d]
// float32 (both null: no norm).  cos, sin [tokens, rot_half] float32.  slots[t] = page * page_size + offset (negative: the
// token's key and value are not stored).
LRS_API int lrs_qkv_norm_prep(void* qkv, int dtype, int tokens, int row_stride, int nq, int nkv, int d, int dv, const float* q_weight,
                              const float* k_weight, float eps, const float* cosv, const float* sinv, int rot_half, void* k_pages,
                              void* v_pages, const int* slots, int page_size, void* stream) {
  LRS_REQUIRE(tokens > 0 && nq > 0 && nkv > 0 && d > 0 && dv > 0, "qkv_norm_prep: bad sizes tokens=%d nq=%d nkv=%d d=%d dv=%d", tokens, nq, nkv, d, dv);
  LRS_REQUIRE(row_stride >= nq * d + nkv * d + nkv * dv, "qkv_norm_prep: rows of %d hold fewer than q, k and v", row_stride);
  LRS_REQUIRE(rot_half >= 0 && 2 * rot_half <= d, "qkv_norm_prep: rotary width %d exceeds head_dim %d", 2 * rot_half, d);
  LRS_REQUIRE(rot_half == 0 || (cosv && sinv), "qkv_norm_prep: rotation asked for without tables");
  LRS_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "qkv_norm_prep: q and k norm weights must come together");
  LRS_REQUIRE(!q_weight || eps > 0.f, "qkv_norm_prep: eps must be positive");
  LRS_REQUIRE(k_pages && v_pages && slots && page_size > 0, "qkv_norm_prep: cache write needs pages, slots and a page size");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_F32)
    qkv_norm_prep_kernel<float><<<tokens, 256, 0, s>>>((float*)qkv, row_stride, nq, nkv, d, dv, q_weight, k_weight, eps, cosv, sinv, rot_half,
                                                       (float*)k_pages, (float*)v_pages, slots, page_size);
  else if (dtype == LRS_BF16 && d % 8 == 0 && rot_half % 8 == 0 && row_stride % 8 == 0 &&
           ((uintptr_t)qkv | (uintptr_t)q_weight | (uintptr_t)k_weight | (uintptr_t)cosv | (uintptr_t)sinv) % 16 == 0 &&
           (nq + nkv) * (d - rot_half) / 8 <= 256 * PREP_ITEMS)
    qkv_norm_prep_vec_kernel<<<tokens, 256, 0, s>>>((bf16*)qkv, row_stride, nq, nkv, d, dv, q_weight, k_weight, eps, cosv, sinv, rot_half,
                                                    (bf16*)k_pages, (bf16*)v_pages, slots, page_size);
  else if (dtype == LRS_BF16)
    qkv_norm_prep_kernel<bf16><<<tokens, 256, 0, s>>>((bf16*)qkv, row_stride, nq, nkv, d, dv, q_weight, k_weight, eps, cosv, sinv, rot_half,
                                                      (bf16*)k_pages, (bf16*)v_pages, slots, page_size);
  else return lrs_fail("qkv_norm_prep: unknown dtype %d", dtype);
  return lrs_check_launch("qkv_norm_prep");
}

LRS_API int lrs_sigmoid_gate(void* out, int out_stride, const void* gate, int gate_stride, int dtype, int rows, int cols, int group, void* stream) {
  LRS_REQUIRE(rows > 0 && cols > 0 && group > 0 && cols % group == 0 && out_stride >= cols && gate_stride >= cols / group,
              "sigmoid_gate: bad sizes rows=%d cols=%d group=%d", rows, cols, group);
  const int64_t count = (int64_t)rows * cols;
  const unsigned blocks = (unsigned)((count + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_F32) sigmoid_gate_kernel<float><<<blocks, 256, 0, s>>>((float*)out, out_stride, (const float*)gate, gate_stride, rows, cols, group);
  else if (dtype == LRS_BF16) sigmoid_gate_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)out, out_stride, (const bf16*)gate, gate_stride, rows, cols, group);
  else return lrs_fail("sigmoid_gate: unknown dtype %d", dtype);
  return lrs_check_launch("sigmoid_gate");
}

// out = alpha * a + beta * b, float32 [rows, cols] contiguous (out may be a or b).  norm_weight given: normed [rows, cols] in
// normed_dtype receives out / sqrt(mean(out^2) + eps) * norm_weight as well.
LRS_API int lrs_axpby(float* out, const float* a, float alpha, const float* b, float beta, int rows, int cols, const float* norm_weight,
                      float eps, void* normed, int normed_dtype, void* stream) {
  LRS_REQUIRE(rows > 0 && cols > 0, "axpby: bad sizes rows=%d cols=%d", rows, cols);
  hipStream_t s = (hipStream_t)stream;
  if (norm_weight == nullptr) {
    const int64_t count = (int64_t)rows * cols;
    axpby_kernel<<<(unsigned)((count + 255) / 256), 256, 0, s>>>(out, a, alpha, b, beta, count);
  } else {
    LRS_REQUIRE(normed && eps > 0.f, "axpby: the norm needs a buffer and a positive eps");
    const bool vec = cols % 4 == 0 && cols <= 8192 && ((uintptr_t)out | (uintptr_t)a | (uintptr_t)b | (uintptr_t)norm_weight | (uintptr_t)normed) % 16 == 0;
    if (normed_dtype == LRS_F32 && vec) axpby_norm_vec_kernel<float><<<rows, 256, 0, s>>>(out, a, alpha, b, beta, cols, norm_weight, eps, (float*)normed);
    else if (normed_dtype == LRS_BF16 && vec) axpby_norm_vec_kernel<bf16><<<rows, 256, 0, s>>>(out, a, alpha, b, beta, cols, norm_weight, eps, (bf16*)normed);
    else if (normed_dtype == LRS_F32) axpby_norm_kernel<float><<<rows, 256, 0, s>>>(out, a, alpha, b, beta, cols, norm_weight, eps, (float*)normed);
    else if (normed_dtype == LRS_BF16) axpby_norm_kernel<bf16><<<rows, 256, 0, s>>>(out, a, alpha, b, beta, cols, norm_weight, eps, (bf16*)normed);
    else return lrs_fail("axpby: unknown dtype %d", normed_dtype);
  }
  return lrs_check_launch("axpby");
}

LRS_API int lrs_activation(void* out, const void* x, int dtype, int64_t count, int kind, void* stream) {
  LRS_REQUIRE(count > 0 && kind >= 0 && kind <= 3, "activation: bad arguments count=%lld kind=%d", (long long)count, kind);
  const unsigned blocks = (unsigned)((count + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_F32) activation_kernel<float><<<blocks, 256, 0, s>>>((float*)out, (const float*)x, count, kind);
  else if (dtype == LRS_BF16) activation_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)out, (const bf16*)x, count, kind);
  else return lrs_fail("activation: unknown dtype %d", dtype);
  return lrs_check_launch("activation");
}

// Kernels of blocks whose sublayers run side by side on the same input, and of attention whose projections carry
// biases and are normed as a whole.
//
//   scaled_sum_norm   stream' = stream + mult * sum_i scale_i (.) term_i, then up to two RMS norms of stream' with
//                     weights of their own (the inputs of the next layer's two sublayers), one pass over the row
//   softcap           z <- cap * tanh(z / cap), in place, float32
//   qkv_prepare       per token, on the unrounded sums of the packed q/k/v product: + bias; RMS norm of all query
//                     rows at once and of all key rows at once; a query temperature that grows with the logarithm of
//                     the position; values blended with those an earlier layer made for the same token; keys and
//                     values into their pages, queries out in the compute dtype
//
// Sums, norms, temperatures and the blend are float32; every stored value is rounded once.
#include "common.h"

#define PS_MAX_TERMS 4

struct SumTerms {
  const void* ptr[PS_MAX_TERMS];       // [parts, T, n]
  const float* scale[PS_MAX_TERMS];    // [n] or null (1)
  int64_t part_stride[PS_MAX_TERMS];
  int parts[PS_MAX_TERMS];
  int dtype[PS_MAX_TERMS];
  int count;
};

// One element of a term: its partial sums added in order, times the term's scale.
__device__ __forceinline__ float term_value(const void* ptr, int dtype, int parts, int64_t stride, const float* scale,
                                            int64_t at, int i) {
  float v = 0.f;
  if (dtype == ME_F32) {
    const float* p = (const float*)ptr + at;
    for (int q = 0; q < parts; ++q) v += p[q * stride];
  } else {
    const bf16_t* p = (const bf16_t*)ptr + at;
    for (int q = 0; q < parts; ++q) v += static_cast<float>(p[q * stride]);
  }
  return scale ? scale[i] * v : v;
}

// The same for 4 neighbours (16-byte loads where the term is float32).
__device__ __forceinline__ void term_value4(const void* ptr, int dtype, int parts, int64_t stride, const float* scale,
                                            int64_t at, int i, float (&out)[4]) {
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (dtype == ME_F32) {
    const float* p = (const float*)ptr + at;
    for (int q = 0; q < parts; ++q) {
      const float4 t = *reinterpret_cast<const float4*>(p + q * stride);
      v[0] += t.x; v[1] += t.y; v[2] += t.z; v[3] += t.w;
    }
  } else {
    const bf16_t* p = (const bf16_t*)ptr + at;
    for (int q = 0; q < parts; ++q) {
      const bf16x4 t = *reinterpret_cast<const bf16x4*>(p + q * stride);
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] += static_cast<float>(t[j]);
    }
  }
  float4 sc = make_float4(1.f, 1.f, 1.f, 1.f);
  if (scale) sc = *reinterpret_cast<const float4*>(scale + i);
  out[0] += sc.x * v[0]; out[1] += sc.y * v[1]; out[2] += sc.z * v[2]; out[3] += sc.w * v[3];
}

// One workgroup per row; the row stays in LDS between the sum and the norms. The terms are walked by a loop that the
// compiler unrolls, so that their pointers stay in scalar registers. VEC: rows in whole groups of 4 with every operand
// 16-byte aligned: a thread takes 4 neighbours at a time.
template <typename TY, bool VEC>
__global__ void __launch_bounds__(1024)
scaled_sum_norm_kernel(const void* __restrict__ stream_in, int stream_dtype, SumTerms terms, float mult,
                       float* __restrict__ stream_out, const float* __restrict__ w1, const float* __restrict__ w2,
                       TY* __restrict__ y1, TY* __restrict__ y2, int n, float eps) {
  __shared__ float scratch[16];
  extern __shared__ __align__(16) float row[];
  const int64_t t = blockIdx.x;
  float ss = 0.f;
  if constexpr (VEC) {
    for (int i = threadIdx.x * 4; i < n; i += blockDim.x * 4) {
      const int64_t at = t * n + i;
      float add[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k = 0; k < PS_MAX_TERMS; ++k)
        if (k < terms.count) term_value4(terms.ptr[k], terms.dtype[k], terms.parts[k], terms.part_stride[k], terms.scale[k], at, i, add);
      float base[4];
      if (stream_dtype == ME_F32) {
        const float4 b = *reinterpret_cast<const float4*>((const float*)stream_in + at);
        base[0] = b.x; base[1] = b.y; base[2] = b.z; base[3] = b.w;
      } else {
        const bf16x4 b = *reinterpret_cast<const bf16x4*>((const bf16_t*)stream_in + at);
#pragma unroll
        for (int j = 0; j < 4; ++j) base[j] = static_cast<float>(b[j]);
      }
      float s[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s[j] = terms.count ? base[j] + mult * add[j] : base[j];
        ss += s[j] * s[j];
      }
      const float4 out = make_float4(s[0], s[1], s[2], s[3]);
      if (stream_out) *reinterpret_cast<float4*>(stream_out + at) = out;
      *reinterpret_cast<float4*>(row + i) = out;
    }
  } else {
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int64_t at = t * n + i;
      float add = 0.f;
#pragma unroll
      for (int k = 0; k < PS_MAX_TERMS; ++k)
        if (k < terms.count) add += term_value(terms.ptr[k], terms.dtype[k], terms.parts[k], terms.part_stride[k], terms.scale[k], at, i);
      const float base = stream_dtype == ME_F32 ? ((const float*)stream_in)[at] : static_cast<float>(((const bf16_t*)stream_in)[at]);
      const float s = terms.count ? base + mult * add : base;
      if (stream_out) stream_out[at] = s;
      row[i] = s;
      ss += s * s;
    }
  }
  if (!w1) return;
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float u = row[i] * inv;
    y1[t * n + i] = from_f32<TY>(u * w1[i]);
    if (w2) y2[t * n + i] = from_f32<TY>(u * w2[i]);
  }
}

// terms: `count` entries of (pointer, dtype, parts, part stride in elements, scale pointer or null).
extern "C" int me_scaled_sum_norm(const void* stream_in, int stream_dtype, int count, const void* const* term_ptr,
                                  const int* term_dtype, const int* term_parts, const int64_t* term_stride,
                                  const float* const* term_scale, float mult, float* stream_out, const float* w1,
                                  const float* w2, void* y1, void* y2, int out_dtype, int64_t T, int n, float eps,
                                  hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(n >= 1 && n <= 15360, "scaled_sum_norm: width %d outside 1..15360", n);
  ME_CHECK(count >= 0 && count <= PS_MAX_TERMS, "scaled_sum_norm: up to %d terms", PS_MAX_TERMS);
  ME_CHECK(T < (1ll << 31), "scaled_sum_norm: too many rows");
  ME_CHECK(!w2 || w1, "scaled_sum_norm: a second norm needs the first");
  SumTerms terms;
  terms.count = count;
  for (int k = 0; k < PS_MAX_TERMS; ++k) {
    const bool on = k < count;
    terms.ptr[k] = on ? term_ptr[k] : nullptr;
    terms.scale[k] = on ? term_scale[k] : nullptr;
    terms.part_stride[k] = on ? term_stride[k] : 0;
    terms.parts[k] = on ? term_parts[k] : 0;
    terms.dtype[k] = on ? term_dtype[k] : ME_F32;
    ME_CHECK(!on || (terms.parts[k] >= 1 && terms.parts[k] <= 64), "scaled_sum_norm: 1 to 64 partial sums per term");
    ME_CHECK(!on || terms.parts[k] == 1 || terms.dtype[k] == ME_F32, "scaled_sum_norm: partial sums are float32");
  }
  // whole groups of 4 and every operand 16-byte aligned (a bfloat16 group is 8 bytes): the vector form
  uintptr_t bits = reinterpret_cast<uintptr_t>(stream_in) | reinterpret_cast<uintptr_t>(stream_out);
  bool vec = n % 4 == 0;
  for (int k = 0; k < count; ++k) {
    bits |= reinterpret_cast<uintptr_t>(terms.ptr[k]) | reinterpret_cast<uintptr_t>(terms.scale[k]);
    vec = vec && terms.part_stride[k] % 4 == 0;
  }
  vec = vec && bits % 16 == 0;
  // few rows: a row's threads are all the launch has, so as many as its groups fill; many rows: 256
  const int per = vec ? 4 : 1;
  int threads = T >= 512 ? 256 : 1024;
  while (threads > 64 && threads * per / 2 >= n) threads >>= 1;
  const size_t lds = (size_t)n * sizeof(float);
#define PS_LAUNCH(TY, V)                                                                                                   \
  scaled_sum_norm_kernel<TY, V><<<dim3((unsigned)T), dim3(threads), lds, stream>>>(stream_in, stream_dtype, terms, mult, stream_out, \
                                                                                w1, w2, (TY*)y1, (TY*)y2, n, eps)
  if (out_dtype == ME_F32) { if (vec) PS_LAUNCH(float, true); else PS_LAUNCH(float, false); }
  else { if (vec) PS_LAUNCH(bf16_t, true); else PS_LAUNCH(bf16_t, false); }
#undef PS_LAUNCH
  ME_LAUNCH_CHECK();
  return 0;
}

__global__ void softcap_kernel(float* __restrict__ z, int64_t ld, int64_t rows, int n, float cap) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * n) return;
  float* p = z + (i / n) * ld + (i % n);
  *p = cap * tanhf(*p / cap);
}

extern "C" int me_softcap(float* z, int64_t ld, int64_t rows, int n, float cap, hipStream_t stream) {
  if (rows == 0 || n == 0) return 0;
  ME_CHECK(cap > 0.f, "softcap: the cap must be positive");
  const int64_t total = rows * n;
  ME_CHECK((total + 255) / 256 < (1ll << 31), "softcap: too many elements");
  softcap_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream>>>(z, ld, rows, n, cap);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ q/k/v prologue
// rows: float32 [T, (Hq + 2 Hkv) * D], the packed product's sums, heads laid out in D slots each (slots beyond a
// head's stored size hold zeros: zero weight rows, zero bias). One workgroup per token.
//   q: + bias, divided by the root mean square over all `nq` stored query dimensions (zero slots add nothing to the
//      sum of squares), times its weight, times 1 + coef * ln(floor((p + 1) / every) + 1) at position p
//   k: + bias, the same norm over `nk` stored key dimensions, into the page
//   v: + bias; mix 1: the first `vdim` slots of every head are kept in `v_first` [T, Hkv * vdim] float32 for later layers;
//      mix 2: v <- (1 - lambda) v + lambda v_first; into the (transposed) page
// K [pages, Hkv, page, D], V [pages, Hkv, D, page]; slots < 0 are skipped.
template <typename TY>
__global__ void __launch_bounds__(1024)
qkv_prepare_kernel(const float* __restrict__ rows, int64_t row_stride, const float* __restrict__ bias,
                   const float* __restrict__ q_w, const float* __restrict__ k_w, float eps, int nq, int nk,
                   float temp_coef, int temp_every, const int32_t* __restrict__ positions,
                   const int32_t* __restrict__ slots, TY* __restrict__ k_cache, TY* __restrict__ v_cache,
                   TY* __restrict__ q_out, int64_t q_stride, int Hq, int Hkv, int D, int page, int vdim, int mix,
                   const float* __restrict__ lambda, float* __restrict__ v_first, int64_t vf_stride) {
  __shared__ float scratch[16];
  extern __shared__ float held[];          // q slots, then k slots
  const int64_t t = blockIdx.x;
  const float* r = rows + t * row_stride;
  const int wq = Hq * D, wk = Hkv * D;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < wq + wk; i += blockDim.x) {
    const float v = r[i] + (bias ? bias[i] : 0.f);
    held[i] = v;
    if (i < wq) sq += v * v; else sk += v * v;
  }
  float inv_q = 1.f, inv_k = 1.f;
  if (q_w) {
    sq = block_sum(sq, scratch);
    sk = block_sum(sk, scratch);
    inv_q = 1.0f / sqrtf(sq / (float)nq + eps);
    inv_k = 1.0f / sqrtf(sk / (float)nk + eps);
  } else {
    __syncthreads();
  }
  const int p = positions[t];
  const float temp = temp_every > 0 ? 1.f + temp_coef * logf((float)((p + 1) / temp_every) + 1.f) : 1.f;
  for (int i = threadIdx.x; i < wq; i += blockDim.x)
    q_out[t * q_stride + i] = from_f32<TY>(held[i] * inv_q * (q_w ? q_w[i] : 1.f) * temp);
  const int slot = slots[t];
  const int64_t pg = slot >= 0 ? slot / page : 0, off = slot >= 0 ? slot - pg * page : 0;
  if (slot >= 0) {
    for (int i = threadIdx.x; i < wk; i += blockDim.x) {
      const int h = i / D, d = i - h * D;
      k_cache[((pg * Hkv + h) * page + off) * D + d] = from_f32<TY>(held[wq + i] * inv_k * (k_w ? k_w[i] : 1.f));
    }
  }
  const float lam = mix == 2 ? lambda[0] : 0.f;
  // (Writing a group of 8 tokens' values as 16-byte pieces by the workgroup of the group's first token was measured: that
  // workgroup then does eight tokens' work while seven idle, 54 -> 89 us for 2,048 tokens of 8 heads of 128.)
  for (int i = threadIdx.x; i < wk; i += blockDim.x) {
    const int h = i / D, d = i - h * D;
    float v = r[wq + wk + i] + (bias ? bias[wq + wk + i] : 0.f);
    if (mix && d < vdim) {
      float* f = v_first + t * vf_stride + h * vdim + d;
      if (mix == 1) *f = v; else v = (1.f - lam) * v + lam * *f;
    }
    if (slot >= 0) v_cache[((pg * Hkv + h) * D + d) * page + off] = from_f32<TY>(v);
  }
}

extern "C" int me_qkv_prepare(const float* rows, int64_t row_stride, const float* bias, const float* q_w, const float* k_w,
                              float eps, int nq, int nk, float temp_coef, int temp_every, const int32_t* positions,
                              const int32_t* slots, void* k_cache, void* v_cache, void* q_out, int64_t q_stride, int dtype,
                              int64_t T, int Hq, int Hkv, int D, int page, int vdim, int mix, const float* lambda,
                              float* v_first, int64_t vf_stride, hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(Hq >= 1 && Hkv >= 1 && D >= 1 && page >= 1 && T < (1ll << 31), "qkv_prepare: bad sizes");
  ME_CHECK((Hq + Hkv) * (int64_t)D * 4 <= 60 * 1024, "qkv_prepare: %d query and key slots do not fit a workgroup's memory", (Hq + Hkv) * D);
  ME_CHECK((q_w == nullptr) == (k_w == nullptr) && (!q_w || (nq >= 1 && nk >= 1)), "qkv_prepare: both norm weights with their sizes, or neither");
  ME_CHECK(mix >= 0 && mix <= 2 && (!mix || (v_first && vdim >= 1 && vdim <= D)) && (mix != 2 || lambda), "qkv_prepare: bad value mixing");
  ME_CHECK(temp_every >= 0, "qkv_prepare: bad temperature period");
  const size_t lds = (size_t)(Hq + Hkv) * D * sizeof(float);
  // few tokens: a token's threads are all the launch has
  int threads = T >= 512 ? 256 : 1024;
  while (threads > 64 && threads / 2 >= (Hq + Hkv) * D) threads >>= 1;
  if (dtype == ME_F32)
    qkv_prepare_kernel<float><<<dim3((unsigned)T), dim3(threads), lds, stream>>>(
        rows, row_stride, bias, q_w, k_w, eps, nq, nk, temp_coef, temp_every, positions, slots, (float*)k_cache, (float*)v_cache,
        (float*)q_out, q_stride, Hq, Hkv, D, page, vdim, mix, lambda, v_first, vf_stride);
  else
    qkv_prepare_kernel<bf16_t><<<dim3((unsigned)T), dim3(threads), lds, stream>>>(
        rows, row_stride, bias, q_w, k_w, eps, nq, nk, temp_coef, temp_every, positions, slots, (bf16_t*)k_cache, (bf16_t*)v_cache,
        (bf16_t*)q_out, q_stride, Hq, Hkv, D, page, vdim, mix, lambda, v_first, vf_stride);
  ME_LAUNCH_CHECK();
  return 0;
}

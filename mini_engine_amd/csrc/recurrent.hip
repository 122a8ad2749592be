// Kernels of the mixers that keep a fixed-size state per request (linear attention with a decay, selective
// state-space layers), of blocks whose norms sit on the sublayers' outputs, and a few elementwise helpers.
//
//   add_rms_norm      stream += w * y / rms(y)                      (float32 stream, rounded copy for the next product)
//   activation        silu / squared relu of a row view
//   head_gate         o[t, h, :] *= sigmoid(g[t, h])
//   causal_conv       short causal convolution per channel over a request's tokens, continued from its state, + silu
//   recurrence        S_t = a_t S_(t-1) + b_t k_t v_t^T,  y_t = S_t^T q_t (+ skip v_t): float32 state per head
//   gated_rms_norm    unit root mean square per group with a gate in front of or behind it
//
// Everything that enters a recurrence is float32: step sizes, decays, their exponentials, the state, the sums.
#include "common.h"

#define RC_MAX_PARTIALS 8

// ------------------------------------------------------------------ stream += w * y / rms(y)
// One workgroup per row. y may be `parts` stacked float32 partial sums, added here in a fixed order.
template <typename TX, typename TY>
__global__ void add_rms_norm_kernel(const TX* __restrict__ y, int parts, int64_t part_stride, const float* __restrict__ w,
                                    const float* __restrict__ stream_in, float* __restrict__ stream_out,
                                    TY* __restrict__ rounded, int n, float eps) {
  __shared__ float scratch[16];
  extern __shared__ float row[];
  const int64_t t = blockIdx.x;
  const TX* yr = y + t * n;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += to_f32<TX>(yr[p * part_stride + i]);
    row[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float s = stream_in[t * n + i] + row[i] * inv * w[i];
    stream_out[t * n + i] = s;
    if (rounded) rounded[t * n + i] = from_f32<TY>(s);
  }
}

extern "C" int me_add_rms_norm(const void* y, int y_dtype, int parts, int64_t part_stride, const float* w,
                               const float* stream_in, float* stream_out, void* rounded, int64_t T, int n, float eps,
                               hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(n >= 1 && n <= 15360, "add_rms_norm: width %d outside 1..15360", n);
  ME_CHECK(parts >= 1 && parts <= RC_MAX_PARTIALS && (parts == 1 || y_dtype == ME_F32), "add_rms_norm: up to %d float32 partial sums", RC_MAX_PARTIALS);
  const dim3 grid((unsigned)T), block(n >= 1024 ? 256 : (n > 256 ? 128 : 64));
  const size_t lds = (size_t)n * sizeof(float);
  if (y_dtype == ME_F32)
    add_rms_norm_kernel<float, float><<<grid, block, lds, stream>>>((const float*)y, parts, part_stride, w, stream_in, stream_out,
                                                                    (float*)nullptr, n, eps);
  else
    add_rms_norm_kernel<bf16_t, bf16_t><<<grid, block, lds, stream>>>((const bf16_t*)y, parts, part_stride, w, stream_in,
                                                                      stream_out, (bf16_t*)rounded, n, eps);
  ME_LAUNCH_CHECK();
  return 0;
}

// float32 partial sums with a bfloat16 rounded copy (products split over K on the bfloat16 path)
extern "C" int me_add_rms_norm_partials(const float* y, int parts, int64_t part_stride, const float* w, const float* stream_in,
                                        float* stream_out, void* rounded, int64_t T, int n, float eps, hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(n >= 1 && n <= 15360, "add_rms_norm: width %d outside 1..15360", n);
  ME_CHECK(parts >= 1 && parts <= RC_MAX_PARTIALS, "add_rms_norm: up to %d partial sums", RC_MAX_PARTIALS);
  const dim3 grid((unsigned)T), block(n >= 1024 ? 256 : (n > 256 ? 128 : 64));
  add_rms_norm_kernel<float, bf16_t><<<grid, block, (size_t)n * sizeof(float), stream>>>(y, parts, part_stride, w, stream_in,
                                                                                        stream_out, (bf16_t*)rounded, n, eps);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ activations
__device__ __forceinline__ float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float silu_f(float v) { return v * sigmoid_f(v); }

template <typename TX, int KIND>
__global__ void activation_kernel(const TX* __restrict__ x, int64_t x_stride, TX* __restrict__ out, int64_t T, int n) {
  const int64_t total = T * n;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / n;
    const float v = to_f32<TX>(x[t * x_stride + (i - t * n)]);
    float r;
    if (KIND == 0) r = silu_f(v);
    else { const float p = fmaxf(v, 0.f); r = p * p; }
    out[i] = from_f32<TX>(r);
  }
}

extern "C" int me_activation(const void* x, int64_t x_stride, void* out, int dtype, int kind, int64_t T, int n, hipStream_t stream) {
  if (T == 0 || n == 0) return 0;
  ME_CHECK(kind == 0 || kind == 1, "activation: unknown kind %d", kind);
  const int64_t total = T * n;
  const dim3 grid((unsigned)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535)), block(256);
#define ACT(TX, K) activation_kernel<TX, K><<<grid, block, 0, stream>>>((const TX*)x, x_stride, (TX*)out, T, n)
  if (dtype == ME_F32) { if (kind == 0) ACT(float, 0); else ACT(float, 1); }
  else { if (kind == 0) ACT(bf16_t, 0); else ACT(bf16_t, 1); }
#undef ACT
  ME_LAUNCH_CHECK();
  return 0;
}

// o[t, h, :] *= sigmoid(g[t, h]); o contiguous [T, H * D], g a view with token stride g_stride.
template <typename TX>
__global__ void head_gate_kernel(TX* __restrict__ o, const TX* __restrict__ g, int64_t g_stride, int64_t T, int H, int D) {
  const int64_t total = T * H * D;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t th = i / D;
    const int64_t t = th / H;
    const int h = (int)(th - t * H);
    o[i] = from_f32<TX>(to_f32<TX>(o[i]) * sigmoid_f(to_f32<TX>(g[t * g_stride + h])));
  }
}

extern "C" int me_head_gate(void* o, const void* g, int64_t g_stride, int dtype, int64_t T, int H, int D, hipStream_t stream) {
  if (T == 0) return 0;
  const int64_t total = T * H * D;
  const dim3 grid((unsigned)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535)), block(256);
  if (dtype == ME_F32) head_gate_kernel<float><<<grid, block, 0, stream>>>((float*)o, (const float*)g, g_stride, T, H, D);
  else head_gate_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)o, (const bf16_t*)g, g_stride, T, H, D);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ short causal convolution + silu
// out[t, c] = silu(bias[c] + sum_j w[c, j] * in(t - (taps - 1) + j)); the inputs before the step's first token of a
// request come from its state row: per channel taps - 1 values, oldest first. One thread per (token, channel).
#define CONV_MAX_TAPS 16

template <typename TX>
__global__ void causal_conv_kernel(const TX* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                   const float* __restrict__ bias, const float* __restrict__ state, int64_t state_stride,
                                   const int32_t* __restrict__ slots, const int32_t* __restrict__ cu,
                                   const int32_t* __restrict__ seq_of_token, TX* __restrict__ out, int C, int taps) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = seq_of_token[t];
  const int64_t first = cu[b];
  const int local = (int)(t - first);
  const float* held = state + (int64_t)slots[b] * state_stride + (int64_t)c * (taps - 1);
  float acc = bias[c];
  for (int j = 0; j < taps; ++j) {
    const int src = local - (taps - 1) + j;
    const float v = src >= 0 ? to_f32<TX>(x[(first + src) * x_stride + c]) : held[src + taps - 1];
    acc += w[(int64_t)c * taps + j] * v;
  }
  out[t * C + c] = from_f32<TX>(silu_f(acc));
}

// The state moves on: per (request, channel) the last taps - 1 inputs of (held inputs, this step's inputs).
template <typename TX>
__global__ void causal_conv_state_kernel(const TX* __restrict__ x, int64_t x_stride, float* __restrict__ state,
                                         int64_t state_stride, const int32_t* __restrict__ slots,
                                         const int32_t* __restrict__ cu, int C, int taps) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int64_t first = cu[b];
  const int n = (int)(cu[b + 1] - first);
  if (n <= 0) return;
  float* held = state + (int64_t)slots[b] * state_stride + (int64_t)c * (taps - 1);
  float next[CONV_MAX_TAPS];
  for (int s = 0; s < taps - 1; ++s) {
    const int src = n - (taps - 1) + s;
    next[s] = src >= 0 ? to_f32<TX>(x[(first + src) * x_stride + c]) : held[src + taps - 1];
  }
  for (int s = 0; s < taps - 1; ++s) held[s] = next[s];
}

extern "C" int me_causal_conv(const void* x, int64_t x_stride, int dtype, const float* w, const float* bias, float* state,
                              int64_t state_stride, const int32_t* slots, const int32_t* cu, const int32_t* seq_of_token,
                              void* out, int64_t T, int num_seqs, int C, int taps, hipStream_t stream) {
  if (T == 0 || C == 0) return 0;
  ME_CHECK(taps >= 1 && taps <= CONV_MAX_TAPS, "causal_conv: %d taps outside 1..%d", taps, CONV_MAX_TAPS);
  const dim3 block(C >= 256 ? 256 : 64);
  ME_CHECK(T <= 2147483647ll && num_seqs <= 65535 && (C + block.x - 1) / block.x <= 65535,
           "causal_conv: too many tokens, requests or channels for one launch");
  const dim3 grid((unsigned)T, (C + block.x - 1) / block.x);
  if (dtype == ME_F32)
    causal_conv_kernel<float><<<grid, block, 0, stream>>>((const float*)x, x_stride, w, bias, state, state_stride, slots, cu,
                                                          seq_of_token, (float*)out, C, taps);
  else
    causal_conv_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, x_stride, w, bias, state, state_stride, slots, cu,
                                                           seq_of_token, (bf16_t*)out, C, taps);
  ME_LAUNCH_CHECK();
  if (taps > 1) {
    const dim3 sgrid((C + block.x - 1) / block.x, num_seqs);
    if (dtype == ME_F32)
      causal_conv_state_kernel<float><<<sgrid, block, 0, stream>>>((const float*)x, x_stride, state, state_stride, slots, cu, C, taps);
    else
      causal_conv_state_kernel<bf16_t><<<sgrid, block, 0, stream>>>((const bf16_t*)x, x_stride, state, state_stride, slots, cu, C, taps);
    ME_LAUNCH_CHECK();
  }
  return 0;
}

// ------------------------------------------------------------------ the recurrence
// One wave per (request, head, 64 columns of P, NT rows of N, span of tokens). Lane p keeps column p of its NT state
// rows in registers; the tokens' k and q slices, decays and input scales pass through LDS 16 tokens at a time and
// are read from there by all lanes at once. Products and sums are float32 in the order of the tokens.
//
// A launch is one of three passes (PASS):
//   0  whole: a request's tokens from its state row, y written, the state row written back
//   1  spans, first pass: every span of `span` tokens from zero; its end state and the product of its decays go to
//      scratch (no y)
//   2  spans, last pass: every span from the state that precedes it (the carry kernel has put it into scratch), y
//      written; the span that ends the request's tokens writes the state row
// Between 1 and 2 the carry kernel walks a request's spans in order: in[0] = state row, in[c + 1] = decay[c] * in[c]
// + end[c].
struct RecArgs {
  const void* q; const void* k; const void* v;      // [T, G * N], [T, G * N], [T, H * P] views, token strides below
  int64_t q_stride, k_stride, v_stride;
  const void* dt; int64_t dt_stride;                // [T, H] view, or null: fixed decays
  const float* decay;                               // [H] fixed decays (dt null)
  const float* dt_bias; const float* rate; const float* skip;   // [H] each (skip may be null)
  float* state; int64_t state_stride;               // [slots, H * N * P] view
  const int32_t* slots; const int32_t* cu;
  float* y; int64_t y_slice_stride;                 // [slices of N, T, H * P] float32
  float* span_state; float* span_decay;             // scratch: [requests, spans, H, N, P], [requests, spans, H]
  int H, G, N, P, span, max_spans;
};

#define REC_TB 16

template <typename TX, int NT, int PASS>
__global__ void __launch_bounds__(64) recurrence_kernel(RecArgs a) {
  __shared__ float sk[REC_TB][NT], sq[REC_TB][NT], sa[REC_TB], sb[REC_TB];
  const int lane = threadIdx.x;
  const int bh = blockIdx.x, b = bh / a.H, h = bh - b * a.H;
  const int g = h / (a.H / a.G);
  const int p = blockIdx.y * 64 + lane;
  const int n0 = blockIdx.z % ((a.N + NT - 1) / NT) * NT;
  const int slice = blockIdx.z % ((a.N + NT - 1) / NT);
  const int c = blockIdx.z / ((a.N + NT - 1) / NT);              // span index (0 in pass 0)
  const int64_t first = a.cu[b], end_all = a.cu[b + 1];
  int64_t t0 = first, t1 = end_all;
  if (PASS != 0) {
    t0 = first + (int64_t)c * a.span;
    t1 = t0 + a.span < end_all ? t0 + a.span : end_all;
  }
  if (t0 >= t1) return;
  const bool on = p < a.P;
  const int pc = on ? p : 0;
  float S[NT];
  float* row = a.state + (int64_t)a.slots[b] * a.state_stride + (int64_t)h * a.N * a.P;
  float* span_row = PASS == 0 ? nullptr
                              : a.span_state + (((int64_t)b * a.max_spans + c) * a.H + h) * (int64_t)a.N * a.P;
  if (PASS == 1) {
#pragma unroll
    for (int i = 0; i < NT; ++i) S[i] = 0.f;
  } else {
    const float* from = PASS == 0 ? row : span_row;
#pragma unroll
    for (int i = 0; i < NT; ++i) S[i] = (on && n0 + i < a.N) ? from[(int64_t)(n0 + i) * a.P + pc] : 0.f;
  }
  const TX* qp = (const TX*)a.q + (int64_t)g * a.N + n0;
  const TX* kp = (const TX*)a.k + (int64_t)g * a.N + n0;
  const TX* vp = (const TX*)a.v + (int64_t)h * a.P + pc;
  const float skip = a.skip ? a.skip[h] : 0.f;
  float total_decay = 1.f;
  for (int64_t tb = t0; tb < t1; tb += REC_TB) {
    const int nt = (int)(t1 - tb < REC_TB ? t1 - tb : REC_TB);
    __syncthreads();
    for (int i = lane; i < REC_TB * NT; i += 64) {
      const int tt = i / NT, nn = i - tt * NT;
      const bool have = tt < nt && n0 + nn < a.N;
      sk[tt][nn] = have ? to_f32<TX>(kp[(tb + tt) * a.k_stride + nn]) : 0.f;
      if (PASS != 1) sq[tt][nn] = have ? to_f32<TX>(qp[(tb + tt) * a.q_stride + nn]) : 0.f;
    }
    if (lane < REC_TB) {
      float da = 1.f, db = 0.f;
      if (lane < nt) {
        if (a.dt) {
          const float z = to_f32<TX>(((const TX*)a.dt)[(tb + lane) * a.dt_stride + h]) + a.dt_bias[h];
          const float step = z > 20.f ? z : log1pf(expf(z));
          da = expf(-a.rate[h] * step);
          db = step;
        } else {
          da = a.decay[h];
          db = 1.f;
        }
      }
      sa[lane] = da; sb[lane] = db;
    }
    float vv[REC_TB];
#pragma unroll
    for (int tt = 0; tt < REC_TB; ++tt) vv[tt] = (tt < nt && on) ? to_f32<TX>(vp[(tb + tt) * a.v_stride]) : 0.f;
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float da = sa[tt], bv = sb[tt] * vv[tt];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        S[i] = da * S[i] + sk[tt][i] * bv;
        if (PASS != 1) acc += S[i] * sq[tt][i];
      }
      if (PASS == 1) total_decay *= da;
      else if (on) {
        if (slice == 0) acc += skip * vv[tt];
        a.y[slice * a.y_slice_stride + (tb + tt) * ((int64_t)a.H * a.P) + (int64_t)h * a.P + p] = acc;
      }
    }
  }
  if (PASS == 1) {
    if (on)
#pragma unroll
      for (int i = 0; i < NT; ++i)
        if (n0 + i < a.N) span_row[(int64_t)(n0 + i) * a.P + p] = S[i];
    if (lane == 0 && blockIdx.y == 0 && slice == 0) a.span_decay[((int64_t)b * a.max_spans + c) * a.H + h] = total_decay;
  } else if (on && t1 == end_all) {
#pragma unroll
    for (int i = 0; i < NT; ++i)
      if (n0 + i < a.N) row[(int64_t)(n0 + i) * a.P + p] = S[i];
  }
}

// in[0] = the request's state row; in[c + 1] = decay[c] * in[c] + end[c]. scratch[c] holds end[c] on entry and in[c] on
// exit. One thread per state element, the spans in order.
__global__ void recurrence_carry_kernel(RecArgs a) {
  const int b = blockIdx.y;
  const int64_t per_head = (int64_t)a.N * a.P, per_req = per_head * a.H;
  const int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (e >= per_req) return;
  const int h = (int)(e / per_head);
  const int64_t len = a.cu[b + 1] - a.cu[b];
  const int spans = (int)((len + a.span - 1) / a.span);
  if (spans <= 0) return;
  float carry = a.state[(int64_t)a.slots[b] * a.state_stride + e];
  for (int c = 0; c < spans; ++c) {
    float* at = a.span_state + ((int64_t)b * a.max_spans + c) * per_req + e;
    const float ended = *at;
    *at = carry;
    carry = a.span_decay[((int64_t)b * a.max_spans + c) * a.H + h] * carry + ended;
  }
}

template <typename TX, int NT>
static int launch_recurrence(RecArgs& a, int num_seqs, int spans, hipStream_t stream) {
  const int slices = (a.N + NT - 1) / NT;
  const dim3 block(64);
  if (spans <= 1) {
    recurrence_kernel<TX, NT, 0><<<dim3(num_seqs * a.H, (a.P + 63) / 64, slices), block, 0, stream>>>(a);
    ME_LAUNCH_CHECK();
    return 0;
  }
  const dim3 grid(num_seqs * a.H, (a.P + 63) / 64, slices * spans);
  recurrence_kernel<TX, NT, 1><<<grid, block, 0, stream>>>(a);
  ME_LAUNCH_CHECK();
  const int64_t per_req = (int64_t)a.H * a.N * a.P;
  recurrence_carry_kernel<<<dim3((unsigned)((per_req + 255) / 256), num_seqs), dim3(256), 0, stream>>>(a);
  ME_LAUNCH_CHECK();
  recurrence_kernel<TX, NT, 2><<<grid, block, 0, stream>>>(a);
  ME_LAUNCH_CHECK();
  return 0;
}

// spans <= 1: every request's tokens in one pass. Otherwise the tokens are cut into spans of `span` tokens that run
// side by side (at most `spans` per request), and scratch holds spans * H * N * P + spans * H floats per request.
extern "C" int me_linear_recurrence(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                    int64_t v_stride, int dtype, const void* dt, int64_t dt_stride, const float* decay,
                                    const float* dt_bias, const float* rate, const float* skip, float* state,
                                    int64_t state_stride, const int32_t* slots, const int32_t* cu, float* y,
                                    int64_t y_slice_stride, int num_seqs, int H, int G, int N, int P, int rows_per_wave,
                                    int span, int spans, float* scratch, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  ME_CHECK(H >= 1 && G >= 1 && H % G == 0 && N >= 1 && P >= 1, "recurrence: bad sizes H=%d G=%d N=%d P=%d", H, G, N, P);
  ME_CHECK((dt != nullptr) != (decay != nullptr), "recurrence: give fixed decays or step sizes, not both");
  ME_CHECK(dt == nullptr || (dt_bias && rate), "recurrence: step sizes need their bias and rates");
  ME_CHECK((int64_t)num_seqs * H <= 2147483647ll, "recurrence: too many (request, head) pairs");
  ME_CHECK(spans <= 1 || (span >= 1 && scratch != nullptr), "recurrence: spans need a length and scratch");
  RecArgs a;
  a.q = q; a.k = k; a.v = v; a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride;
  a.dt = dt; a.dt_stride = dt_stride; a.decay = decay; a.dt_bias = dt_bias; a.rate = rate; a.skip = skip;
  a.state = state; a.state_stride = state_stride; a.slots = slots; a.cu = cu; a.y = y; a.y_slice_stride = y_slice_stride;
  a.H = H; a.G = G; a.N = N; a.P = P; a.span = span > 0 ? span : 1; a.max_spans = spans > 1 ? spans : 1;
  a.span_state = scratch;
  a.span_decay = scratch ? scratch + (int64_t)num_seqs * a.max_spans * H * N * P : nullptr;
  const int slices = (N + rows_per_wave - 1) / rows_per_wave;
  ME_CHECK((int64_t)slices * a.max_spans <= 65535, "recurrence: too many slices and spans for one launch");
#define REC(TX)                                                                              \
  switch (rows_per_wave) {                                                                   \
    case 16: return launch_recurrence<TX, 16>(a, num_seqs, spans, stream);                   \
    case 32: return launch_recurrence<TX, 32>(a, num_seqs, spans, stream);                   \
    case 48: return launch_recurrence<TX, 48>(a, num_seqs, spans, stream);                   \
    case 64: return launch_recurrence<TX, 64>(a, num_seqs, spans, stream);                   \
    default: ME_CHECK(false, "recurrence: %d state rows per wave is not one of 16, 32, 48, 64", rows_per_wave); \
  }
  if (dtype == ME_F32) { REC(float) } else { REC(bf16_t) }
#undef REC
  return 0;
}

// ------------------------------------------------------------------ unit rms per group, with a gate
// KIND 0: u = y * silu(gate); out = u / rms_group(u) * w.    KIND 1: out = y / rms_group(y) * w * sigmoid(gate).
// y: `parts` stacked float32 slices [parts, T, n], added here. One workgroup per row.
template <typename TX, int KIND>
__global__ void gated_rms_norm_kernel(const float* __restrict__ y, int parts, int64_t part_stride, const TX* __restrict__ gate,
                                      int64_t gate_stride, const float* __restrict__ w, TX* __restrict__ out, int n,
                                      int groups, float eps) {
  __shared__ float scratch[16];
  extern __shared__ float row[];
  const int64_t t = blockIdx.x;
  const int per = n / groups;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += y[p * part_stride + t * n + i];
    if (KIND == 0) v *= silu_f(to_f32<TX>(gate[t * gate_stride + i]));
    row[i] = v;
  }
  __syncthreads();
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < per; i += blockDim.x) { const float v = row[g * per + i]; ss += v * v; }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)per + eps);
    for (int i = threadIdx.x; i < per; i += blockDim.x) {
      const int j = g * per + i;
      float r = row[j] * inv * w[j];
      if (KIND == 1) r *= sigmoid_f(to_f32<TX>(gate[t * gate_stride + j]));
      out[t * n + j] = from_f32<TX>(r);
    }
  }
}

extern "C" int me_gated_rms_norm(const float* y, int parts, int64_t part_stride, const void* gate, int64_t gate_stride,
                                 int dtype, const float* w, void* out, int64_t T, int n, int groups, int kind, float eps,
                                 hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(n >= 1 && n <= 15360 && groups >= 1 && n % groups == 0, "gated_rms_norm: width %d, %d groups", n, groups);
  ME_CHECK(parts >= 1 && parts <= 64 && (kind == 0 || kind == 1), "gated_rms_norm: bad slice count or kind");
  const dim3 grid((unsigned)T), block(n >= 1024 ? 256 : (n > 256 ? 128 : 64));
  const size_t lds = (size_t)n * sizeof(float);
#define GN(TX, K) gated_rms_norm_kernel<TX, K><<<grid, block, lds, stream>>>(y, parts, part_stride, (const TX*)gate, gate_stride, w, (TX*)out, n, groups, eps)
  if (dtype == ME_F32) { if (kind == 0) GN(float, 0); else GN(float, 1); }
  else { if (kind == 0) GN(bf16_t, 0); else GN(bf16_t, 1); }
#undef GN
  ME_LAUNCH_CHECK();
  return 0;
}

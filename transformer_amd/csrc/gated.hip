// Pieces of a block whose sublayers are gated and whose mixer reads a token-shifted input,
// and of an embedding that adds a hashed row for the pair (previous token, token).
//
//   gated_add_rmsnorm : v = x + mult * sigmoid(gate + gate_bias) * (sum of delta planes + delta_bias),
//                       x = v, out = v / sqrt(mean(v^2) + eps) * weight      (all float32, one rounding)
//   token_shift       : hs_t = h_t + (h_{t-1} - h_t) * mu, h_{-1} from the sequence's state
//   pair_embed_add    : x_t += table[hash(previous token, token)]
//   scale             : t *= s
//
// Per-sequence state (the last row of h, the last token) is read and then written by the
// workgroup of the sequence's FIRST token of the step only, so no other workgroup races it.
#include "common.h"

// sequence that owns token t: the last b with cu_q[b] <= t
__device__ __forceinline__ int seq_of_token(const int* __restrict__ cu_q, int batch, int t) {
  int lo = 0, hi = batch - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x / TA_WAVE;
  __syncthreads();
  if (threadIdx.x % TA_WAVE == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < (int)(blockDim.x / TA_WAVE); ++i) s += red[i];
  return s;
}

template <typename TO>
__global__ __launch_bounds__(256) void gated_add_rmsnorm_kernel(
    float* __restrict__ x, const float* __restrict__ delta, int planes, size_t plane,
    const float* __restrict__ delta_bias, const float* __restrict__ gate,
    const float* __restrict__ gate_bias, float mult, const float* __restrict__ weight,
    const int* __restrict__ rows, TO* __restrict__ out, int d, float eps, int store) {
  extern __shared__ float row[];          // [d]
  __shared__ float red[4];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += 256) {
    const size_t at = r * d + c;
    float v = x[at];
    if (delta) {
      float s = delta[at];
      for (int p = 1; p < planes; ++p) s += delta[at + p * plane];
      if (delta_bias) s += delta_bias[c];
      if (gate) {
        float g = gate[at];
        if (gate_bias) g += gate_bias[c];
        s *= 1.0f / (1.0f + expf(-g));
      }
      v += mult * s;
      if (store) x[at] = v;
    }
    row[c] = v;
    ss += v * v;
  }
  const float f = rsqrtf(block_sum_256(ss, red) / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += 256)
    out[(size_t)i * d + c] = from_f32<TO>(row[c] * f * weight[c]);
}

extern "C" int ta_gated_add_rmsnorm(hipStream_t stream, int out_dtype, float* x, const float* delta,
                                    int planes, long long plane, const float* delta_bias,
                                    const float* gate, const float* gate_bias, float mult,
                                    const float* weight, const int* rows, void* out, int n_out, int d,
                                    float eps, int store) {
  TA_REQUIRE(n_out >= 0 && d > 0 && d <= 16000, "ta_gated_add_rmsnorm: bad sizes n=%d d=%d", n_out, d);
  TA_REQUIRE(planes >= 1 && planes <= TA_MAX_PLANES, "ta_gated_add_rmsnorm: %d planes", planes);
  if (n_out == 0) return 0;
  const size_t lds = (size_t)d * sizeof(float);
  if (out_dtype == TA_F32)
    gated_add_rmsnorm_kernel<float><<<n_out, 256, lds, stream>>>(
        x, delta, planes, (size_t)plane, delta_bias, gate, gate_bias, mult, weight, rows, (float*)out, d, eps, store);
  else if (out_dtype == TA_BF16)
    gated_add_rmsnorm_kernel<bf16_t><<<n_out, 256, lds, stream>>>(
        x, delta, planes, (size_t)plane, delta_bias, gate, gate_bias, mult, weight, rows, (bf16_t*)out, d, eps, store);
  else
    return ta_fail("ta_gated_add_rmsnorm: unknown dtype %d", out_dtype);
  return ta_check_launch("ta_gated_add_rmsnorm");
}

// ------------------------------------------------------------------ token shift
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(
    const T* __restrict__ h, T* __restrict__ hs, const float* __restrict__ mu,
    float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ slots,
    int batch, int d) {
  const int t = blockIdx.x;
  const int b = seq_of_token(cu_q, batch, t);
  const int first = cu_q[b], last = cu_q[b + 1] - 1;
  float* st = state + (size_t)slots[b] * d;
  for (int c = threadIdx.x; c < d; c += 256) {
    const float cur = to_f32(h[(size_t)t * d + c]);
    float prev;
    if (t == first) {
      prev = st[c];
      st[c] = to_f32(h[(size_t)last * d + c]);
    } else {
      prev = to_f32(h[(size_t)(t - 1) * d + c]);
    }
    hs[(size_t)t * d + c] = from_f32<T>(cur + (prev - cur) * mu[c]);
  }
}

// h, hs: [nt, d]; mu: [d]; state: [slots, d] float32, the sequence's last unshifted row.
extern "C" int ta_token_shift(hipStream_t stream, int dtype, const void* h, void* hs, const float* mu,
                              float* state, const int* cu_q, const int* slots, int batch, int nt, int d) {
  TA_REQUIRE(batch > 0 && nt >= batch && d > 0, "ta_token_shift: bad sizes batch=%d nt=%d d=%d", batch, nt, d);
  if (dtype == TA_F32)
    token_shift_kernel<float><<<nt, 256, 0, stream>>>((const float*)h, (float*)hs, mu, state, cu_q, slots, batch, d);
  else if (dtype == TA_BF16)
    token_shift_kernel<bf16_t><<<nt, 256, 0, stream>>>((const bf16_t*)h, (bf16_t*)hs, mu, state, cu_q, slots, batch, d);
  else
    return ta_fail("ta_token_shift: unknown dtype %d", dtype);
  return ta_check_launch("ta_token_shift");
}

// ------------------------------------------------------------------ hashed pair embedding
template <typename T>
__global__ __launch_bounds__(256) void pair_embed_add_kernel(
    float* __restrict__ x, const T* __restrict__ table, const int* __restrict__ tokens,
    int* __restrict__ last_token, const int* __restrict__ cu_q, const int* __restrict__ pos0,
    const int* __restrict__ slots, int batch, int d, int buckets, long long mul_prev, long long mul_cur) {
  const int t = blockIdx.x;
  const int b = seq_of_token(cu_q, batch, t);
  const int first = cu_q[b];
  long long prev;
  if (t == first) {
    prev = pos0[b] == 0 ? -1 : (long long)last_token[slots[b]];
  } else {
    prev = tokens[t - 1];
  }
  const long long rowi = prev < 0 ? (long long)buckets : (prev * mul_prev + (long long)tokens[t] * mul_cur) % buckets;
  const T* src = table + (size_t)rowi * d;
  for (int c = threadIdx.x; c < d; c += 256) x[(size_t)t * d + c] += to_f32(src[c]);
  if (t == first && threadIdx.x == 0) last_token[slots[b]] = tokens[cu_q[b + 1] - 1];
}

// x: [nt, d] float32; table: [buckets + 1, d]; last_token: [slots] int32 state.
extern "C" int ta_pair_embed_add(hipStream_t stream, int dtype, float* x, const void* table,
                                 const int* tokens, int* last_token, const int* cu_q, const int* pos0,
                                 const int* slots, int batch, int nt, int d, int buckets,
                                 long long mul_prev, long long mul_cur) {
  TA_REQUIRE(batch > 0 && nt >= batch && d > 0 && buckets > 0, "ta_pair_embed_add: bad sizes");
  TA_REQUIRE(mul_prev >= 0 && mul_cur >= 0 && mul_prev < (1ll << 31) && mul_cur < (1ll << 31),
             "ta_pair_embed_add: multipliers out of range");
  if (dtype == TA_F32)
    pair_embed_add_kernel<float><<<nt, 256, 0, stream>>>(x, (const float*)table, tokens, last_token, cu_q,
                                                        pos0, slots, batch, d, buckets, mul_prev, mul_cur);
  else if (dtype == TA_BF16)
    pair_embed_add_kernel<bf16_t><<<nt, 256, 0, stream>>>(x, (const bf16_t*)table, tokens, last_token, cu_q,
                                                         pos0, slots, batch, d, buckets, mul_prev, mul_cur);
  else
    return ta_fail("ta_pair_embed_add: unknown dtype %d", dtype);
  return ta_check_launch("ta_pair_embed_add");
}

// ------------------------------------------------------------------ scaling in place
__global__ void scale_kernel(float* __restrict__ t, size_t n, float s) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) t[i] *= s;
}

extern "C" int ta_scale_f32(hipStream_t stream, float* t, long long n, float s) {
  TA_REQUIRE(n >= 0, "ta_scale_f32: negative size");
  if (n == 0) return 0;
  size_t blocks = ((size_t)n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  scale_kernel<<<(unsigned)blocks, 256, 0, stream>>>(t, (size_t)n, s);
  return ta_check_launch("ta_scale_f32");
}

// What happens to a token's [q | k | v] projection before attention reads the cache, for the
// attention variant whose queries and keys are normalised over the whole projection and whose
// values have a width of their own:
//
//   q <- rms_norm(q over all heads at once) * wq, k likewise with wk      (float32)
//   the first `rot` coordinates of every head of q and k are rotated in pairs (i, i + rot/2)
//   v <- (1 - lambda) v + lambda v_first      (where the layer mixes in the values of an earlier one)
//   q is written back in place; k and v go to the paged cache (keys [pages][kv heads][PAGE][dk],
//   values [pages][kv heads][dvs][PAGE], dvs >= dv, rows dv.. of a token zero).
//
// One workgroup per token. Everything is float32 until the single rounding of each result.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void qk_prepare_kernel(
    T* __restrict__ qkv, int stride, const float* __restrict__ wq, const float* __restrict__ wk,
    float eps, int normed, const float* __restrict__ angles, int rot,
    const float* __restrict__ lambda, const T* __restrict__ v_first, T* __restrict__ v_keep,
    const int* __restrict__ dest, T* __restrict__ kcache, T* __restrict__ vcache,
    int nh, int nkv, int dk, int dv, int dvs) {
  extern __shared__ float buf[];          // [nh*dk + nkv*dk]
  __shared__ float red[8];
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * stride;
  const int nq = nh * dk, nk = nkv * dk, nv = nkv * dv;
  // Loops over a row go in groups of four turns that are known to lie inside it: a load is
  // not asked for before the test that guards it, so turn by turn every load would wait for
  // the one before (20 trips to memory for a row of 5,120 where 5 do).
  float sq = 0.f, sk = 0.f;
  auto take = [&](int i) {
    const float v = to_f32(row[i]);
    buf[i] = v;
    if (i < nq) sq += v * v; else sk += v * v;
  };
  {
    int i = threadIdx.x;
    for (; i + 768 < nq + nk; i += 1024) {
#pragma unroll
      for (int u = 0; u < 4; ++u) take(i + 256 * u);
    }
    for (; i < nq + nk; i += 256) take(i);
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (threadIdx.x % TA_WAVE == 0) {
    red[threadIdx.x / TA_WAVE] = sq;
    red[4 + threadIdx.x / TA_WAVE] = sk;
  }
  __syncthreads();
  float fq = 1.f, fk = 1.f;
  if (normed) {
    fq = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)nq + eps);
    fk = rsqrtf((red[4] + red[5] + red[6] + red[7]) / (float)nk + eps);
  }
  const int half = rot / 2;
  const float* ang = angles ? angles + (size_t)t * half * 2 : nullptr;
  const int page = dest ? dest[t] / TA_PAGE : 0, off = dest ? dest[t] % TA_PAGE : 0;
  // Every thread reads the LDS copy and writes memory, so nothing it reads is written by another
  // thread. All loads are unconditional (a coordinate that is not rotated reads angle 0 and is
  // not changed by it), so that the loads of several turns are on their way together.
  auto finish = [&](int i) {
    const bool is_q = i < nq;
    const int j = is_q ? i : i - nq;
    const int head = j / dk, c = j - head * dk;
    const float f = is_q ? fq : fk;
    const float* w = is_q ? wq : wk;
    const bool turns = ang != nullptr && c < rot;
    const int pi = turns ? (c < half ? c : c - half) : 0;
    const int shift = turns ? (c < half ? half : -half) : 0;
    const float cs = ang ? ang[2 * pi] : 1.f, sn = ang ? ang[2 * pi + 1] : 0.f;
    float wv = 1.f, wo = 1.f;
    if (normed) {                     // the same for every thread
      wv = w[j];
      wo = w[j + shift];
    }
    float v = buf[i] * f * wv;
    const float o = buf[i + shift] * f * wo;
    if (turns) v = c < half ? v * cs - o * sn : v * cs + o * sn;
    if (is_q) {
      row[i] = from_f32<T>(v);
    } else if (dest) {
      kcache[(((size_t)page * nkv + head) * TA_PAGE + off) * dk + c] = from_f32<T>(v);
    }
  };
  {
    int i = threadIdx.x;
    for (; i + 768 < nq + nk; i += 1024) {
#pragma unroll
      for (int u = 0; u < 4; ++u) finish(i + 256 * u);
    }
    for (; i < nq + nk; i += 256) finish(i);
  }
  const float lam = lambda ? lambda[0] : 0.f;
  for (int i = threadIdx.x; i < nv; i += 256) {
    float v = to_f32(row[nq + nk + i]);
    if (v_keep) v_keep[(size_t)t * nv + i] = from_f32<T>(v);
    if (v_first) v = (1.0f - lam) * v + lam * to_f32(v_first[(size_t)t * nv + i]);
    if (dest) {
      const int g = i / dv, c = i - g * dv;
      vcache[(((size_t)page * nkv + g) * dvs + c) * TA_PAGE + off] = from_f32<T>(v);
    }
  }
  // a cache whose value rows are wider than the values (dvs > dv) holds zeros there
  if (dest && dvs > dv) {
    const int pad = dvs - dv;
    for (int i = threadIdx.x; i < nkv * pad; i += 256) {
      const int g = i / pad, c = dv + (i - g * pad);
      vcache[(((size_t)page * nkv + g) * dvs + c) * TA_PAGE + off] = from_f32<T>(0.f);
    }
  }
}

// qkv: [nt, stride] rows of [nh*dk | nkv*dk | nkv*dv]. wq [nh*dk], wk [nkv*dk] (used when normed).
// angles: [nt, rot/2, 2] (cos, sin) or null. lambda: one float on the device, v_first [nt, nkv*dv]
// (both or neither). v_keep [nt, nkv*dv] or null: receives the unmixed values. dest [nt] or null:
// page * PAGE + offset of each token in the cache layer.
extern "C" int ta_qk_prepare(hipStream_t stream, int dtype, void* qkv, int stride, const float* wq,
                             const float* wk, float eps, int normed, const float* angles, int rot,
                             const float* lambda, const void* v_first, void* v_keep, const int* dest,
                             void* kcache, void* vcache, int nt, int nh, int nkv, int dk, int dv,
                             int dvs) {
  TA_REQUIRE(nt >= 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0, "ta_qk_prepare: bad sizes");
  TA_REQUIRE(stride >= (nh + nkv) * dk + nkv * dv, "ta_qk_prepare: row stride %d too small", stride);
  TA_REQUIRE(rot >= 0 && rot <= dk && rot % 2 == 0, "ta_qk_prepare: %d rotated coordinates of %d", rot, dk);
  TA_REQUIRE((lambda == nullptr) == (v_first == nullptr), "ta_qk_prepare: lambda and v_first go together");
  TA_REQUIRE(!normed || (wq && wk), "ta_qk_prepare: norm weights missing");
  TA_REQUIRE(!dest || (kcache && vcache), "ta_qk_prepare: cache layer missing");
  TA_REQUIRE(dvs >= dv, "ta_qk_prepare: cache rows of %d cannot hold values of %d", dvs, dv);
  const size_t lds = (size_t)(nh + nkv) * dk * sizeof(float);
  TA_REQUIRE(lds <= 60000, "ta_qk_prepare: %d + %d heads of %d do not fit", nh, nkv, dk);
  if (nt == 0) return 0;
  if (rot == 0) angles = nullptr;
  if (dtype == TA_F32)
    qk_prepare_kernel<float><<<nt, 256, lds, stream>>>(
        (float*)qkv, stride, wq, wk, eps, normed, angles, rot, lambda, (const float*)v_first, (float*)v_keep,
        dest, (float*)kcache, (float*)vcache, nh, nkv, dk, dv, dvs);
  else if (dtype == TA_BF16)
    qk_prepare_kernel<bf16_t><<<nt, 256, lds, stream>>>(
        (bf16_t*)qkv, stride, wq, wk, eps, normed, angles, rot, lambda, (const bf16_t*)v_first, (bf16_t*)v_keep,
        dest, (bf16_t*)kcache, (bf16_t*)vcache, nh, nkv, dk, dv, dvs);
  else
    return ta_fail("ta_qk_prepare: unknown dtype %d", dtype);
  return ta_check_launch("ta_qk_prepare");
}

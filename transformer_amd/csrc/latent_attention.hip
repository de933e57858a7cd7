// Attention over a cache that keeps ONE row per token for all heads: a latent c [rank] from
// which every head's unrotated key and value are linear maps (k_h = Uk_h c, v_h = Uv_h c), and
// a rotated key part [rot] that the heads share. The maps are applied to the query and to the
// result instead of to the cached rows:
//
//   score(h, i, j) = ((Uk_h^T q_h,i) . c_j + qrot_h,i . krot_j) * scale
//   out_h,i        = Uv_h (sum_j p(h, i, j) c_j)
//
// so the kernels here see one "key" row [rank + rot] per token, queries of the same width,
// and return the weighted sums of the first `rank` coordinates.
//
//   latent_prepare   : from the rows of a step's first product: RMS norm of the query latent;
//                      RMS norm of the key/value latent and rotation of the shared key part,
//                      both stored into the cache row of the token
//   latent_query_rot : the rotated part of every head's query, rotated, into the last `rot`
//                      coordinates of the wide query rows
//   latent_attention : causal (windowed) softmax attention of the wide queries over the
//                      cached rows with an output gate per (token, head): float32 on the
//                      vector ALU; for bfloat16 rows on the matrix cores, with a workgroup's
//                      waves sharing their chunks of keys in steps of many rows and a row's
//                      keys dealt to several waves in steps of few
//
// Rotation: coordinates (2i, 2i + 1), i < dims / 2, of a rotated part turn by the token's
// angle i; angles come as (cos, sin) float32 [nt, dims / 2, 2]. Everything between loads and
// the one rounding of each result is float32. Keys are walked in chunks of 32 aligned to
// absolute positions, so a row's bits depend on its own query and keys only.
#include "common.h"
#include <type_traits>

__device__ __forceinline__ float la_block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x / TA_WAVE;
  __syncthreads();
  if (threadIdx.x % TA_WAVE == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < (int)(blockDim.x / TA_WAVE); ++i) s += red[i];
  return s;
}

template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ proj, int stride, int q_rank, const float* __restrict__ qw, T* __restrict__ cq,
    int kvoff, int rank, int rot, int rot_dims, const float* __restrict__ kw, float eps,
    const float* __restrict__ angles, const int* __restrict__ dest, T* __restrict__ kcache, int dc) {
  __shared__ float red[4];
  const size_t t = blockIdx.x;
  const T* row = proj + t * stride;
  if (q_rank > 0) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < q_rank; c += 256) {
      const float v = to_f32(row[c]);
      ss += v * v;
    }
    const float f = rsqrtf(la_block_sum(ss, red) / (float)q_rank + eps);
    for (int c = threadIdx.x; c < q_rank; c += 256)
      cq[t * q_rank + c] = from_f32<T>(to_f32(row[c]) * f * qw[c]);
  }
  if (dest == nullptr) return;
  const T* kv = row + kvoff;
  float ss = 0.f;
  for (int c = threadIdx.x; c < rank; c += 256) {
    const float v = to_f32(kv[c]);
    ss += v * v;
  }
  const float f = rsqrtf(la_block_sum(ss, red) / (float)rank + eps);
  T* out = kcache + (size_t)dest[t] * dc;
  for (int c = threadIdx.x; c < rank; c += 256) out[c] = from_f32<T>(to_f32(kv[c]) * f * kw[c]);
  for (int c = rank + rot + threadIdx.x; c < dc; c += 256) out[c] = from_f32<T>(0.f);
  const float* ang = angles + t * (size_t)rot_dims;          // (cos, sin) pairs: rot_dims floats a token
  for (int i = threadIdx.x; i < rot / 2 + (rot & 1); i += 256) {
    const float u = to_f32(kv[rank + 2 * i]);
    if (2 * i + 1 >= rot) { out[rank + 2 * i] = from_f32<T>(u); continue; }
    const float v = to_f32(kv[rank + 2 * i + 1]);
    if (2 * i + 1 < rot_dims) {
      const float c = ang[2 * i], s = ang[2 * i + 1];
      out[rank + 2 * i] = from_f32<T>(u * c - v * s);
      out[rank + 2 * i + 1] = from_f32<T>(v * c + u * s);
    } else {
      out[rank + 2 * i] = from_f32<T>(u);
      out[rank + 2 * i + 1] = from_f32<T>(v);
    }
  }
}

// proj: [nt, stride] rows: the query latent (q_rank) first, the key/value latent (rank) and the
// shared key part (rot) from column kvoff. cq: [nt, q_rank]. dest null: the step's rows store
// nothing (the layer reads rows that another layer stored). kcache: [pages, 1, PAGE, dc], dc >=
// rank + rot; the rest of a row is zeroed.
extern "C" int ta_latent_prepare(hipStream_t stream, int dtype, const void* proj, int stride, int q_rank,
                                 const float* qw, void* cq, int kvoff, int rank, int rot, int rot_dims,
                                 const float* kw, float eps, const float* angles, const int* dest,
                                 void* kcache, int dc, int nt) {
  TA_REQUIRE(nt >= 0 && q_rank >= 0 && rank >= 1 && rot >= 0 && rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0,
             "ta_latent_prepare: bad sizes nt=%d q_rank=%d rank=%d rot=%d dims=%d", nt, q_rank, rank, rot, rot_dims);
  TA_REQUIRE(q_rank > 0 || dest != nullptr, "ta_latent_prepare: nothing to do");
  TA_REQUIRE(dest == nullptr || dc >= rank + rot, "ta_latent_prepare: cache rows of %d for %d + %d", dc, rank, rot);
  TA_REQUIRE(dest == nullptr || rot_dims == 0 || angles != nullptr, "ta_latent_prepare: angles are required");
  if (nt == 0) return 0;
  if (dtype == TA_F32)
    latent_prepare_kernel<float><<<nt, 256, 0, stream>>>((const float*)proj, stride, q_rank, qw, (float*)cq, kvoff, rank,
                                                        rot, rot_dims, kw, eps, angles, dest, (float*)kcache, dc);
  else if (dtype == TA_BF16)
    latent_prepare_kernel<bf16_t><<<nt, 256, 0, stream>>>((const bf16_t*)proj, stride, q_rank, qw, (bf16_t*)cq, kvoff,
                                                         rank, rot, rot_dims, kw, eps, angles, dest, (bf16_t*)kcache, dc);
  else
    return ta_fail("ta_latent_prepare: unknown dtype %d", dtype);
  return ta_check_launch("ta_latent_prepare");
}

// ------------------------------------------------------------------ rotated query parts
template <typename T>
__global__ __launch_bounds__(256) void latent_query_rot_kernel(const T* __restrict__ q, int H, int dn, int rot,
                                                               int rot_dims, const float* __restrict__ angles,
                                                               T* __restrict__ qa, int rank, int dc) {
  const size_t t = blockIdx.x;
  for (int idx = threadIdx.x; idx < H * (dc - rank - rot); idx += 256) {      // the rows' padding
    const int h = idx / (dc - rank - rot), i = idx % (dc - rank - rot);
    qa[(t * H + h) * (size_t)dc + rank + rot + i] = from_f32<T>(0.f);
  }
  const float* ang = angles + t * (size_t)rot_dims;
  const int pairs = (rot + 1) / 2;
  for (int idx = threadIdx.x; idx < H * pairs; idx += 256) {
    const int h = idx / pairs, i = idx % pairs;
    const T* src = q + (t * H + h) * (size_t)(dn + rot) + dn;
    T* dst = qa + (t * H + h) * (size_t)dc + rank;
    const float u = to_f32(src[2 * i]);
    if (2 * i + 1 >= rot) { dst[2 * i] = from_f32<T>(u); continue; }
    const float v = to_f32(src[2 * i + 1]);
    if (2 * i + 1 < rot_dims) {
      const float c = ang[2 * i], s = ang[2 * i + 1];
      dst[2 * i] = from_f32<T>(u * c - v * s);
      dst[2 * i + 1] = from_f32<T>(v * c + u * s);
    } else {
      dst[2 * i] = from_f32<T>(u);
      dst[2 * i + 1] = from_f32<T>(v);
    }
  }
}

// q: [nt, H, dn + rot] (each head: unrotated part, then the part to rotate); qa: [nt, H, dc], dc >=
// rank + rot, whose coordinates from ``rank`` on are written (the rotated part, then zeros).
extern "C" int ta_latent_query_rot(hipStream_t stream, int dtype, const void* q, int H, int dn, int rot,
                                   int rot_dims, const float* angles, void* qa, int rank, int dc, int nt) {
  TA_REQUIRE(nt >= 0 && H >= 1 && dn >= 0 && rot >= 0 && rank >= 1 && rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0,
             "ta_latent_query_rot: bad sizes");
  TA_REQUIRE(dc >= rank + rot, "ta_latent_query_rot: rows of %d for %d + %d", dc, rank, rot);
  if (nt == 0 || dc == rank) return 0;
  if (dtype == TA_F32)
    latent_query_rot_kernel<float><<<nt, 256, 0, stream>>>((const float*)q, H, dn, rot, rot_dims, angles, (float*)qa, rank, dc);
  else if (dtype == TA_BF16)
    latent_query_rot_kernel<bf16_t><<<nt, 256, 0, stream>>>((const bf16_t*)q, H, dn, rot, rot_dims, angles, (bf16_t*)qa, rank, dc);
  else
    return ta_fail("ta_latent_query_rot: unknown dtype %d", dtype);
  return ta_check_launch("ta_latent_query_rot");
}

// ------------------------------------------------------------------ attention
// A workgroup owns 16 rows, row = (query token, head); 16 lanes share a row. The 32 keys of
// a chunk sit in LDS once and serve as keys (all D coordinates) and as values (the first
// `rank`). NACC: output coordinates per lane (rank <= 16 * NACC).
#define LA_ROWS 16
#define LA_CHUNK 32

__device__ __forceinline__ float la16_max(float v) {
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 16));
  return v;
}
__device__ __forceinline__ float la16_sum(float v) {
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 16);
  return v;
}

template <typename T, int NACC>
__global__ __launch_bounds__(256) void latent_attention_kernel(
    const T* __restrict__ qa, T* __restrict__ out, const T* __restrict__ kcache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ pos0, int H, int rank, int rot, float scale, int window,
    const T* __restrict__ gate, int gate_stride, int dc) {
  extern __shared__ float smem[];
  const int D = rank + rot, DP = D + 1;
  const int b = blockIdx.y;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int nrows = qlen * H;
  const int row0 = blockIdx.x * LA_ROWS;
  if (row0 >= nrows) return;
  const int p0 = pos0[b];
  const int rloc = threadIdx.x / 16, lane = threadIdx.x % 16;
  const int row = row0 + rloc;
  const bool row_ok = row < nrows;
  const int qi = row_ok ? row / H : 0;
  const int head = row_ok ? row % H : 0;
  float* Qs = smem;                          // [LA_ROWS][D]
  float* Ks = Qs + LA_ROWS * D;              // [LA_CHUNK][D + 1]
  float* Ps = Ks + LA_CHUNK * DP;            // [LA_ROWS][LA_CHUNK]

  for (int i = threadIdx.x; i < LA_ROWS * D; i += 256) {
    const int r = i / D, d = i - r * D, rr = row0 + r;
    Qs[i] = rr < nrows ? to_f32(qa[((size_t)(q0 + rr / H) * H + rr % H) * dc + d]) : 0.f;
  }
  const int qi_min = row0 / H;
  const int last_row = (row0 + LA_ROWS - 1 < nrows - 1) ? row0 + LA_ROWS - 1 : nrows - 1;
  const int tile_end = p0 + last_row / H + 1;                          // exclusive
  int tile_start = 0;
  if (window > 0) {
    tile_start = p0 + qi_min + 1 - window;
    if (tile_start < 0) tile_start = 0;
  }
  const int my_end = p0 + qi + 1;
  int my_start = 0;
  if (window > 0) {
    my_start = my_end - window;
    if (my_start < 0) my_start = 0;
  }
  float acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int* table = block_table + (size_t)b * max_blocks;
  for (int c = tile_start / LA_CHUNK; c * LA_CHUNK < tile_end; ++c) {
    const int key0 = c * LA_CHUNK;
    const size_t page = (size_t)table[key0 / TA_PAGE];
    const size_t base = (page * TA_PAGE + key0 % TA_PAGE) * (size_t)dc;
    __syncthreads();                         // the chunk before has been read
    for (int i = threadIdx.x; i < LA_CHUNK * D; i += 256) {
      const int k = i / D, d = i - k * D;
      Ks[k * DP + d] = (key0 + k < tile_end) ? to_f32(kcache[base + (size_t)k * dc + d]) : 0.f;
    }
    __syncthreads();
    float s0 = 0.f, s1 = 0.f;
    {
      const float* qr = Qs + rloc * D;
      const float* k0 = Ks + lane * DP;
      const float* k1 = Ks + (lane + 16) * DP;
      for (int d = 0; d < D; ++d) {
        const float qv = qr[d];
        s0 = fmaf(qv, k0[d], s0);
        s1 = fmaf(qv, k1[d], s1);
      }
    }
    const int kk0 = key0 + lane, kk1 = kk0 + 16;
    const bool v0 = row_ok && kk0 >= my_start && kk0 < my_end;
    const bool v1 = row_ok && kk1 >= my_start && kk1 < my_end;
    s0 = v0 ? s0 * scale : -INFINITY;
    s1 = v1 ? s1 * scale : -INFINITY;
    const float m_new = fmaxf(m, la16_max(fmaxf(s0, s1)));
    float alpha = 1.f, e0 = 0.f, e1 = 0.f;
    if (m_new != -INFINITY) {
      alpha = expf(m - m_new);
      e0 = v0 ? expf(s0 - m_new) : 0.f;
      e1 = v1 ? expf(s1 - m_new) : 0.f;
    }
    l = l * alpha + la16_sum(e0 + e1);
    m = m_new;
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] *= alpha;
    Ps[rloc * LA_CHUNK + lane] = e0;
    Ps[rloc * LA_CHUNK + lane + 16] = e1;
    __syncthreads();
    {
      const float* pr = Ps + rloc * LA_CHUNK;
      for (int k = 0; k < LA_CHUNK; ++k) {
        const float p = pr[k];
        const float* vr = Ks + k * DP + lane;
#pragma unroll
        for (int i = 0; i < NACC; ++i)
          if (16 * i + lane < rank) acc[i] = fmaf(p, vr[16 * i], acc[i]);
      }
    }
  }
  if (row_ok) {
    float f = l > 0.f ? 1.0f / l : 0.f;
    if (gate) {
      const float g = to_f32(gate[(size_t)(q0 + qi) * gate_stride + head]);
      f *= 1.0f / (1.0f + expf(-g));
    }
    T* o = out + ((size_t)(q0 + qi) * H + head) * rank + lane;
#pragma unroll
    for (int i = 0; i < NACC; ++i)
      if (16 * i + lane < rank) o[16 * i] = from_f32<T>(acc[i] * f);
  }
}

template <typename T, int NACC>
static int latent_attention_run(hipStream_t stream, dim3 g, size_t lds, const void* qa, void* out,
                                const void* kcache, const int* block_table, int max_blocks, const int* cu_q,
                                const int* pos0, int H, int rank, int rot, float scale, int window,
                                const void* gate, int gate_stride, int dc) {
  auto kern = latent_attention_kernel<T, NACC>;
  static size_t allowed = 64 * 1024;                    // per instantiation: asked for once, not at every launch
  if (lds > allowed) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return ta_fail("ta_latent_attention: %zu bytes of LDS refused (%s)", lds, hipGetErrorString(e));
    allowed = lds;
  }
  kern<<<g, 256, lds, stream>>>((const T*)qa, (T*)out, (const T*)kcache, block_table, max_blocks, cu_q, pos0, H,
                                rank, rot, scale, window, (const T*)gate, gate_stride, dc);
  return 0;
}

// ------------------------------------------------------------------ the same on the matrix cores (bfloat16)
// Steps of few rows: a wave owns RT tiles of 16 rows and a share of their keys; a workgroup is four
// such waves that share nothing (no barrier between them). Keys come in chunks of 32 aligned to absolute
// positions: the wave copies a chunk's rows into its own piece of LDS, forms S^T = K Q^T on
// v_mfma_f32_16x16x32_bf16 (a lane then holds 4 keys x 2 tiles of ONE row: the softmax stays in
// the lane but for two shuffles), and O^T += C^T P^T with the latent's coordinates gathered
// from the same LDS rows. Scores, maxima, sums and weights are float32; a weight enters the
// second product as THREE bfloat16 pieces (p = p0 + p1 + p2 exactly: 3 x 8 bits of mantissa), so
// the product sees all of its 24 bits and only the cached rows are bfloat16.
// With `splits` > 1 a tile's chunks are dealt to that many waves, which leave (sums, maximum,
// sum of weights) in `partial` for `latent_merge_kernel`: steps of single tokens have few rows
// and long key ranges.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 la_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float la_floatx4;
union LaFrag {
  la_bf16x8 v;
  uint4 q;
  uint32_t w[4];
  uint16_t s[8];
};

// One chunk of 32 keys, already in LDS at Ks (rows RS elements apart), for the RT tiles of a wave:
// scores, softmax in the log2 domain, weighted sums of the coordinate blocks from qb0 on.
template <int KS, int CTP, int RT>
__device__ __forceinline__ void la_chunk(const bf16_t* __restrict__ Ks, int RS, int dc, int rank, int key0, int c, int g,
                                         const LaFrag (&qf)[RT][KS], const bool (&ok)[RT], const int (&my_start)[RT],
                                         const int (&my_end)[RT], float scale_log2, float (&m)[RT], float (&l)[RT],
                                         la_floatx4 (&O)[RT][CTP], int qb0) {
    // ---- scores: register j of tile t of a lane is key 16 t + 4 g + j for the lane's row c
    la_floatx4 S[RT][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int t = 0; t < 2; ++t) S[rt][t] = la_floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 32 * ks + 8 * g;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        LaFrag kf;
        kf.q = d < dc ? *reinterpret_cast<const uint4*>(Ks + (16 * t + c) * RS + d) : uint4{0, 0, 0, 0};
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          S[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[rt][ks].v, S[rt][t], 0, 0, 0);
      }
      if (KS > 10 && ks % 3 == 2) __builtin_amdgcn_sched_barrier(0);    // wide rows: operands are not all asked for at once
    }
    // ---- softmax of the lane's rows over the chunk, in the log2 domain
    LaFrag pf[RT][3];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float sv[8];
      float mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = key0 + 16 * (e / 4) + 4 * g + (e % 4);
        const bool vis = ok[rt] && key >= my_start[rt] && key < my_end[rt];
        sv[e] = vis ? S[rt][e / 4][e % 4] * scale_log2 : -INFINITY;
        mx = fmaxf(mx, sv[e]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, TA_WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, TA_WAVE));
      const float m_new = fmaxf(m[rt], mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m[rt] - m_use);       // m = -inf gives 0
      float rs = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(sv[e] - m_use);          // -inf gives 0
        rs += p;
        const float r1 = p - to_f32(from_f32<bf16_t>(p));
        const float r2 = r1 - to_f32(from_f32<bf16_t>(r1));
        pf[rt][0].s[e] = f32_to_bf16_bits(p);
        pf[rt][1].s[e] = f32_to_bf16_bits(r1);
        pf[rt][2].s[e] = f32_to_bf16_bits(r2);
      }
      rs += __shfl_xor(rs, 16, TA_WAVE);
      rs += __shfl_xor(rs, 32, TA_WAVE);
      l[rt] = l[rt] * alpha + rs;
      m[rt] = m_new;
      if (__any(alpha != 1.f)) {
#pragma unroll
        for (int ct = 0; ct < CTP; ++ct)
#pragma unroll
          for (int j = 0; j < 4; ++j) O[rt][ct][j] *= alpha;
      }
    }
    // ---- weighted sums. A lane reads 4 neighbouring coordinates (8 bytes) of each of its 8
    // keys and feeds four products from them: in product q of a block of 64 coordinates row i
    // of the first operand stands for coordinate 4 i + q, so register j of O[4 qb + q] is
    // coordinate 64 qb + 16 g + 4 j + q of the lane's row c.
#pragma unroll
    for (int qi = 0; qi < CTP / 4; ++qi) {
      const int qb = qb0 + qi;
      if (64 * qb >= rank) break;
      int col = 64 * qb + 4 * c;
      if (col > RS - 4) col = RS - 4;                     // past the row: coordinates nobody stores
      uint2 wv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        wv[e] = *reinterpret_cast<const uint2*>(Ks + (16 * (e / 4) + 4 * g + (e % 4)) * RS + col);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        LaFrag vf;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t lo = q < 2 ? wv[2 * i].x : wv[2 * i].y, hi = q < 2 ? wv[2 * i + 1].x : wv[2 * i + 1].y;
          vf.w[i] = __builtin_amdgcn_perm(hi, lo, (q & 1) ? 0x07060302u : 0x05040100u);
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int sp = 0; sp < 3; ++sp)
            O[rt][4 * qi + q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf[rt][sp].v, O[rt][4 * qi + q], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

template <int KS, int CT, int RT>
__global__ __launch_bounds__(256, ((KS <= 6 && RT == 1) ? 2 : 1)) void latent_attention_mfma_kernel(
    const bf16_t* __restrict__ qa, bf16_t* __restrict__ out, const bf16_t* __restrict__ kcache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ pos0, int H, int rank, int dc, float scale_log2, int window,
    const bf16_t* __restrict__ gate, int gate_stride, int splits, int tiles_max, float* __restrict__ partial) {
  extern __shared__ __attribute__((aligned(16))) unsigned char la_lds[];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int c = lane % 16, g = lane / 16;
  const int RS = dc + 8;                                  // elements between rows of the LDS copy
  bf16_t* Ks = reinterpret_cast<bf16_t*>(la_lds) + (size_t)wave * 32 * RS;
  const int b = blockIdx.y, split = blockIdx.z;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int nrows = qlen * H;
  // HALVES: rows too wide for one wave's registers (128 accumulators and 72 query registers): two
  // waves take the same tile, form the same scores, and each sums one half of the coordinates.
  constexpr bool HALVES = KS > 10;
  const int wid = blockIdx.x * 4 + wave;
  const int tile = HALVES ? wid / 2 : wid, half = HALVES ? wid % 2 : 0;
  const int row0 = tile * 16 * RT;
  if (row0 >= nrows) return;                              // a wave leaves alone: nothing below waits for others
  const int p0 = pos0[b];
  int my_start[RT], my_end[RT];
  bool ok[RT];
  LaFrag qf[RT][KS];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = row0 + 16 * rt + c;
    ok[rt] = row < nrows;
    const int qi = ok[rt] ? row / H : 0;
    my_end[rt] = p0 + qi + 1;
    my_start[rt] = window > 0 ? (my_end[rt] - window > 0 ? my_end[rt] - window : 0) : 0;
    const bf16_t* qrow = qa + ((size_t)q0 * H + (ok[rt] ? row : 0)) * dc;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 32 * ks + 8 * g;
      qf[rt][ks].q = (ok[rt] && d < dc) ? *reinterpret_cast<const uint4*>(qrow + d) : uint4{0, 0, 0, 0};
    }
  }
  const int last_row = (row0 + 16 * RT - 1 < nrows - 1) ? row0 + 16 * RT - 1 : nrows - 1;
  const int tile_end = p0 + last_row / H + 1;
  int tile_start = 0;
  if (window > 0) {
    tile_start = p0 + row0 / H + 1 - window;
    if (tile_start < 0) tile_start = 0;
  }
  const int c0 = tile_start / 32, c1 = (tile_end + 31) / 32;
  const int n = c1 - c0;
  const int ca = c0 + (int)((long long)n * split / splits), cb = c0 + (int)((long long)n * (split + 1) / splits);
  constexpr int CTP = HALVES ? CT / 2 : CT;               // coordinate tiles this wave sums
  const int qb0 = half * (CTP / 4);                       // its first block of 64 coordinates
  la_floatx4 O[RT][CTP];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ct = 0; ct < CTP; ++ct) O[rt][ct] = la_floatx4{0.f, 0.f, 0.f, 0.f};
  float m[RT], l[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) { m[rt] = -INFINITY; l[rt] = 0.f; }
  const int* table = block_table + (size_t)b * max_blocks;
  const int pieces = dc / 8;                              // 16-byte pieces of a row
  // A chunk is 32 * pieces pieces, NL = 2 KS of them a lane at most. With PRE they are asked for
  // one chunk ahead and wait in registers while the chunk before is multiplied.
  constexpr int NL = 2 * KS;
  constexpr bool PRE = KS <= 10;
  uint4 pre[PRE ? NL : 1];
  auto fetch = [&](int ch, uint4* buf, auto I0, auto I1) {
    constexpr int i0 = decltype(I0)::value, i1 = decltype(I1)::value;
    const int key0 = ch * 32;
    const size_t page = (size_t)table[key0 / TA_PAGE];
    const bf16_t* src = kcache + (page * TA_PAGE + key0 % TA_PAGE) * (size_t)dc;
#pragma unroll
    for (int i = i0; i < i1; ++i) {
      const int idx = lane + 64 * i;
      const int k = idx / pieces, pc = idx - k * pieces;
      const bool live = idx < 32 * pieces && key0 + k < tile_end;       // keys not written yet read as zero
      const uint4 v = *reinterpret_cast<const uint4*>(live ? src + (size_t)k * dc + pc * 8 : kcache);
      buf[i - i0] = live ? v : uint4{0, 0, 0, 0};
    }
  };
  auto stash = [&](const uint4* buf, auto I0, auto I1) {
    constexpr int i0 = decltype(I0)::value, i1 = decltype(I1)::value;
#pragma unroll
    for (int i = i0; i < i1; ++i) {
      const int idx = lane + 64 * i;
      const int k = idx / pieces, pc = idx - k * pieces;
      if (idx < 32 * pieces) *reinterpret_cast<uint4*>(Ks + k * RS + pc * 8) = buf[i - i0];
    }
  };
  using la_i0 = std::integral_constant<int, 0>;
  using la_nl = std::integral_constant<int, NL>;
  constexpr int NB = 12;                                  // pieces a lane brings in together without PRE
  if (PRE && ca < cb) fetch(ca, pre, la_i0{}, la_nl{});
  for (int ch = ca; ch < cb; ++ch) {
    const int key0 = ch * 32;
    __builtin_amdgcn_wave_barrier();                      // the chunk before has been read
    if (PRE) {
      stash(pre, la_i0{}, la_nl{});
      if (ch + 1 < cb) fetch(ch + 1, pre, la_i0{}, la_nl{});
    } else {
      uint4 buf[NB];
      using b0 = std::integral_constant<int, 0>;
      using b1 = std::integral_constant<int, (NB < NL ? NB : NL)>;
      using b2 = std::integral_constant<int, (2 * NB < NL ? 2 * NB : NL)>;
      using b3 = std::integral_constant<int, (3 * NB < NL ? 3 * NB : NL)>;
      static_assert(3 * NB >= NL, "three batches cover a chunk");
      fetch(ch, buf, b0{}, b1{});
      stash(buf, b0{}, b1{});
      __builtin_amdgcn_sched_barrier(0);
      fetch(ch, buf, b1{}, b2{});
      stash(buf, b1{}, b2{});
      __builtin_amdgcn_sched_barrier(0);
      fetch(ch, buf, b2{}, b3{});
      stash(buf, b2{}, b3{});
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_wave_barrier();
    la_chunk<KS, CTP, RT>(Ks, RS, dc, rank, key0, c, g, qf, ok, my_start, my_end, scale_log2, m, l, O, qb0);
  }
  // ---- results: register j of O[4 qi + q] is coordinate 64 (qb0 + qi) + 16 g + 4 j + q of the lane's row c
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (!ok[rt]) continue;
    const int row = row0 + 16 * rt + c;
    if (splits > 1) {
      float* dst = partial + ((((size_t)b * tiles_max + tile) * splits + split) * (16 * RT) + 16 * rt + c) * (rank + 2);
#pragma unroll
      for (int ct = 0; ct < CTP; ++ct)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int coord = 64 * (qb0 + ct / 4) + 16 * g + 4 * j + (ct % 4);
          if (coord < rank) dst[coord] = O[rt][ct][j];
        }
      if (g == 0 && half == 0) { dst[rank] = m[rt]; dst[rank + 1] = l[rt]; }
      continue;
    }
    float f = l[rt] > 0.f ? 1.0f / l[rt] : 0.f;
    if (gate) {
      const float gv = to_f32(gate[(size_t)(q0 + row / H) * gate_stride + row % H]);
      f *= 1.0f / (1.0f + expf(-gv));
    }
    bf16_t* o = out + ((size_t)q0 * H + row) * rank;
#pragma unroll
    for (int ct = 0; ct < CTP; ++ct)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int coord = 64 * (qb0 + ct / 4) + 16 * g + 4 * j + (ct % 4);
        if (coord < rank) o[coord] = from_f32<bf16_t>(O[rt][ct][j] * f);
      }
  }
}

// Steps of many rows (prompts): the four waves of a workgroup own four neighbouring tiles of 16
// rows, whose key ranges all but coincide, and SHARE every chunk: 256 threads bring a chunk in
// with whole-row loads, two chunks ahead in registers and two more in a ring of three LDS
// buffers, behind a barrier that waits for LDS traffic only (a plain __syncthreads would wait for
// the loads that are meant to stay in flight). Each chunk is read from memory once per 64 rows
// instead of once per 16, and a wave's registers hold two small sets of pieces instead of a whole
// chunk, so rows of every width get their chunks ahead of time.
template <int KS, int CT>
__global__ __launch_bounds__(256, (KS <= 10 ? 2 : 1)) void latent_attention_mfma_wg_kernel(
    const bf16_t* __restrict__ qa, bf16_t* __restrict__ out, const bf16_t* __restrict__ kcache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ pos0, int H, int rank, int dc, float scale_log2, int window,
    const bf16_t* __restrict__ gate, int gate_stride) {
  extern __shared__ __attribute__((aligned(16))) unsigned char la_lds[];
  constexpr int NBUF = 3;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int c = lane % 16, g = lane / 16;
  const int RS = dc + 8;
  bf16_t* ring = reinterpret_cast<bf16_t*>(la_lds);       // [NBUF][32][RS]
  const int b = blockIdx.y;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int nrows = qlen * H;
  // HALVES (rows too wide for one wave's registers): two tiles a workgroup, and two waves a tile,
  // which form the same scores and sum one half of the coordinates each
  constexpr bool HALVES = KS > 10;
  constexpr int WG_ROWS = HALVES ? 32 : 64, CTP = HALVES ? CT / 2 : CT;
  const int wg_row0 = blockIdx.x * WG_ROWS;
  if (wg_row0 >= nrows) return;                           // the whole workgroup
  const int p0 = pos0[b];
  const int row0 = wg_row0 + 16 * (HALVES ? wave / 2 : wave);
  const int qb0 = HALVES ? (wave % 2) * (CTP / 4) : 0;
  const bool active = row0 < nrows;                       // a wave without rows still brings chunks in
  int my_start[1], my_end[1];
  bool ok[1];
  LaFrag qf[1][KS];
  {
    const int row = row0 + c;
    ok[0] = row < nrows;
    const int qi = ok[0] ? row / H : 0;
    my_end[0] = p0 + qi + 1;
    my_start[0] = window > 0 ? (my_end[0] - window > 0 ? my_end[0] - window : 0) : 0;
    const bf16_t* qrow = qa + ((size_t)q0 * H + (ok[0] ? row : 0)) * dc;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 32 * ks + 8 * g;
      qf[0][ks].q = (ok[0] && d < dc) ? *reinterpret_cast<const uint4*>(qrow + d) : uint4{0, 0, 0, 0};
    }
  }
  // the wave's own keys and the workgroup's
  const int w_last = (row0 + 15 < nrows - 1) ? row0 + 15 : nrows - 1;
  const int w_end = active ? p0 + w_last / H + 1 : 0;
  const int w_start = (active && window > 0 && p0 + row0 / H + 1 - window > 0) ? p0 + row0 / H + 1 - window : 0;
  const int g_last = (wg_row0 + WG_ROWS - 1 < nrows - 1) ? wg_row0 + WG_ROWS - 1 : nrows - 1;
  const int g_end = p0 + g_last / H + 1;
  const int g_start = (window > 0 && p0 + wg_row0 / H + 1 - window > 0) ? p0 + wg_row0 / H + 1 - window : 0;
  const int c0 = g_start / 32, n = (g_end + 31) / 32 - c0;
  la_floatx4 O[1][CTP];
#pragma unroll
  for (int ct = 0; ct < CTP; ++ct) O[0][ct] = la_floatx4{0.f, 0.f, 0.f, 0.f};
  float m[1] = {-INFINITY}, l[1] = {0.f};
  const int* table = block_table + (size_t)b * max_blocks;
  const int pieces = dc / 8, total = 32 * pieces;
  constexpr int NP = (KS + 1) / 2;                        // pieces of a chunk a thread brings: 32 * 4 KS / 256
  struct Set {
    uint4 v[NP];
  };
  // loads without conditions (a piece that is not there reads the chunk's first): what is not
  // there is decided when the pieces go to LDS, after the wait that is due then anyway
  auto fetch = [&](Set& q, int i) {
    const int key0 = (c0 + i) * 32;
    const size_t page = (size_t)table[key0 / TA_PAGE];
    const bf16_t* src = kcache + (page * TA_PAGE + key0 % TA_PAGE) * (size_t)dc;
#pragma unroll
    for (int u = 0; u < NP; ++u) {
      const int idx = tid + 256 * u;
      const int k = idx / pieces, pc = idx - k * pieces;
      q.v[u] = *reinterpret_cast<const uint4*>(idx < total ? src + (size_t)k * dc + pc * 8 : src);
    }
  };
  auto stash = [&](const Set& q, int i) {
    const int key0 = (c0 + i) * 32;
    bf16_t* Ks = ring + (size_t)(i % NBUF) * 32 * RS;
#pragma unroll
    for (int u = 0; u < NP; ++u) {
      const int idx = tid + 256 * u;
      const int k = idx / pieces, pc = idx - k * pieces;
      if (idx < total)                                      // keys not written yet are stored as zero
        *reinterpret_cast<uint4*>(Ks + k * RS + pc * 8) = key0 + k < g_end ? q.v[u] : uint4{0, 0, 0, 0};
    }
  };
  auto multiply = [&](int i) {
    const int key0 = (c0 + i) * 32;
    if (!active || key0 + 32 <= w_start || key0 >= w_end) return;      // none of the wave's rows sees this chunk
    la_chunk<KS, CTP, 1>(ring + (size_t)(i % NBUF) * 32 * RS, RS, dc, rank, key0, c, g, qf, ok, my_start, my_end,
                         scale_log2, m, l, O, qb0);
  };
  auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  Set sa, sb;
  fetch(sa, 0);
  if (n > 1) fetch(sb, 1);
  stash(sa, 0);
  if (n > 1) stash(sb, 1);
  if (n > 2) fetch(sa, 2);
  if (n > 3) fetch(sb, 3);
  lds_barrier();
  // chunk i is multiplied from buffer i % 3 while chunk i + 1 waits in the next buffer; the pieces
  // of chunk i + 2 then leave their set for the third buffer and the set asks for chunk i + 4
  for (int i = 0; i < n; i += 2) {
    multiply(i);
    if (i + 2 < n) {
      stash(sa, i + 2);
      if (i + 4 < n) fetch(sa, i + 4);
    }
    lds_barrier();
    if (i + 1 >= n) break;
    multiply(i + 1);
    if (i + 3 < n) {
      stash(sb, i + 3);
      if (i + 5 < n) fetch(sb, i + 5);
    }
    lds_barrier();
  }
  if (!active || !ok[0]) return;
  const int row = row0 + c;
  float f = l[0] > 0.f ? 1.0f / l[0] : 0.f;
  if (gate) {
    const float gv = to_f32(gate[(size_t)(q0 + row / H) * gate_stride + row % H]);
    f *= 1.0f / (1.0f + expf(-gv));
  }
  bf16_t* o = out + ((size_t)q0 * H + row) * rank;
#pragma unroll
  for (int ct = 0; ct < CTP; ++ct)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int coord = 64 * (qb0 + ct / 4) + 16 * g + 4 * j + (ct % 4);
      if (coord < rank) o[coord] = from_f32<bf16_t>(O[0][ct][j] * f);
    }
}

template <int KS, int CT>
static int latent_mfma_wg_run(hipStream_t stream, dim3 g, size_t lds, const void* qa, void* out, const void* kcache,
                              const int* block_table, int max_blocks, const int* cu_q, const int* pos0, int H,
                              int rank, int dc, float scale_log2, int window, const void* gate, int gate_stride) {
  auto kern = latent_attention_mfma_wg_kernel<KS, CT>;
  static size_t allowed = 64 * 1024;                    // per instantiation: asked for once, not at every launch
  if (lds > allowed) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return ta_fail("ta_latent_attention: %zu bytes of LDS refused (%s)", lds, hipGetErrorString(e));
    allowed = lds;
  }
  kern<<<g, 256, lds, stream>>>((const bf16_t*)qa, (bf16_t*)out, (const bf16_t*)kcache, block_table, max_blocks,
                                cu_q, pos0, H, rank, dc, scale_log2, window, (const bf16_t*)gate, gate_stride);
  return 0;
}

// One wave per row: the shares of a row's keys are put together.
__global__ __launch_bounds__(64) void latent_merge_kernel(const float* __restrict__ partial, bf16_t* __restrict__ out,
                                                          const int* __restrict__ cu_q, int H, int rank, int splits,
                                                          int tiles_max, int rows_per_tile,
                                                          const bf16_t* __restrict__ gate, int gate_stride) {
  const int b = blockIdx.y, row = blockIdx.x;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  if (row >= qlen * H) return;
  const int tile = row / rows_per_tile, rl = row % rows_per_tile;
  const float* base = partial + (((size_t)b * tiles_max + tile) * splits * rows_per_tile + rl) * (rank + 2);
  const size_t step = (size_t)rows_per_tile * (rank + 2);
  extern __shared__ float wts[];          // [splits] weight of every share
  float M = -INFINITY;
  for (int s = threadIdx.x; s < splits; s += 64) M = fmaxf(M, base[s * step + rank]);
  M = wave_max(M);
  float L = 0.f;
  for (int s = threadIdx.x; s < splits; s += 64) {
    const float ms = base[s * step + rank];
    const float w = ms != -INFINITY ? exp2f(ms - M) : 0.f;
    wts[s] = w;
    L += w * base[s * step + rank + 1];
  }
  L = wave_sum(L);
  __syncthreads();
  float f = L > 0.f ? 1.0f / L : 0.f;
  if (gate) {
    const float gv = to_f32(gate[(size_t)(q0 + row / H) * gate_stride + row % H]);
    f *= 1.0f / (1.0f + expf(-gv));
  }
  bf16_t* o = out + ((size_t)q0 * H + row) * rank;
  for (int cdx = threadIdx.x; cdx < rank; cdx += 64) {
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < splits; ++s) acc = fmaf(wts[s], base[s * step + cdx], acc);     // shares in order
    o[cdx] = from_f32<bf16_t>(acc * f);
  }
}

template <int KS, int CT, int RT>
static int latent_mfma_run(hipStream_t stream, dim3 g, size_t lds, const void* qa, void* out, const void* kcache,
                           const int* block_table, int max_blocks, const int* cu_q, const int* pos0, int H,
                           int rank, int dc, float scale_log2, int window, const void* gate, int gate_stride,
                           int splits, int tiles_max, float* partial) {
  auto kern = latent_attention_mfma_kernel<KS, CT, RT>;
  static size_t allowed = 64 * 1024;                    // per instantiation: asked for once, not at every launch
  if (lds > allowed) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return ta_fail("ta_latent_attention: %zu bytes of LDS refused (%s)", lds, hipGetErrorString(e));
    allowed = lds;
  }
  kern<<<g, 256, lds, stream>>>((const bf16_t*)qa, (bf16_t*)out, (const bf16_t*)kcache, block_table, max_blocks,
                                cu_q, pos0, H, rank, dc, scale_log2, window, (const bf16_t*)gate, gate_stride, splits,
                                tiles_max, partial);
  return 0;
}

// Rows per tile that the matrix-core kernel gives a wave for this geometry (0: it does not take
// it), and the float32 values of scratch that `splits` shares of the keys need.
extern "C" int ta_latent_mfma_rows(int rank, int dc, int max_qlen, int H) {
  if (dc % 8 || rank < 1 || rank > 512 || dc > 576 || dc < rank) return 0;
  if (dc <= 192 && rank <= 128) return (long long)max_qlen * H >= 64 ? 32 : 16;
  return 16;
}
extern "C" long long ta_latent_mfma_scratch(int batch, int max_qlen, int H, int rank, int dc, int splits) {
  const int rows = ta_latent_mfma_rows(rank, dc, max_qlen, H);
  if (rows == 0 || splits <= 1) return 0;
  const long long tiles = ((long long)max_qlen * H + rows - 1) / rows;
  return (long long)batch * tiles * splits * rows * (rank + 2);
}

// qa: [nt, H, dc] wide queries (dc >= rank + rot, the rest zero). out: [nt, H, rank]. kcache: one
// layer, [pages][1][TA_PAGE][dc]. gate (or null): pre-activation of a sigmoid gate per
// (token, head), element h of a row of gate_stride elements. window <= 0: all earlier keys.
// bfloat16 with rows of whole 16-byte pieces runs on the matrix cores; `splits` > 1 deals a
// row's keys to that many waves (scratch: ta_latent_mfma_scratch floats). float32, and rows
// that are no multiple of 8 wide, run on the vector ALU (splits is ignored).
extern "C" int ta_latent_attention(hipStream_t stream, int dtype, const void* qa, void* out, const void* kcache,
                                   const int* block_table, int max_blocks, const int* cu_q, const int* pos0,
                                   int batch, int max_qlen, int H, int rank, int rot, int dc, float scale, int window,
                                   const void* gate, int gate_stride, int splits, float* scratch) {
  TA_REQUIRE(batch >= 0 && batch <= 65535 && max_qlen >= 0 && H >= 1, "ta_latent_attention: bad batch=%d max_qlen=%d heads=%d", batch, max_qlen, H);
  TA_REQUIRE(rank >= 1 && rank <= 512 && rot >= 0 && rot <= 512, "ta_latent_attention: latent of %d / rotated part of %d outside [1, 512] / [0, 512]", rank, rot);
  TA_REQUIRE(dc >= rank + rot, "ta_latent_attention: rows of %d for %d + %d", dc, rank, rot);
  TA_REQUIRE(max_blocks > 0, "ta_latent_attention: empty block table");
  TA_REQUIRE(gate == nullptr || gate_stride >= H, "ta_latent_attention: gate rows too short");
  if (batch == 0 || max_qlen == 0) return 0;
  const int rows = dtype == TA_BF16 ? ta_latent_mfma_rows(rank, dc, max_qlen, H) : 0;
  if (rows > 0) {
    TA_REQUIRE(splits >= 1 && splits <= 65535 && (splits == 1 || scratch != nullptr), "ta_latent_attention: %d shares without scratch", splits);
    if (splits == 1 && (long long)max_qlen * H >= 64) {   // many rows: workgroups of four tiles share their chunks
      const int wg_rows = (dc <= 320 && rank <= 256) ? 64 : 32;      // wide rows: two waves a tile, see the kernel
      const long long wgs = ((long long)max_qlen * H + wg_rows - 1) / wg_rows;
      TA_REQUIRE(wgs <= 2147483647ll, "ta_latent_attention: too many rows");
      dim3 gw((unsigned)wgs, batch);
      const size_t ldw = (size_t)3 * 32 * (dc + 8) * sizeof(bf16_t);
      const float sl2w = scale * 1.4426950408889634f;
      int rcw;
#define LA_WG(KS, CT) latent_mfma_wg_run<KS, CT>(stream, gw, ldw, qa, out, kcache, block_table, max_blocks, cu_q, pos0, H, rank, dc, sl2w, window, gate, gate_stride)
      if (dc <= 192 && rank <= 128) rcw = LA_WG(6, 8);
      else if (dc <= 320 && rank <= 256) rcw = LA_WG(10, 16);
      else rcw = LA_WG(18, 32);
#undef LA_WG
      if (rcw) return rcw;
      return ta_check_launch("ta_latent_attention");
    }
    const long long tiles = ((long long)max_qlen * H + rows - 1) / rows;
    TA_REQUIRE(tiles <= 2147483647ll, "ta_latent_attention: too many rows");
    const bool halves = !(dc <= 320 && rank <= 256);      // two waves a tile: see the kernel
    dim3 g((unsigned)(((halves ? 2 : 1) * tiles + 3) / 4), batch, splits);
    const size_t lds = (size_t)4 * 32 * (dc + 8) * sizeof(bf16_t);
    const float sl2 = scale * 1.4426950408889634f;
    int rc;
#define LA_MFMA(KS, CT, RT) latent_mfma_run<KS, CT, RT>(stream, g, lds, qa, out, kcache, block_table, max_blocks, cu_q, pos0, H, rank, dc, sl2, window, gate, gate_stride, splits, (int)tiles, scratch)
    if (dc <= 192 && rank <= 128) rc = rows == 32 ? LA_MFMA(6, 8, 2) : LA_MFMA(6, 8, 1);
    else if (dc <= 320 && rank <= 256) rc = LA_MFMA(10, 16, 1);
    else rc = LA_MFMA(18, 32, 1);
#undef LA_MFMA
    if (rc) return rc;
    if (splits > 1) {
      dim3 gm((unsigned)(max_qlen * H), batch);
      latent_merge_kernel<<<gm, 64, (size_t)splits * sizeof(float), stream>>>(scratch, (bf16_t*)out, cu_q, H, rank, splits, (int)tiles, rows,
                                                 (const bf16_t*)gate, gate_stride);
    }
    return ta_check_launch("ta_latent_attention");
  }
  const long long tiles = ((long long)max_qlen * H + LA_ROWS - 1) / LA_ROWS;
  TA_REQUIRE(tiles <= 2147483647ll, "ta_latent_attention: too many rows");
  dim3 g((unsigned)tiles, batch);
  const int D = rank + rot;
  const size_t lds = (size_t)(LA_ROWS * D + LA_CHUNK * (D + 1) + LA_ROWS * LA_CHUNK) * sizeof(float);
  TA_REQUIRE(lds <= 160 * 1024, "ta_latent_attention: rows of %d do not fit the LDS", D);
  int rc;
#define LA_RUN(T)                                                                                              \
  (rank <= 128 ? latent_attention_run<T, 8>(stream, g, lds, qa, out, kcache, block_table, max_blocks, cu_q, pos0, H, rank, rot, scale, window, gate, gate_stride, dc)   \
   : rank <= 256 ? latent_attention_run<T, 16>(stream, g, lds, qa, out, kcache, block_table, max_blocks, cu_q, pos0, H, rank, rot, scale, window, gate, gate_stride, dc) \
                 : latent_attention_run<T, 32>(stream, g, lds, qa, out, kcache, block_table, max_blocks, cu_q, pos0, H, rank, rot, scale, window, gate, gate_stride, dc))
  if (dtype == TA_F32) rc = LA_RUN(float);
  else if (dtype == TA_BF16) rc = LA_RUN(bf16_t);
  else return ta_fail("ta_latent_attention: unknown dtype %d", dtype);
#undef LA_RUN
  if (rc) return rc;
  return ta_check_launch("ta_latent_attention");
}

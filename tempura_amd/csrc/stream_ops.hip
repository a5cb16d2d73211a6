// Memory-bound kernels around several copies of the residual stream (hyper-connections), positions that are added
// to the embedding, biased query/key rows on their way into the cache, and a gated activation with limits.
// Everything is float32 arithmetic; only stored activations may be bfloat16.
#include <math.h>

#include "common.h"

// ---- embedding + sinusoidal position, written to every stream ---------------------------------
// out[t, s, j] = table[token[t], j] + pe(pos[t], j) for s < streams, where pe(p, 2i) = sin(p * f_i),
// pe(p, 2i + 1) = cos(p * f_i) and f_i = inv_freq[i] (float64, made on the host).  The angle is formed in float64
// and reduced to one turn there (rope_cos_sin), so large positions lose nothing.  inv_freq == nullptr: no position.
template <typename T>
__global__ void embed_pos_kernel(const int* __restrict__ tokens, const int* __restrict__ positions,
                                 const T* __restrict__ table, const double* __restrict__ inv_freq,
                                 float* __restrict__ out, int hidden, int streams) {
  const int t = blockIdx.x;
  const int j = blockIdx.y * blockDim.x + threadIdx.x;
  if (j >= hidden) return;
  float v = to_float(table[(size_t)tokens[t] * hidden + j]);
  if (inv_freq != nullptr) {
    float c, sn;
    rope_cos_sin(positions[t], inv_freq[j >> 1], 1.0f, c, sn);
    v += (j & 1) ? c : sn;
  }
  for (int s = 0; s < streams; ++s) out[((size_t)t * streams + s) * hidden + j] = v;
}

extern "C" int tp_embed_pos(const int* tokens, const int* positions, const void* table, int table_dt,
                            const double* inv_freq, float* out, int n, int hidden, int streams, hipStream_t s) {
  TP_REQUIRE(n >= 0 && hidden > 0 && streams > 0, "embed_pos: bad sizes n=%d hidden=%d streams=%d", n, hidden, streams);
  TP_REQUIRE(inv_freq == nullptr || positions != nullptr, "embed_pos: positions missing");
  if (n == 0) return 0;
  const dim3 grid(n, (hidden + 255) / 256);
  TP_REQUIRE(grid.y <= 65535, "embed_pos: hidden size too large");
  if (table_dt == TP_F32)
    hipLaunchKernelGGL(embed_pos_kernel<float>, grid, dim3(256), 0, s, tokens, positions, (const float*)table, inv_freq,
                       out, hidden, streams);
  else if (table_dt == TP_BF16)
    hipLaunchKernelGGL(embed_pos_kernel<bf16_t>, grid, dim3(256), 0, s, tokens, positions, (const bf16_t*)table,
                       inv_freq, out, hidden, streams);
  else
    TP_REQUIRE(false, "embed_pos: unknown dtype %d", table_dt);
  TP_CHECK_LAUNCH("embed_pos");
  return 0;
}

// ---- one step of the streams ------------------------------------------------------------------
// h [tokens, S, W] float32 holds S copies of the residual stream.  For output row i (token t = rows ? rows[i] : i):
//   1. with y (a sublayer's output, float32 [tokens, W]):   h'_t[b] = sum_a mix[a, b] h_t[a] + outc[b] * y_t
//      (all streams at once from the old ones; written back when write_h);
//   2. with inc:   u = sum_a inc[a] h'_t[a]  (inc == nullptr: plain sum);
//   3. with norm_w:   x = u / sqrt(mean(u^2) + eps) * norm_w, else x = u;   stored to x_out[i] (float32 or bfloat16).
// One call therefore closes a sublayer and opens the next one: the update of the streams, the next sublayer's input
// combination and its norm read and write the streams once.  Without x_out only step 1 runs.
// One block per row; u is kept in LDS between the two passes of the norm.
template <int SMAX, typename TO>
__global__ void hc_step_kernel(float* __restrict__ h, const float* __restrict__ y, const float* __restrict__ mix,
                               const float* __restrict__ outc, const float* __restrict__ inc,
                               const float* __restrict__ norm_w, float eps, TO* __restrict__ x_out,
                               const int* __restrict__ rows, int S, int W, int write_h) {
  extern __shared__ float lds[];   // W floats of u, then 32 of scratch, then S * S + 2 S coefficients
  float* u_s = lds;
  float* scratch = lds + W;
  float* cf = scratch + 32;
  const int i = blockIdx.x;
  const int t = rows ? rows[i] : i;
  for (int k = threadIdx.x; k < S * S + 2 * S; k += blockDim.x) {
    float v;
    if (k < S * S) v = mix ? mix[k] : ((k / S) == (k % S) ? 1.f : 0.f);
    else if (k < S * S + S) v = outc ? outc[k - S * S] : 1.f;
    else v = inc ? inc[k - S * S - S] : 1.f;
    cf[k] = v;
  }
  __syncthreads();
  float* ht = h + (size_t)t * S * W;
  float ss = 0.f;
  for (int j = threadIdx.x; j < W; j += blockDim.x) {
    float v[SMAX];
#pragma unroll
    for (int a = 0; a < SMAX; ++a) v[a] = a < S ? ht[(size_t)a * W + j] : 0.f;
    if (y != nullptr) {
      const float yv = y[(size_t)t * W + j];
      float nv[SMAX];
#pragma unroll
      for (int b = 0; b < SMAX; ++b) {
        float acc = 0.f;
#pragma unroll
        for (int a = 0; a < SMAX; ++a)
          if (a < S && b < S) acc = fmaf(cf[a * S + b], v[a], acc);
        nv[b] = b < S ? fmaf(cf[S * S + b], yv, acc) : 0.f;
      }
#pragma unroll
      for (int b = 0; b < SMAX; ++b) {
        v[b] = nv[b];
        if (write_h && b < S) ht[(size_t)b * W + j] = nv[b];
      }
    }
    if (x_out != nullptr) {
      float u = 0.f;
#pragma unroll
      for (int a = 0; a < SMAX; ++a)
        if (a < S) u = fmaf(cf[S * S + S + a], v[a], u);
      u_s[j] = u;
      ss = fmaf(u, u, ss);
    }
  }
  if (x_out == nullptr) return;
  TO* o = x_out + (size_t)i * W;
  if (norm_w == nullptr) {
    for (int j = threadIdx.x; j < W; j += blockDim.x) from_float(o + j, u_s[j]);   // (each thread reads what it wrote)
    return;
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)W + eps);
  for (int j = threadIdx.x; j < W; j += blockDim.x) from_float(o + j, u_s[j] * rstd * norm_w[j]);
}

extern "C" int tp_hc_step(float* h, const float* y, const float* mix, const float* outc, const float* inc,
                          const float* norm_w, float eps, void* x_out, int x_dt, const int* rows, int n_out, int S, int W,
                          int write_h, hipStream_t s) {
  TP_REQUIRE(n_out >= 0 && S > 0 && S <= 16 && W > 0 && W <= 32768, "hc_step: bad sizes rows=%d streams=%d width=%d", n_out, S, W);
  TP_REQUIRE(h != nullptr, "hc_step: no streams");
  TP_REQUIRE(x_out != nullptr || (y != nullptr && write_h), "hc_step: nothing to do");
  if (n_out == 0) return 0;
  const int threads = W >= 4096 ? 1024 : (W >= 512 ? 256 : 64);
  const size_t shmem = (size_t)(W + 32 + S * S + 2 * S) * sizeof(float);
  const int smax = S <= 1 ? 1 : (S <= 2 ? 2 : (S <= 4 ? 4 : (S <= 8 ? 8 : 16)));
#define HC_LAUNCH(SM, TO)                                                                                          \
  do {                                                                                                             \
    if (shmem > 48 * 1024)                                                                                         \
      (void)hipFuncSetAttribute((const void*)hc_step_kernel<SM, TO>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem); \
    hipLaunchKernelGGL((hc_step_kernel<SM, TO>), dim3(n_out), dim3(threads), shmem, s, h, y, mix, outc, inc, norm_w, eps, \
                       (TO*)x_out, rows, S, W, write_h);                                                            \
  } while (0)
#define HC_DISPATCH(TO)          \
  switch (smax) {                \
    case 1: HC_LAUNCH(1, TO); break;  \
    case 2: HC_LAUNCH(2, TO); break;  \
    case 4: HC_LAUNCH(4, TO); break;  \
    case 8: HC_LAUNCH(8, TO); break;  \
    default: HC_LAUNCH(16, TO); break; \
  }
  if (x_out == nullptr || x_dt == TP_F32) {
    HC_DISPATCH(float);
  } else if (x_dt == TP_BF16) {
    HC_DISPATCH(bf16_t);
  } else {
    TP_REQUIRE(false, "hc_step: unknown dtype %d", x_dt);
  }
#undef HC_DISPATCH
#undef HC_LAUNCH
  TP_CHECK_LAUNCH("hc_step");
  return 0;
}

// ---- x *= scale, float32, in place ------------------------------------------------------------
__global__ void scale_f32_kernel(float* __restrict__ x, size_t n, float scale) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] *= scale;
}

extern "C" int tp_scale_f32(float* x, size_t n, float scale, hipStream_t s) {
  if (n == 0) return 0;
  TP_REQUIRE((n + 255) / 256 < ((size_t)1 << 31), "scale: tensor too large");
  hipLaunchKernelGGL(scale_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, n, scale);
  TP_CHECK_LAUNCH("scale");
  return 0;
}

// ---- gated activation with limits -------------------------------------------------------------
// gu [m, 2 I] (gate columns, then up columns; or, interleaved, eight gate columns and eight up columns in turn, as
// the products with the activation in their epilogue have their weights): g = min(gate, limit),
// u = clamp(up, -limit, limit) (limit <= 0: no limits), out = g * sigmoid(slope * g) * (u + up_offset).
// slope 1, no limit and offset 0 is SwiGLU.
template <typename TI, typename TO>
__global__ void gated_act_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inter, size_t total, float slope,
                                 float limit, float up_offset, int interleaved) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t m = idx / inter;
  const int i = (int)(idx % inter);
  const int gc = interleaved ? (i / 8) * 16 + i % 8 : i;
  const int uc = interleaved ? gc + 8 : inter + i;
  float g = to_float(gu[m * 2 * inter + gc]);
  float u = to_float(gu[m * 2 * inter + uc]);
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  from_float(out + idx, g / (1.0f + expf(-slope * g)) * (u + up_offset));
}

extern "C" int tp_gated_act(const void* gu, int in_dt, void* out, int out_dt, int m, int inter, float slope, float limit,
                            float up_offset, int interleaved, hipStream_t s) {
  TP_REQUIRE(m >= 0 && inter > 0 && (!interleaved || inter % 8 == 0), "gated_act: bad sizes");
  if (m == 0) return 0;
  const size_t total = (size_t)m * inter;
  const dim3 grid((unsigned)((total + 255) / 256));
#define LAUNCH(TI, TO)                                                                                         \
  hipLaunchKernelGGL((gated_act_kernel<TI, TO>), grid, dim3(256), 0, s, (const TI*)gu, (TO*)out, inter, total, slope, \
                     limit, up_offset, interleaved)
  if (in_dt == TP_F32 && out_dt == TP_F32)
    LAUNCH(float, float);
  else if (in_dt == TP_F32 && out_dt == TP_BF16)
    LAUNCH(float, bf16_t);
  else if (in_dt == TP_BF16 && out_dt == TP_BF16)
    LAUNCH(bf16_t, bf16_t);
  else
    TP_REQUIRE(false, "gated_act: unsupported dtypes %d -> %d", in_dt, out_dt);
#undef LAUNCH
  TP_CHECK_LAUNCH("gated_act");
  return 0;
}

// ---- biased queries and keys into place -------------------------------------------------------
// rows [n, row_stride] float32 hold [q heads | k heads] x head_dim as a projection left them (no rotation).  A bias
// per column is added (q_bias [n_heads * head_dim], k_bias [n_kv * head_dim], either may be null), q goes to
// q_out [n, n_heads, head_dim], k into the key cache [page, kv_head, page_size, head_dim] at place slots[t] and,
// when v_cache is given (the values are the keys), also into the transposed value cache
// [page, kv_head, head_dim, page_size].  slots == nullptr: the rows hold q only.  Any head size.
template <typename TQ, typename TC>
__global__ void qk_store_kernel(const float* __restrict__ rows, int row_stride, const float* __restrict__ q_bias,
                                const float* __restrict__ k_bias, const int* __restrict__ slots, int n_heads, int n_kv,
                                int head_dim, TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                int page_size) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int q_dim = n_heads * head_dim;
  const int total = q_dim + (slots ? n_kv * head_dim : 0);
  if (c >= total) return;
  float v = rows[(size_t)t * row_stride + c];
  if (c < q_dim) {
    if (q_bias) v += q_bias[c];
    from_float(q_out + (size_t)t * q_dim + c, v);
    return;
  }
  const int kc = c - q_dim;
  if (k_bias) v += k_bias[kc];
  const int kh = kc / head_dim, d = kc % head_dim;
  const int slot = slots[t];
  const size_t page = (size_t)(slot / page_size), off = (size_t)(slot % page_size);
  from_float(k_cache + ((page * n_kv + kh) * page_size + off) * head_dim + d, v);
  if (v_cache != nullptr) from_float(v_cache + ((page * n_kv + kh) * head_dim + d) * page_size + off, v);
}

extern "C" int tp_qk_store(const float* rows, int row_stride, const float* q_bias, const float* k_bias, const int* slots,
                           int n, int n_heads, int n_kv, int head_dim, void* q_out, int q_dt, void* k_cache, void* v_cache,
                           int cache_dt, int page_size, hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_heads > 0 && n_kv >= 0 && head_dim > 0, "qk_store: bad sizes");
  TP_REQUIRE(slots == nullptr || (k_cache != nullptr && page_size > 0), "qk_store: cache missing");
  TP_REQUIRE(row_stride >= (n_heads + (slots ? n_kv : 0)) * head_dim, "qk_store: row too short");
  if (n == 0) return 0;
  const int total = (n_heads + (slots ? n_kv : 0)) * head_dim;
  const dim3 grid(n, (total + 255) / 256);
  TP_REQUIRE(grid.y <= 65535, "qk_store: row too wide");
#define LAUNCH(TQ, TC)                                                                                              \
  hipLaunchKernelGGL((qk_store_kernel<TQ, TC>), grid, dim3(256), 0, s, rows, row_stride, q_bias, k_bias, slots, n_heads, \
                     n_kv, head_dim, (TQ*)q_out, (TC*)k_cache, (TC*)v_cache, page_size)
  if (q_dt == TP_F32 && cache_dt == TP_F32)
    LAUNCH(float, float);
  else if (q_dt == TP_BF16 && cache_dt == TP_BF16)
    LAUNCH(bf16_t, bf16_t);
  else if (q_dt == TP_F32 && cache_dt == TP_BF16)
    LAUNCH(float, bf16_t);
  else if (q_dt == TP_BF16 && cache_dt == TP_F32)
    LAUNCH(bf16_t, float);
  else
    TP_REQUIRE(false, "qk_store: unknown dtypes %d %d", q_dt, cache_dt);
#undef LAUNCH
  TP_CHECK_LAUNCH("qk_store");
  return 0;
}

// A gated delta-rule mixer over a batch of requests that each bring a run of tokens: the recurrence over a
// per-request state, the small second product of a low-rank projection with the recurrence's decay or a sigmoid in
// its epilogue, and the per-head norm with its gate behind the recurrence.  All arithmetic is float32; the state
// [heads, key_dim, value_dim] lives in float32 rows of a per-request state tensor (row = request slot).
//
// A request r of the batch owns tokens cu_seqlens[r] .. cu_seqlens[r + 1] - 1 and the state row state_slots[r];
// everything is read from device memory, so the same launches serve prompt portions, single decoded tokens and
// captured steps.  A token's result does not depend on how its run was cut: every token is one step of the same
// chain, in the same order of operations.
#include <math.h>

#include "common.h"

__device__ inline float d_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
// ln(1 + e^v) without overflow: max(v, 0) + ln(1 + e^-|v|)
__device__ inline float d_softplus(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// ---- the recurrence ---------------------------------------------------------------------------
// Per head h (its q and k are those of key head h / (heads / kv_heads)), with q and k made unit vectors
// (x / sqrt(sum x^2 + unit_eps); q also times q_scale), beta = sigmoid(beta_raw) and a decay g per key channel:
//   S <- g * S (rows are key channels);  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
// With P = (g * S_old)^T k and R = (g * S_old)^T q the read-out is o = R + u (k . q), so one pass over a thread's
// state entries forms both sums, one reduction over the lanes that share a column adds them, and a second pass
// writes k u^T.
//
// qkv [n, row_stride] float32 holds, per token, q [kv_heads * dim] | k [kv_heads * dim] | v [heads * vdim] (after the
// convolution and its activation); decay [n, heads * dim]; beta_raw is column beta_col0 + h of `proj`.
//
// Two kernels.  delta_prep (a wave per token and key head, all tokens side by side) makes q and k unit vectors in
// place and leaves k . q per token and key head.  delta_scan is the chain: a block owns one request, one head and
// CB = 256 / KS value columns; a thread holds PER consecutive key channels of one column in registers, and the KS
// neighbouring lanes that share a column split the key channels among them (their sums meet by row permutes, no
// trip through LDS up to 16 lanes).  A wave has one instruction stream, so the time of a token is the number of
// instructions a wave issues for it: few state entries a lane (8 up to a key size of 128) keep that near 60.
// Tokens are taken TC at a time through LDS (rows padded to KS * PER channels with q = k = 0 and decay 1, so the
// run itself needs no bounds); the next chunk's values travel from memory into registers while this chunk runs.
struct DeltaArgs {
  float* qkv;
  int row_stride;
  const float* decay;
  const float* proj;
  int proj_stride, beta_col0;
  float* state;
  size_t state_stride, state_off;
  const int* cu_seqlens;
  const int* state_slots;
  float* y;
  float* kq;   // [n, kv_heads]
  int heads, kv_heads, dim, vdim;
  float q_scale, unit_eps;
};

__global__ __launch_bounds__(256) void delta_prep_kernel(DeltaArgs a, long pairs) {
  const long p = (long)blockIdx.x * 4 + threadIdx.x / TP_WAVE;
  const int lane = threadIdx.x % TP_WAVE;
  if (p >= pairs) return;
  const long t = p / a.kv_heads;
  const int g = (int)(p % a.kv_heads);
  float* q = a.qkv + (size_t)t * a.row_stride + (size_t)g * a.dim;
  float* k = q + (size_t)a.kv_heads * a.dim;
  float sq = 0.f, sk = 0.f;
  for (int i = lane; i < a.dim; i += TP_WAVE) {
    sq = fmaf(q[i], q[i], sq);
    sk = fmaf(k[i], k[i], sk);
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  const float rq = a.q_scale / sqrtf(sq + a.unit_eps), rk = 1.0f / sqrtf(sk + a.unit_eps);
  float dot = 0.f;
  for (int i = lane; i < a.dim; i += TP_WAVE) {
    const float qv = q[i] * rq, kv = k[i] * rk;
    q[i] = qv;
    k[i] = kv;
    dot = fmaf(qv, kv, dot);
  }
  dot = wave_sum(dot);
  if (lane == 0) a.kq[p] = dot;
}

// sum over KS neighbouring lanes (from a multiple of KS on); every lane gets it
template <int KS>
__device__ inline float column_sum(float v) {
#define DPP_ADD(ctrl) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, false))
  if (KS >= 2) DPP_ADD(0xB1);    // quad_perm [1, 0, 3, 2]
  if (KS >= 4) DPP_ADD(0x4E);    // quad_perm [2, 3, 0, 1]
  if (KS >= 8) DPP_ADD(0x141);   // row_half_mirror
  if (KS >= 16) DPP_ADD(0x140);  // row_mirror
#undef DPP_ADD
  if (KS >= 32) v += __shfl_xor(v, 16, TP_WAVE);
  return v;
}

template <int PER, int KS>
__global__ __launch_bounds__(256) void delta_scan_kernel(DeltaArgs a) {
  constexpr int DP = PER * KS, CW = TP_WAVE / KS, CB = 4 * CW;
  constexpr int TC = DP <= 256 ? 16 : 4096 / DP;
  constexpr int NI = (TC * DP + 255) / 256, NV = (TC * CB + 255) / 256;
  __shared__ __attribute__((aligned(16))) float qs[TC * DP];
  __shared__ __attribute__((aligned(16))) float kk[TC * DP];
  __shared__ __attribute__((aligned(16))) float gs[TC * DP];
  __shared__ float vs[TC * CB];
  __shared__ float bs[TC];
  __shared__ float kqs[TC];
  const int r = blockIdx.x, h = blockIdx.y;
  const int start = a.cu_seqlens[r], len = a.cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  const int tid = threadIdx.x, wave = tid / TP_WAVE, lane = tid % TP_WAVE;
  const int ks = lane % KS, jl = wave * CW + lane / KS;
  const int j = blockIdx.z * CB + jl;
  const bool col_ok = j < a.vdim;
  const int kvh = h / (a.heads / a.kv_heads);

  float* S_mem = a.state + (size_t)a.state_slots[r] * a.state_stride + a.state_off + (size_t)h * a.dim * a.vdim;
  float S[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = ks * PER + e;
    S[e] = (col_ok && i < a.dim) ? S_mem[(size_t)i * a.vdim + j] : 0.f;
  }
  const int q_col = kvh * a.dim, k_col = (a.kv_heads + kvh) * a.dim, v_col = 2 * a.kv_heads * a.dim + h * a.vdim;
  const int out_width = a.heads * a.vdim;
  const size_t decay_stride = (size_t)a.heads * a.dim;

  float rq[NI], rk[NI], rg[NI], rv[NV], rb = 0.f, rkq = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * 256 + tid;
      const int t = idx / DP, i = idx % DP;
      const bool in = idx < TC * DP && t0 + t < len && i < a.dim;
      const size_t row = (size_t)(start + t0 + t);
      rq[it] = in ? a.qkv[row * a.row_stride + q_col + i] : 0.f;
      rk[it] = in ? a.qkv[row * a.row_stride + k_col + i] : 0.f;
      rg[it] = in ? a.decay[row * decay_stride + (size_t)h * a.dim + i] : 1.f;
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = it * 256 + tid;
      const int t = idx / CB, c = idx % CB;
      const int col = blockIdx.z * CB + c;
      rv[it] = (idx < TC * CB && t0 + t < len && col < a.vdim) ? a.qkv[(size_t)(start + t0 + t) * a.row_stride + v_col + col] : 0.f;
    }
    if (tid < TC && t0 + tid < len) {
      const size_t row = (size_t)(start + t0 + tid);
      rb = d_sigmoid(a.proj[row * a.proj_stride + a.beta_col0 + h]);
      rkq = a.kq[row * a.kv_heads + kvh];
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < len; t0 += TC) {
    const int tc = min(TC, len - t0);
    __syncthreads();   // the chunk before has been consumed
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * 256 + tid;
      if (idx < TC * DP) {
        qs[idx] = rq[it];
        kk[idx] = rk[it];
        gs[idx] = rg[it];
      }
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = it * 256 + tid;
      if (idx < TC * CB) vs[idx] = rv[it];
    }
    if (tid < TC) {
      bs[tid] = rb;
      kqs[tid] = rkq;
    }
    __syncthreads();
    if (t0 + TC < len) fetch(t0 + TC);   // on its way while this chunk runs
    for (int t = 0; t < tc; ++t) {
      const float4* q4 = (const float4*)(qs + t * DP + ks * PER);
      const float4* k4 = (const float4*)(kk + t * DP + ks * PER);
      const float4* g4 = (const float4*)(gs + t * DP + ks * PER);
      float kr[PER];
      float pred[PER / 4], read[PER / 4];
#pragma unroll
      for (int e4 = 0; e4 < PER / 4; ++e4) {
        const float4 q = q4[e4], k = k4[e4], g = g4[e4];
        const float qa[4] = {q.x, q.y, q.z, q.w}, ka[4] = {k.x, k.y, k.z, k.w}, ga[4] = {g.x, g.y, g.z, g.w};
        float p = 0.f, rd = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int e = e4 * 4 + c;
          kr[e] = ka[c];
          S[e] *= ga[c];
          p = fmaf(S[e], ka[c], p);
          rd = fmaf(S[e], qa[c], rd);
        }
        pred[e4] = p;
        read[e4] = rd;
      }
      float ps = pred[0], rs = read[0];
#pragma unroll
      for (int e4 = 1; e4 < PER / 4; ++e4) {   // (a fixed order: the same sums wherever the token stands)
        ps += pred[e4];
        rs += read[e4];
      }
      ps = column_sum<KS>(ps);
      rs = column_sum<KS>(rs);
      const float u = bs[t] * (vs[t * CB + jl] - ps);
#pragma unroll
      for (int e = 0; e < PER; ++e) S[e] = fmaf(kr[e], u, S[e]);
      if (ks == 0 && col_ok) a.y[(size_t)(start + t0 + t) * out_width + (size_t)h * a.vdim + j] = fmaf(u, kqs[t], rs);
    }
  }
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = ks * PER + e;
    if (col_ok && i < a.dim) S_mem[(size_t)i * a.vdim + j] = S[e];
  }
}

extern "C" int tp_delta_scan(float* qkv, int row_stride, const float* decay, const float* proj, int proj_stride,
                             int beta_col0, float* state, size_t state_stride, size_t state_off, const int* cu_seqlens,
                             const int* state_slots, float* y, float* kq, int n, int n_req, int heads, int kv_heads, int dim,
                             int vdim, float q_scale, float unit_eps, hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_req >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "delta_scan: bad sizes");
  TP_REQUIRE(heads % kv_heads == 0, "delta_scan: %d heads is not a multiple of %d key heads", heads, kv_heads);
  TP_REQUIRE(dim <= 1024, "delta_scan: key size %d exceeds 1024", dim);
  TP_REQUIRE(row_stride >= 2 * kv_heads * dim + heads * vdim, "delta_scan: rows too short");
  TP_REQUIRE(state_stride >= state_off + (size_t)heads * dim * vdim, "delta_scan: state rows too short");
  TP_REQUIRE(heads <= 65535, "delta_scan: too many heads");
  if (n == 0 || n_req == 0) return 0;
  DeltaArgs a{qkv, row_stride, decay, proj, proj_stride, beta_col0, state, state_stride, state_off, cu_seqlens, state_slots, y, kq,
              heads, kv_heads, dim, vdim, q_scale, unit_eps};
  const long pairs = (long)n * kv_heads;
  TP_REQUIRE((pairs + 3) / 4 < 0x7fffffffL, "delta_scan: too many rows");
  hipLaunchKernelGGL(delta_prep_kernel, dim3((unsigned)((pairs + 3) / 4)), dim3(256), 0, s, a, pairs);
  // PER key channels a lane (8 up to a key size of 128, then 16, then 32), KS lanes a column (a power of two)
  const int per = dim <= 128 ? 8 : (dim <= 256 ? 16 : 32);
  int ks = 1;
  while (ks * per < dim) ks *= 2;
  const int cb = 4 * (TP_WAVE / ks);
  const dim3 grid(n_req, heads, (vdim + cb - 1) / cb);
  TP_REQUIRE(grid.z <= 65535, "delta_scan: too many value columns");
#define SCAN(P, K) hipLaunchKernelGGL((delta_scan_kernel<P, K>), grid, dim3(256), 0, s, a)
  if (per == 8) {
    if (ks == 1) SCAN(8, 1);
    else if (ks == 2) SCAN(8, 2);
    else if (ks == 4) SCAN(8, 4);
    else if (ks == 8) SCAN(8, 8);
    else SCAN(8, 16);
  } else if (per == 16) {
    SCAN(16, 16);
  } else {
    if (ks <= 16) SCAN(32, 16);
    else SCAN(32, 32);
  }
#undef SCAN
  TP_CHECK_LAUNCH("delta_scan");
  return 0;
}

// ---- the second product of a low-rank projection ----------------------------------------------
// out[t, c] = f(sum_i x[t, col0 + i] * wt[i, c]) for a small inner size `rank`; x are float32 rows (the first
// product's sums), wt float32 [rank, n_out] (the weight transposed, so that neighbouring lanes read neighbouring
// values).  f: 0 the sum itself; 1 its sigmoid; 2 a decay, exp(-exp(a_log[c / per_head]) * softplus(sum + bias[c])).
// A block takes eight rows and 256 columns; a row's sum has the same order of additions wherever the row stands.
#define LR_ROWS 8

__global__ __launch_bounds__(256) void lowrank_up_kernel(const float* __restrict__ x, int x_stride, int col0, int rank,
                                                         const float* __restrict__ wt, float* __restrict__ out, int n,
                                                         int n_out, int mode, const float* __restrict__ a_log,
                                                         const float* __restrict__ bias, int per_head) {
  extern __shared__ __attribute__((aligned(16))) float xs[];   // [LR_ROWS][rank4]: rows padded with zeros to four
  const int rank4 = (rank + 3) & ~3;
  const int t0 = blockIdx.x * LR_ROWS, c = blockIdx.y * 256 + threadIdx.x;
  for (int idx = threadIdx.x; idx < LR_ROWS * rank4; idx += 256) {
    const int t = idx / rank4, i = idx % rank4;
    xs[idx] = (t0 + t < n && i < rank) ? x[(size_t)(t0 + t) * x_stride + col0 + i] : 0.f;
  }
  __syncthreads();
  if (c >= n_out) return;
  float acc[LR_ROWS];
#pragma unroll
  for (int t = 0; t < LR_ROWS; ++t) acc[t] = 0.f;
  for (int i = 0; i < rank4; i += 4) {   // (ascending i for every row: the same sums wherever the row stands)
    float w[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) w[d] = i + d < rank ? wt[(size_t)(i + d) * n_out + c] : 0.f;
#pragma unroll
    for (int t = 0; t < LR_ROWS; ++t) {
      const float4 v = *(const float4*)(xs + t * rank4 + i);
      acc[t] = fmaf(v.x, w[0], acc[t]);
      acc[t] = fmaf(v.y, w[1], acc[t]);
      acc[t] = fmaf(v.z, w[2], acc[t]);
      acc[t] = fmaf(v.w, w[3], acc[t]);
    }
  }
  float rate = 0.f, b = 0.f;
  if (mode == 2) {
    rate = expf(a_log[c / per_head]);
    b = bias[c];
  }
#pragma unroll
  for (int t = 0; t < LR_ROWS; ++t) {
    if (t0 + t >= n) break;
    float v = acc[t];
    if (mode == 1) v = d_sigmoid(v);
    if (mode == 2) v = expf(-rate * d_softplus(v + b));
    out[(size_t)(t0 + t) * n_out + c] = v;
  }
}

extern "C" int tp_lowrank_up(const float* x, int x_stride, int col0, int rank, const float* wt, float* out, int n, int n_out,
                             int mode, const float* a_log, const float* bias, int per_head, hipStream_t s) {
  TP_REQUIRE(n >= 0 && rank > 0 && n_out > 0 && col0 >= 0 && x_stride >= col0 + rank, "lowrank_up: bad sizes");
  TP_REQUIRE(rank <= 1024, "lowrank_up: inner size %d exceeds 1024", rank);
  TP_REQUIRE(mode >= 0 && mode <= 2, "lowrank_up: unknown epilogue %d", mode);
  TP_REQUIRE(mode != 2 || (a_log && bias && per_head > 0), "lowrank_up: the decay needs its rates and biases");
  if (n == 0) return 0;
  const dim3 grid((n + LR_ROWS - 1) / LR_ROWS, (n_out + 255) / 256);
  TP_REQUIRE(grid.y <= 65535, "lowrank_up: too many columns");
  hipLaunchKernelGGL(lowrank_up_kernel, grid, dim3(256), sizeof(float) * LR_ROWS * ((rank + 3) & ~3), s, x, x_stride, col0, rank, wt, out, n,
                     n_out, mode, a_log, bias, per_head);
  TP_CHECK_LAUNCH("lowrank_up");
  return 0;
}

// ---- norm per head with a gate ----------------------------------------------------------------
// out[t, out_col0 + h * vdim + d] = o[t, h, d] / sqrt(mean_d o^2 + eps) * w[d] * gate[t, h * vdim + d] * scale;
// gate (float32, already between 0 and 1) may be missing.  One wave per (token, head).
template <typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             const float* __restrict__ gate, float eps, float scale,
                                                             TO* __restrict__ out, int out_stride, int out_col0, long pairs,
                                                             int heads, int vdim) {
  const long p = (long)blockIdx.x * 4 + threadIdx.x / TP_WAVE;
  const int lane = threadIdx.x % TP_WAVE;
  if (p >= pairs) return;
  const long t = p / heads;
  const int h = (int)(p % heads);
  const float* row = o + (size_t)p * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += TP_WAVE) ss = fmaf(row[d], row[d], ss);
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)vdim + eps);
  TO* dst = out + (size_t)t * out_stride + out_col0 + (size_t)h * vdim;
  for (int d = lane; d < vdim; d += TP_WAVE) {
    float v = row[d] * rstd * w[d];
    if (gate != nullptr) v *= gate[(size_t)p * vdim + d];
    from_float(dst + d, v * scale);
  }
}

extern "C" int tp_head_norm_gate(const float* o, const float* w, const float* gate, float eps, float scale, void* out, int out_dt,
                                 int out_stride, int out_col0, int n, int heads, int vdim, hipStream_t s) {
  TP_REQUIRE(n >= 0 && heads > 0 && vdim > 0 && out_col0 >= 0 && out_stride >= out_col0 + heads * vdim, "head_norm_gate: bad sizes");
  if (n == 0) return 0;
  const long pairs = (long)n * heads;
  const long blocks = (pairs + 3) / 4;
  TP_REQUIRE(blocks < 0x7fffffffL, "head_norm_gate: too many rows");
  if (out_dt == TP_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, o, w, gate, eps, scale, (float*)out,
                       out_stride, out_col0, pairs, heads, vdim);
  else if (out_dt == TP_BF16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, s, o, w, gate, eps, scale, (bf16_t*)out,
                       out_stride, out_col0, pairs, heads, vdim);
  else
    TP_REQUIRE(false, "head_norm_gate: unknown dtype %d", out_dt);
  TP_CHECK_LAUNCH("head_norm_gate");
  return 0;
}

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
// A block owns one request, one head and CB = 256 / KS value columns; a thread holds PER consecutive key channels
// of one column in registers, and the KS lanes of a wave that share a column (lane = ks * (64 / KS) + column) split
// the key channels among them.  Tokens are taken TC at a time: their q, k, decay, v and beta are staged in LDS (rows
// padded to KS * PER channels with q = k = 0, so the run itself needs no bounds), the unit norms and k . q are
// formed there by a wave per token, then the run over the chunk is register arithmetic and 16-byte LDS reads that
// most lanes share.
#define DELTA_TC_MAX 16   // (fewer when the padded key size is large: the chunk has to fit 60 KB of LDS)

struct DeltaArgs {
  const float* qkv;
  int row_stride;
  const float* decay;
  const float* proj;
  int proj_stride, beta_col0;
  float* state;
  size_t state_stride, state_off;
  const int* cu_seqlens;
  const int* state_slots;
  float* y;
  int heads, kv_heads, dim, vdim;
  int KS, TC;
  float q_scale, unit_eps;
};

template <int PER>
__global__ __launch_bounds__(256) void delta_scan_kernel(DeltaArgs a) {
  extern __shared__ float lds[];
  const int r = blockIdx.x, h = blockIdx.y;
  const int start = a.cu_seqlens[r], len = a.cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  const int KS = a.KS, CW = TP_WAVE / KS, CB = 4 * CW, DP = KS * PER;
  const int tid = threadIdx.x, wave = tid / TP_WAVE, lane = tid % TP_WAVE;
  const int ks = lane / CW, jl = wave * CW + lane % CW;
  const int j = blockIdx.z * CB + jl;
  const bool col_ok = j < a.vdim;
  const int kvh = h / (a.heads / a.kv_heads);
  const int TC = a.TC;
  float* qs = lds;                         // [TC][DP]
  float* kk = qs + TC * DP;          // [TC][DP]
  float* gs = kk + TC * DP;          // [TC][DP]
  float* vs = gs + TC * DP;          // [TC][CB]
  float* bs = vs + TC * CB;          // [TC] beta
  float* kq = bs + TC;               // [TC] k . q

  float* S_mem = a.state + (size_t)a.state_slots[r] * a.state_stride + a.state_off + (size_t)h * a.dim * a.vdim;
  float S[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = ks * PER + e;
    S[e] = (col_ok && i < a.dim) ? S_mem[(size_t)i * a.vdim + j] : 0.f;
  }
  const int q_col = kvh * a.dim, k_col = (a.kv_heads + kvh) * a.dim, v_col = 2 * a.kv_heads * a.dim + h * a.vdim;
  const int out_width = a.heads * a.vdim;

  for (int t0 = 0; t0 < len; t0 += TC) {
    const int tc = min(TC, len - t0);
    __syncthreads();   // the chunk before has been consumed
    for (int idx = tid; idx < tc * DP; idx += 256) {
      const int t = idx / DP, i = idx % DP;
      const size_t row = (size_t)(start + t0 + t);
      const bool in = i < a.dim;
      qs[idx] = in ? a.qkv[row * a.row_stride + q_col + i] : 0.f;
      kk[idx] = in ? a.qkv[row * a.row_stride + k_col + i] : 0.f;
      gs[idx] = in ? a.decay[row * ((size_t)a.heads * a.dim) + (size_t)h * a.dim + i] : 1.f;
    }
    for (int idx = tid; idx < tc * CB; idx += 256) {
      const int t = idx / CB, c = idx % CB;
      const int col = blockIdx.z * CB + c;
      vs[idx] = col < a.vdim ? a.qkv[(size_t)(start + t0 + t) * a.row_stride + v_col + col] : 0.f;
    }
    if (tid < tc) bs[tid] = d_sigmoid(a.proj[(size_t)(start + t0 + tid) * a.proj_stride + a.beta_col0 + h]);
    __syncthreads();
    // unit vectors and k . q: a wave per token
    for (int t = wave; t < tc; t += 4) {
      float sq = 0.f, sk = 0.f;
      for (int i = lane; i < DP; i += TP_WAVE) {
        const float qv = qs[t * DP + i], kv = kk[t * DP + i];
        sq = fmaf(qv, qv, sq);
        sk = fmaf(kv, kv, sk);
      }
      sq = wave_sum(sq);
      sk = wave_sum(sk);
      const float rq = a.q_scale / sqrtf(sq + a.unit_eps), rk = 1.0f / sqrtf(sk + a.unit_eps);
      float dot = 0.f;
      for (int i = lane; i < DP; i += TP_WAVE) {
        const float qv = qs[t * DP + i] * rq, kv = kk[t * DP + i] * rk;
        qs[t * DP + i] = qv;
        kk[t * DP + i] = kv;
        dot = fmaf(qv, kv, dot);
      }
      dot = wave_sum(dot);
      if (lane == 0) kq[t] = dot;
    }
    __syncthreads();
    for (int t = 0; t < tc; ++t) {
      const float4* q4 = (const float4*)(qs + t * DP + ks * PER);
      const float4* k4 = (const float4*)(kk + t * DP + ks * PER);
      const float4* g4 = (const float4*)(gs + t * DP + ks * PER);
      float kr[PER];
      float pred = 0.f, read = 0.f;
#pragma unroll
      for (int e4 = 0; e4 < PER / 4; ++e4) {
        const float4 q = q4[e4], k = k4[e4], g = g4[e4];
        const float qa[4] = {q.x, q.y, q.z, q.w}, ka[4] = {k.x, k.y, k.z, k.w}, ga[4] = {g.x, g.y, g.z, g.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int e = e4 * 4 + c;
          kr[e] = ka[c];
          S[e] *= ga[c];
          pred = fmaf(S[e], ka[c], pred);
          read = fmaf(S[e], qa[c], read);
        }
      }
      for (int o = CW; o < TP_WAVE; o <<= 1) {   // over the KS lanes of this column, the same order in every lane
        pred += __shfl_xor(pred, o, TP_WAVE);
        read += __shfl_xor(read, o, TP_WAVE);
      }
      const float u = bs[t] * (vs[t * CB + jl] - pred);
#pragma unroll
      for (int e = 0; e < PER; ++e) S[e] = fmaf(kr[e], u, S[e]);
      if (ks == 0 && col_ok) a.y[(size_t)(start + t0 + t) * out_width + (size_t)h * a.vdim + j] = fmaf(u, kq[t], read);
    }
  }
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = ks * PER + e;
    if (col_ok && i < a.dim) S_mem[(size_t)i * a.vdim + j] = S[e];
  }
}

extern "C" int tp_delta_scan(const float* qkv, int row_stride, const float* decay, const float* proj, int proj_stride,
                             int beta_col0, float* state, size_t state_stride, size_t state_off, const int* cu_seqlens,
                             const int* state_slots, float* y, int n_req, int heads, int kv_heads, int dim, int vdim,
                             float q_scale, float unit_eps, hipStream_t s) {
  TP_REQUIRE(n_req >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "delta_scan: bad sizes");
  TP_REQUIRE(heads % kv_heads == 0, "delta_scan: %d heads is not a multiple of %d key heads", heads, kv_heads);
  TP_REQUIRE(dim <= 1024, "delta_scan: key size %d exceeds 1024", dim);
  TP_REQUIRE(row_stride >= 2 * kv_heads * dim + heads * vdim, "delta_scan: rows too short");
  TP_REQUIRE(state_stride >= state_off + (size_t)heads * dim * vdim, "delta_scan: state rows too short");
  TP_REQUIRE(heads <= 65535, "delta_scan: too many heads");
  if (n_req == 0) return 0;
  // PER key channels a lane, KS lanes a column (a power of two up to 32): the least padding of the key size
  const int per = dim <= 64 ? 8 : (dim <= 256 ? 16 : 32);
  int ks = 1;
  while (ks * per < dim) ks *= 2;
  TP_REQUIRE(ks <= 32, "delta_scan: key size %d does not fit", dim);
  const int cb = 4 * (TP_WAVE / ks), dp = ks * per;
  int tc = DELTA_TC_MAX;
  while (tc > 1 && sizeof(float) * ((size_t)tc * (3 * dp + cb) + 2 * tc) > 60 * 1024) tc /= 2;
  DeltaArgs a{qkv, row_stride, decay, proj, proj_stride, beta_col0, state, state_stride, state_off, cu_seqlens, state_slots, y,
              heads, kv_heads, dim, vdim, ks, tc, q_scale, unit_eps};
  const dim3 grid(n_req, heads, (vdim + cb - 1) / cb);
  TP_REQUIRE(grid.z <= 65535, "delta_scan: too many value columns");
  const size_t shmem = sizeof(float) * ((size_t)tc * (3 * dp + cb) + 2 * tc);
  if (per == 8)
    hipLaunchKernelGGL(delta_scan_kernel<8>, grid, dim3(256), shmem, s, a);
  else if (per == 16)
    hipLaunchKernelGGL(delta_scan_kernel<16>, grid, dim3(256), shmem, s, a);
  else
    hipLaunchKernelGGL(delta_scan_kernel<32>, grid, dim3(256), shmem, s, a);
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
  extern __shared__ float xs[];   // [LR_ROWS][rank]
  const int t0 = blockIdx.x * LR_ROWS, c = blockIdx.y * 256 + threadIdx.x;
  for (int idx = threadIdx.x; idx < LR_ROWS * rank; idx += 256) {
    const int t = idx / rank, i = idx % rank;
    xs[idx] = t0 + t < n ? x[(size_t)(t0 + t) * x_stride + col0 + i] : 0.f;
  }
  __syncthreads();
  if (c >= n_out) return;
  float acc[LR_ROWS];
#pragma unroll
  for (int t = 0; t < LR_ROWS; ++t) acc[t] = 0.f;
  for (int i = 0; i < rank; ++i) {
    const float w = wt[(size_t)i * n_out + c];
#pragma unroll
    for (int t = 0; t < LR_ROWS; ++t) acc[t] = fmaf(xs[t * rank + i], w, acc[t]);
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
  hipLaunchKernelGGL(lowrank_up_kernel, grid, dim3(256), sizeof(float) * LR_ROWS * rank, s, x, x_stride, col0, rank, wt, out, n,
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

// A selective state-space mixer (state-space duality form) over a batch of requests that each bring a run of
// tokens: short causal convolution with carried inputs, the recurrence over a per-request state, and the gated
// grouped norm behind it.  All arithmetic is float32; the state lives in float32 rows of a per-request state tensor
// (row = request slot): first the convolution's last taps - 1 inputs, [taps - 1, channels], oldest first, then
// the recurrent state, [heads, state, head_dim].
//
// A request r of the batch owns tokens cu_seqlens[r] .. cu_seqlens[r + 1] - 1 and the state row state_slots[r];
// everything is read from device memory, so the same launches serve prompt portions, single decoded tokens and
// captured steps.  Results do not depend on how a prompt was cut: the recurrence runs token by token in order.
#include <math.h>

#include "common.h"

__device__ inline float silu_f(float v) { return v / (1.0f + expf(-v)); }
// ln(1 + e^v) without overflow: max(v, 0) + ln(1 + e^-|v|)
__device__ inline float softplus_f(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// ---- causal convolution per channel + SiLU ----------------------------------------------------
// in: rows [n, in_stride] float32, the channels at column col0; w [channels, taps] (the last column is the current
// token's), b [channels].  The inputs before a run's first token come from the request's state row (zeros for a
// fresh request).  out [n, channels] = silu(conv + b).
__global__ void causal_conv_kernel(const float* __restrict__ in, int in_stride, int col0, const float* __restrict__ w,
                                   const float* __restrict__ b, const float* __restrict__ state, size_t state_stride,
                                   const int* __restrict__ cu_seqlens, const int* __restrict__ token_req,
                                   const int* __restrict__ state_slots, float* __restrict__ out, int channels, int taps) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int r = token_req[t];
  const int start = cu_seqlens[r];
  const int i = t - start;
  const float* st = state + (size_t)state_slots[r] * state_stride;
  float acc = b[c];
  for (int k = 0; k < taps; ++k) {
    const int src = i - (taps - 1 - k);
    const float v = src >= 0 ? in[(size_t)(start + src) * in_stride + col0 + c] : st[(size_t)(taps - 1 + src) * channels + c];
    acc = fmaf(w[(size_t)c * taps + k], v, acc);
  }
  out[(size_t)t * channels + c] = silu_f(acc);
}

// The state after a run: the last taps - 1 inputs of (carried inputs, then the run's).  In place, ascending: entry j
// takes entry j + len of the old state or an input of the run, and entries below j are never read again.
__global__ void conv_state_kernel(const float* __restrict__ in, int in_stride, int col0, float* __restrict__ state,
                                  size_t state_stride, const int* __restrict__ cu_seqlens,
                                  const int* __restrict__ state_slots, int channels, int taps) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int start = cu_seqlens[r], len = cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  float* st = state + (size_t)state_slots[r] * state_stride;
  for (int j = 0; j < taps - 1; ++j) {
    const int src = len - (taps - 1) + j;
    const float v = src >= 0 ? in[(size_t)(start + src) * in_stride + col0 + c] : st[(size_t)(j + len) * channels + c];
    st[(size_t)j * channels + c] = v;
  }
}

extern "C" int tp_causal_conv(const float* in, int in_stride, int col0, const float* w, const float* b, float* state,
                              size_t state_stride, const int* cu_seqlens, const int* token_req, const int* state_slots,
                              float* out, int n, int n_req, int channels, int taps, hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_req >= 0 && channels > 0 && taps >= 1, "causal_conv: bad sizes");
  TP_REQUIRE(in_stride >= col0 + channels && state_stride >= (size_t)(taps - 1) * channels, "causal_conv: rows too short");
  if (n == 0) return 0;
  const int threads = channels >= 256 ? 256 : 64;
  const dim3 grid(n, (channels + threads - 1) / threads);
  TP_REQUIRE(grid.y <= 65535, "causal_conv: too many channels");
  hipLaunchKernelGGL(causal_conv_kernel, grid, dim3(threads), 0, s, in, in_stride, col0, w, b, state, state_stride,
                     cu_seqlens, token_req, state_slots, out, channels, taps);
  if (taps > 1 && n_req > 0)
    hipLaunchKernelGGL(conv_state_kernel, dim3(n_req, grid.y), dim3(threads), 0, s, in, in_stride, col0, state,
                       state_stride, cu_seqlens, state_slots, channels, taps);
  TP_CHECK_LAUNCH("causal_conv");
  return 0;
}

// ---- the recurrence ---------------------------------------------------------------------------
// Per head h (its inputs B and C are those of group h / (heads / groups)), with dt = softplus(dt_raw + dt_bias[h])
// and a = exp(-exp(a_log[h]) * dt):
//   S <- a S + dt * B x^T        (S is [state, head_dim], float32)
//   y  = S^T C + d_skip[h] * x
// xbc [n, channels] float32 holds, per token, x [heads * head_dim] | B [groups * state] | C [groups * state] (after
// the convolution); dt_raw is column dt_col0 + h of the projection's rows.
//
// A block owns one request, one head and PC = 256 / R value columns; R lanes (a power of two, one part of a
// wave) share a column and split the state index among them (n = lane + R i), NPT entries each in registers.
// Tokens are taken TC at a time: their B, C, x, dt and decay are staged in LDS by all threads, then the run over
// the chunk is register arithmetic, LDS broadcasts and one lane reduction per token.
struct ScanArgs {
  const float* xbc;
  const float* proj;
  int proj_stride, dt_col0;
  const float* dt_bias;
  const float* a_log;
  const float* d_skip;
  float* state;
  size_t state_stride, state_off;
  const int* cu_seqlens;
  const int* state_slots;
  float* y;
  int heads, head_dim, n_state, groups, channels;
  int R, TC;
};

template <int NPT>
__global__ __launch_bounds__(256) void ssm_scan_kernel(ScanArgs a) {
  extern __shared__ float lds[];
  const int N = a.n_state, P = a.head_dim, R = a.R, PC = 256 / a.R, TC = a.TC;
  float* Bs = lds;                 // [TC, N]
  float* Cs = Bs + (size_t)TC * N; // [TC, N]
  float* xs = Cs + (size_t)TC * N; // [TC, PC]
  float* dts = xs + (size_t)TC * PC;
  float* das = dts + TC;
  const int r = blockIdx.x, h = blockIdx.y, slice = blockIdx.z;
  const int col = threadIdx.x / R, rr = threadIdx.x % R;
  const int p = slice * PC + col;
  const bool active = p < P;
  const int g = h / (a.heads / a.groups);
  const int start = a.cu_seqlens[r], len = a.cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  const int inner = a.heads * P;
  float* S = a.state + (size_t)a.state_slots[r] * a.state_stride + a.state_off + (size_t)h * N * P;
  float st[NPT];
#pragma unroll
  for (int i = 0; i < NPT; ++i) {
    const int n = rr + R * i;
    st[i] = (active && n < N) ? S[(size_t)n * P + p] : 0.f;
  }
  const float A = -expf(a.a_log[h]);
  const float dtb = a.dt_bias[h], Dh = a.d_skip[h];
  for (int t0 = 0; t0 < len; t0 += TC) {
    const int nt = min(TC, len - t0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < nt * N; idx += 256) {
      const int tt = idx / N, n = idx % N;
      const float* row = a.xbc + (size_t)(start + t0 + tt) * a.channels + inner + g * N + n;
      Bs[idx] = row[0];
      Cs[idx] = row[(size_t)a.groups * N];
    }
    for (int idx = threadIdx.x; idx < nt * PC; idx += 256) {
      const int tt = idx / PC, pp = slice * PC + idx % PC;
      xs[idx] = pp < P ? a.xbc[(size_t)(start + t0 + tt) * a.channels + h * P + pp] : 0.f;
    }
    for (int idx = threadIdx.x; idx < nt; idx += 256) {
      const float dt = softplus_f(a.proj[(size_t)(start + t0 + idx) * a.proj_stride + a.dt_col0 + h] + dtb);
      dts[idx] = dt;
      das[idx] = expf(A * dt);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float dt = dts[tt], da = das[tt];
      const float xv = xs[tt * PC + col];
      const float dx = dt * xv;
      const float* Bt = Bs + (size_t)tt * N;
      const float* Ct = Cs + (size_t)tt * N;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NPT; ++i) {
        const int n = rr + R * i;
        if (n < N) {
          st[i] = fmaf(da, st[i], dx * Bt[n]);
          acc = fmaf(st[i], Ct[n], acc);
        }
      }
      for (int o = R >> 1; o > 0; o >>= 1) acc += __shfl_xor(acc, o, TP_WAVE);
      if (rr == 0 && active) a.y[(size_t)(start + t0 + tt) * inner + h * P + p] = fmaf(Dh, xv, acc);
    }
  }
#pragma unroll
  for (int i = 0; i < NPT; ++i) {
    const int n = rr + R * i;
    if (active && n < N) S[(size_t)n * P + p] = st[i];
  }
}

extern "C" int tp_ssm_scan(const float* xbc, const float* proj, int proj_stride, int dt_col0, const float* dt_bias,
                           const float* a_log, const float* d_skip, float* state, size_t state_stride, size_t state_off,
                           const int* cu_seqlens, const int* state_slots, float* y, int n_req, int heads, int head_dim,
                           int n_state, int groups, hipStream_t s) {
  TP_REQUIRE(n_req >= 0 && heads > 0 && head_dim > 0 && n_state > 0 && groups > 0 && heads % groups == 0, "ssm_scan: bad sizes");
  TP_REQUIRE(n_state <= 1024, "ssm_scan: state size %d exceeds 1024", n_state);
  TP_REQUIRE(state_stride >= state_off + (size_t)heads * n_state * head_dim, "ssm_scan: state rows too short");
  TP_REQUIRE(heads <= 65535, "ssm_scan: too many heads");
  if (n_req == 0) return 0;
  ScanArgs a;
  a.xbc = xbc; a.proj = proj; a.proj_stride = proj_stride; a.dt_col0 = dt_col0;
  a.dt_bias = dt_bias; a.a_log = a_log; a.d_skip = d_skip;
  a.state = state; a.state_stride = state_stride; a.state_off = state_off;
  a.cu_seqlens = cu_seqlens; a.state_slots = state_slots; a.y = y;
  a.heads = heads; a.head_dim = head_dim; a.n_state = n_state; a.groups = groups;
  a.channels = heads * head_dim + 2 * groups * n_state;
  // lanes per column: enough that a lane holds at most 8 state entries (16 beyond 512), and no more columns than
  // the head has values
  int R = 1;
  while (R < 64 && R * 8 < n_state) R *= 2;
  int pc_pow2 = 1;
  while (pc_pow2 < head_dim) pc_pow2 *= 2;
  while (R < 64 && 256 / R > pc_pow2) R *= 2;
  const int npt = (n_state + R - 1) / R;
  a.R = R;
  const int PC = 256 / R;
  const int per_token = 2 * n_state + PC + 2;
  int TC = (32 * 1024 / 4) / per_token;
  TC = TC < 1 ? 1 : (TC > 64 ? 64 : TC);
  a.TC = TC;
  const size_t shmem = (size_t)TC * per_token * sizeof(float);
  const dim3 grid(n_req, heads, (head_dim + PC - 1) / PC);
  TP_REQUIRE(grid.z <= 65535, "ssm_scan: head_dim too large");
#define SCAN_LAUNCH(NPT) hipLaunchKernelGGL(ssm_scan_kernel<NPT>, grid, dim3(256), shmem, s, a)
  if (npt <= 1) SCAN_LAUNCH(1);
  else if (npt <= 2) SCAN_LAUNCH(2);
  else if (npt <= 4) SCAN_LAUNCH(4);
  else if (npt <= 8) SCAN_LAUNCH(8);
  else SCAN_LAUNCH(16);
#undef SCAN_LAUNCH
  TP_CHECK_LAUNCH("ssm_scan");
  return 0;
}

// ---- gate, grouped norm, weight ---------------------------------------------------------------
// v = y * silu(z) (z: column z_col0 + j of the projection's rows), normed in `groups` equal parts, each by its own
// root mean square (eps inside the root), times w [inner]; out [n, inner] float32 or bfloat16.
// One block per (token, part).
template <typename TO>
__global__ void gated_group_norm_kernel(const float* __restrict__ y, const float* __restrict__ proj, int proj_stride,
                                        int z_col0, const float* __restrict__ w, float eps, TO* __restrict__ out, int inner,
                                        int part) {
  __shared__ float scratch[32];
  const int t = blockIdx.x, q = blockIdx.y;
  const float* yr = y + (size_t)t * inner + (size_t)q * part;
  const float* zr = proj + (size_t)t * proj_stride + z_col0 + (size_t)q * part;
  float ss = 0.f;
  for (int j = threadIdx.x; j < part; j += blockDim.x) {
    const float v = yr[j] * silu_f(zr[j]);
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)part + eps);
  TO* o = out + (size_t)t * inner + (size_t)q * part;
  const float* wr = w + (size_t)q * part;
  for (int j = threadIdx.x; j < part; j += blockDim.x) from_float(o + j, yr[j] * silu_f(zr[j]) * rstd * wr[j]);
}

extern "C" int tp_gated_group_norm(const float* y, const float* proj, int proj_stride, int z_col0, const float* w, float eps,
                                   void* out, int out_dt, int n, int inner, int groups, hipStream_t s) {
  TP_REQUIRE(n >= 0 && inner > 0 && groups > 0 && inner % groups == 0 && groups <= 65535, "gated_group_norm: bad sizes");
  if (n == 0) return 0;
  const int part = inner / groups;
  const int threads = part >= 2048 ? 1024 : (part >= 256 ? 256 : 64);
  const dim3 grid(n, groups);
  if (out_dt == TP_F32)
    hipLaunchKernelGGL(gated_group_norm_kernel<float>, grid, dim3(threads), 0, s, y, proj, proj_stride, z_col0, w, eps,
                       (float*)out, inner, part);
  else if (out_dt == TP_BF16)
    hipLaunchKernelGGL(gated_group_norm_kernel<bf16_t>, grid, dim3(threads), 0, s, y, proj, proj_stride, z_col0, w, eps,
                       (bf16_t*)out, inner, part);
  else
    TP_REQUIRE(false, "gated_group_norm: unknown dtype %d", out_dt);
  TP_CHECK_LAUNCH("gated_group_norm");
  return 0;
}

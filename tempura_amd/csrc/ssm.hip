// A selective state-space mixer (state-space duality form) over a batch of requests that each bring a run of
// tokens: short causal convolution with carried inputs, the recurrence over a per-request state, and the gated
// grouped norm behind it.  All arithmetic is float32; the state lives in float32 rows of a per-request state tensor
// (row = request slot): first the convolution's last taps - 1 inputs, [taps - 1, channels], oldest first, then
// the recurrent state, [heads, state, head_dim].
//
// A request r of the batch owns tokens cu_seqlens[r] .. cu_seqlens[r + 1] - 1 and the state row state_slots[r];
// everything is read from device memory, so the same launches serve prompt portions, single decoded tokens and
// captured steps.  How a prompt was cut changes rounding only.
#include <math.h>

#include "common.h"

__device__ inline float silu_f(float v) { return v / (1.0f + expf(-v)); }
// ln(1 + e^v) without overflow: max(v, 0) + ln(1 + e^-|v|)
__device__ inline float softplus_f(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// ---- causal convolution per channel (+ SiLU) --------------------------------------------------
// in: rows [n, in_stride] float32, the channels at column col0; w [taps, channels] (tap-major, so that the lanes of
// a wave read neighbouring weights; the last tap is the current token's), b [channels] or none.  The inputs before
// a run's first token come from the request's state row, from element state_off on (zeros for a fresh request).
// out [n, channels] = silu(conv + b), or conv + b itself when `act` is 0.
__global__ void causal_conv_kernel(const float* __restrict__ in, int in_stride, int col0, const float* __restrict__ w,
                                   const float* __restrict__ b, const float* __restrict__ state, size_t state_stride,
                                   const int* __restrict__ cu_seqlens, const int* __restrict__ token_req,
                                   const int* __restrict__ state_slots, float* __restrict__ out, int channels, int taps,
                                   int channel_blocks, size_t state_off, int act) {
  // (neighbouring blocks take neighbouring channels of one token: they read one row of the input after the other)
  const int t = blockIdx.x / channel_blocks;
  const int c = (blockIdx.x % channel_blocks) * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int r = token_req[t];
  const int start = cu_seqlens[r];
  const int i = t - start;
  const float* st = state + (size_t)state_slots[r] * state_stride + state_off;
  float acc = b != nullptr ? b[c] : 0.f;
  for (int k = 0; k < taps; ++k) {
    const int src = i - (taps - 1 - k);
    const float v = src >= 0 ? in[(size_t)(start + src) * in_stride + col0 + c] : st[(size_t)(taps - 1 + src) * channels + c];
    acc = fmaf(w[(size_t)k * channels + c], v, acc);
  }
  out[(size_t)t * channels + c] = act ? silu_f(acc) : acc;
}

// The state after a run: the last taps - 1 inputs of (carried inputs, then the run's).  In place, ascending: entry j
// takes entry j + len of the old state or an input of the run, and entries below j are never read again.
__global__ void conv_state_kernel(const float* __restrict__ in, int in_stride, int col0, float* __restrict__ state,
                                  size_t state_stride, const int* __restrict__ cu_seqlens,
                                  const int* __restrict__ state_slots, int channels, int taps, size_t state_off) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int start = cu_seqlens[r], len = cu_seqlens[r + 1] - start;
  if (len <= 0) return;
  float* st = state + (size_t)state_slots[r] * state_stride + state_off;
  for (int j = 0; j < taps - 1; ++j) {
    const int src = len - (taps - 1) + j;
    const float v = src >= 0 ? in[(size_t)(start + src) * in_stride + col0 + c] : st[(size_t)(j + len) * channels + c];
    st[(size_t)j * channels + c] = v;
  }
}

extern "C" int tp_causal_conv(const float* in, int in_stride, int col0, const float* w, const float* b, float* state,
                              size_t state_stride, size_t state_off, const int* cu_seqlens, const int* token_req,
                              const int* state_slots, float* out, int n, int n_req, int channels, int taps, int act,
                              hipStream_t s) {
  TP_REQUIRE(n >= 0 && n_req >= 0 && channels > 0 && taps >= 1, "causal_conv: bad sizes");
  TP_REQUIRE(in_stride >= col0 + channels && state_stride >= state_off + (size_t)(taps - 1) * channels, "causal_conv: rows too short");
  if (n == 0) return 0;
  const int threads = channels >= 256 ? 256 : 64;
  const int cb = (channels + threads - 1) / threads;
  TP_REQUIRE(cb <= 65535 && (long)n * cb < 0x7fffffffL, "causal_conv: too many channels or tokens");
  hipLaunchKernelGGL(causal_conv_kernel, dim3((unsigned)((long)n * cb)), dim3(threads), 0, s, in, in_stride, col0, w, b, state,
                     state_stride, cu_seqlens, token_req, state_slots, out, channels, taps, cb, state_off, act);
  if (taps > 1 && n_req > 0)
    hipLaunchKernelGGL(conv_state_kernel, dim3(n_req, cb), dim3(threads), 0, s, in, in_stride, col0, state,
                       state_stride, cu_seqlens, state_slots, channels, taps, state_off);
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
// A block owns one request, one head and PC = (256 / R) * TP value columns; a thread holds TN consecutive state
// entries of TP neighbouring columns in registers, and the R lanes (a power of two, neighbours in a wave) that share
// those columns split the state index among them.
// Tokens are taken TC at a time: their B, C, x, dt and decay are staged in LDS by all threads (rows padded with
// zeros to R * TN entries, so the run itself needs no bounds), then the run over the chunk is register
// arithmetic, 16-byte LDS reads that most lanes share, and one reduction over the R lanes per token (row
// permutes up to 16 lanes, which cost an instruction each and no trip through LDS).
//
// Long runs are cut into pieces of `piece` tokens that run side by side (a recurrence is a chain, and a prompt of
// thousands of tokens on a chain leaves most of the chip idle).  Three launches of the same kernel:
//   SCAN_LOCAL   every piece from a zero state: its end state and its total decay, to scratch;
//   SCAN_CARRY   per (request, head, columns), piece by piece: the state a piece starts from is
//                decay(previous piece) * (state the previous piece started from) + (its end state from zero);
//                the state after the last piece is the request's new state;
//   SCAN_OUTPUT  every piece again from the state it starts from, now writing y.
// Short runs (single tokens above all) take SCAN_DIRECT: one launch, from the request's state to its new state.
// How a run is cut changes rounding only.
enum { SCAN_DIRECT = 0, SCAN_LOCAL = 1, SCAN_CARRY = 2, SCAN_OUTPUT = 3 };

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
  int mode, piece, max_pieces;
  float* piece_state;   // [request, head, piece, n_state, head_dim]
  float* piece_decay;   // [request, head, piece]
};

// sum over the R lanes (R a power of two, the lanes neighbours from a multiple of R on); every lane gets it
__device__ inline float lanes_sum(float v, int R) {
#define DPP_ADD(ctrl) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, false))
  if (R >= 2) DPP_ADD(0xB1);    // quad_perm [1, 0, 3, 2]
  if (R >= 4) DPP_ADD(0x4E);    // quad_perm [2, 3, 0, 1]
  if (R >= 8) DPP_ADD(0x141);   // row_half_mirror: lane i of eight reads lane 7 - i
  if (R >= 16) DPP_ADD(0x140);  // row_mirror: lane i of sixteen reads lane 15 - i
#undef DPP_ADD
  if (R >= 32) v += __shfl_xor(v, 16, TP_WAVE);
  if (R >= 64) v += __shfl_xor(v, 32, TP_WAVE);
  return v;
}

template <int TN, int TP>
__global__ __launch_bounds__(256) void ssm_scan_kernel(ScanArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int N = a.n_state, P = a.head_dim, R = a.R, CG = 256 / a.R, PC = CG * TP, TC = a.TC;
  const int NS = R * TN;           // padded row of B and C
  float* Bs = lds;                 // [TC, NS]
  float* Cs = Bs + (size_t)TC * NS;
  float* xs = Cs + (size_t)TC * NS; // [TC, PC]
  float* dts = xs + (size_t)TC * PC;
  float* das = dts + TC;
  const int r = blockIdx.x, h = blockIdx.y;
  const int slices = (P + PC - 1) / PC;
  const int slice = blockIdx.z % slices, pc = blockIdx.z / slices;
  const int cg = threadIdx.x / R, rr = threadIdx.x % R;
  const int p0 = slice * PC + cg * TP;      // this thread's first value column
  const int g = h / (a.heads / a.groups);
  const int run0 = a.cu_seqlens[r], run_len = a.cu_seqlens[r + 1] - run0;
  if (run_len <= 0) return;
  const int inner = a.heads * P;
  const int n0 = rr * TN;
  float* S = a.state + (size_t)a.state_slots[r] * a.state_stride + a.state_off + (size_t)h * N * P;
  const int pieces = a.mode == SCAN_DIRECT ? 1 : (run_len + a.piece - 1) / a.piece;
  float* PS = a.piece_state + ((size_t)(r * a.heads + h) * a.max_pieces) * N * P;
  float* PD = a.piece_decay + (size_t)(r * a.heads + h) * a.max_pieces;
#define SCAN_HAS(i, j) (n0 + (i) < N && p0 + (j) < P)
#define SCAN_AT(i, j) ((size_t)(n0 + (i)) * P + p0 + (j))

  if (a.mode == SCAN_CARRY) {
    // the state each piece starts from, in place of what it ended with from zero; then the request's new state
    float cur[TN][TP];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TP; ++j) cur[i][j] = SCAN_HAS(i, j) ? S[SCAN_AT(i, j)] : 0.f;
    for (int c = 0; c < pieces; ++c) {
      const float decay = PD[c];
      float* ps = PS + (size_t)c * N * P;
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TP; ++j)
          if (SCAN_HAS(i, j)) {
            const float local = ps[SCAN_AT(i, j)];
            ps[SCAN_AT(i, j)] = cur[i][j];
            cur[i][j] = fmaf(decay, cur[i][j], local);
          }
    }
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TP; ++j)
        if (SCAN_HAS(i, j)) S[SCAN_AT(i, j)] = cur[i][j];
    return;
  }
  if (pc >= pieces) return;
  const int start = a.mode == SCAN_DIRECT ? run0 : run0 + pc * a.piece;
  const int len = a.mode == SCAN_DIRECT ? run_len : min(a.piece, run_len - pc * a.piece);
  const float* init = a.mode == SCAN_DIRECT ? S : (a.mode == SCAN_OUTPUT ? PS + (size_t)pc * N * P : nullptr);
  float st[TN][TP];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TP; ++j) st[i][j] = (init != nullptr && SCAN_HAS(i, j)) ? init[SCAN_AT(i, j)] : 0.f;
  const float A = -expf(a.a_log[h]);
  const float dtb = a.dt_bias[h], Dh = a.d_skip[h];
  const bool write_y = a.mode != SCAN_LOCAL;
  float dt_sum = 0.f;
  for (int t0 = 0; t0 < len; t0 += TC) {
    const int nt = min(TC, len - t0);
    __syncthreads();
    // (a wave stages every fourth token, its lanes the entries of a row: no division in the loop)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int tt = wave; tt < nt; tt += 4) {
      const float* row = a.xbc + (size_t)(start + t0 + tt) * a.channels;
      for (int n = lane; n < NS; n += 64) {
        float bv = 0.f, cv = 0.f;
        if (n < N) {
          bv = row[inner + g * N + n];
          cv = row[inner + (a.groups + g) * N + n];
        }
        Bs[tt * NS + n] = bv;
        Cs[tt * NS + n] = cv;
      }
      for (int c = lane; c < PC; c += 64) {
        const int pp = slice * PC + c;
        xs[tt * PC + c] = pp < P ? row[h * P + pp] : 0.f;
      }
    }
    for (int idx = threadIdx.x; idx < nt; idx += 256) {
      const float dt = softplus_f(a.proj[(size_t)(start + t0 + idx) * a.proj_stride + a.dt_col0 + h] + dtb);
      dts[idx] = dt;
      das[idx] = expf(A * dt);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float dt = dts[tt], da = das[tt];
      float xv[TP], dx[TP], acc[TP];
#pragma unroll
      for (int j = 0; j < TP; ++j) {
        xv[j] = xs[tt * PC + cg * TP + j];
        dx[j] = dt * xv[j];
        acc[j] = 0.f;
      }
      const float* Bt = Bs + (size_t)tt * NS + n0;
      const float* Ct = Cs + (size_t)tt * NS + n0;
      float bv[TN], cv[TN];
      if constexpr (TN % 4 == 0) {
#pragma unroll
        for (int i = 0; i < TN; i += 4) {
          const float4 b4 = *(const float4*)(Bt + i), c4 = *(const float4*)(Ct + i);
          bv[i] = b4.x; bv[i + 1] = b4.y; bv[i + 2] = b4.z; bv[i + 3] = b4.w;
          cv[i] = c4.x; cv[i + 1] = c4.y; cv[i + 2] = c4.z; cv[i + 3] = c4.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < TN; ++i) {
          bv[i] = Bt[i];
          cv[i] = Ct[i];
        }
      }
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TP; ++j) {
          st[i][j] = fmaf(da, st[i][j], dx[j] * bv[i]);
          acc[j] = fmaf(st[i][j], cv[i], acc[j]);
        }
      dt_sum += dt;
      if (write_y) {
#pragma unroll
        for (int j = 0; j < TP; ++j) {
          const float total = lanes_sum(acc[j], R);
          if (rr == 0 && p0 + j < P) a.y[(size_t)(start + t0 + tt) * inner + h * P + p0 + j] = fmaf(Dh, xv[j], total);
        }
      }
    }
  }
  if (a.mode == SCAN_OUTPUT) return;
  float* dst = a.mode == SCAN_DIRECT ? S : PS + (size_t)pc * N * P;
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TP; ++j)
      if (SCAN_HAS(i, j)) dst[SCAN_AT(i, j)] = st[i][j];
  if (a.mode == SCAN_LOCAL && slice == 0 && threadIdx.x == 0) PD[pc] = expf(A * dt_sum);
#undef SCAN_HAS
#undef SCAN_AT
}

// scratch floats a scan of n_req requests whose longest run has max_run tokens needs (0: it runs in one launch)
extern "C" size_t tp_ssm_scan_scratch(int n_req, int max_run, int heads, int head_dim, int n_state, int* piece_out) {
  int piece = 0;
  if (max_run > 256) {
    piece = 128;
    while ((max_run + piece - 1) / piece > 32) piece *= 2;    // at most 32 pieces a run
  }
  if (piece_out) *piece_out = piece;
  if (piece == 0) return 0;
  const size_t pieces = (size_t)((max_run + piece - 1) / piece);
  return (size_t)n_req * heads * pieces * ((size_t)n_state * head_dim + 1);
}

extern "C" int tp_ssm_scan(const float* xbc, const float* proj, int proj_stride, int dt_col0, const float* dt_bias,
                           const float* a_log, const float* d_skip, float* state, size_t state_stride, size_t state_off,
                           const int* cu_seqlens, const int* state_slots, float* y, int n_req, int heads, int head_dim,
                           int n_state, int groups, int max_run, float* scratch, size_t scratch_floats, hipStream_t s) {
  TP_REQUIRE(n_req >= 0 && heads > 0 && head_dim > 0 && n_state > 0 && groups > 0 && heads % groups == 0, "ssm_scan: bad sizes");
  TP_REQUIRE(n_state <= 2048, "ssm_scan: state size %d exceeds 2048", n_state);
  TP_REQUIRE(state_stride >= state_off + (size_t)heads * n_state * head_dim, "ssm_scan: state rows too short");
  TP_REQUIRE(heads <= 65535 && max_run >= 0, "ssm_scan: too many heads");
  if (n_req == 0) return 0;
  ScanArgs a;
  a.xbc = xbc; a.proj = proj; a.proj_stride = proj_stride; a.dt_col0 = dt_col0;
  a.dt_bias = dt_bias; a.a_log = a_log; a.d_skip = d_skip;
  a.state = state; a.state_stride = state_stride; a.state_off = state_off;
  a.cu_seqlens = cu_seqlens; a.state_slots = state_slots; a.y = y;
  a.heads = heads; a.head_dim = head_dim; a.n_state = n_state; a.groups = groups;
  a.channels = heads * head_dim + 2 * groups * n_state;
  // A thread holds TN state entries of TP value columns; the R lanes that share those columns split the state index.
  // Two columns a thread halve what a token's B and C cost in LDS reads for each update of the state; sixteen
  // entries a lane keep most of a wave's instructions the recurrence's own.  No more columns a block than the head has.
  const int TP = (head_dim >= 2 && n_state <= 1024) ? 2 : 1;
  const int cap = TP == 2 ? 16 : 32;
  int R = 1;
  while (R < 64 && R * cap < n_state) R *= 2;
  int pc_pow2 = 1;
  while (pc_pow2 < head_dim) pc_pow2 *= 2;
  while (R < 64 && (256 / R) * TP > pc_pow2) R *= 2;
  const int per_lane = (n_state + R - 1) / R;
  int tn = 1;
  while (tn < per_lane) tn *= 2;
  TP_REQUIRE(tn <= cap, "ssm_scan: state size %d does not fit a block", n_state);
  a.R = R;
  const int PC = (256 / R) * TP;
  const int per_token = 2 * R * tn + PC + 2;
  int TC = (32 * 1024 / 4) / per_token;
  TC = TC < 1 ? 1 : (TC > 64 ? 64 : TC);
  a.TC = TC;
  const size_t shmem = (size_t)TC * per_token * sizeof(float);
  const int slices = (head_dim + PC - 1) / PC;
  int piece = 0;
  const size_t need = tp_ssm_scan_scratch(n_req, max_run, heads, head_dim, n_state, &piece);
  a.piece = piece;
  a.max_pieces = piece ? (max_run + piece - 1) / piece : 1;
  a.piece_state = scratch;
  a.piece_decay = scratch ? scratch + (size_t)n_req * heads * a.max_pieces * n_state * head_dim : nullptr;
  TP_REQUIRE(piece == 0 || (scratch != nullptr && scratch_floats >= need), "ssm_scan: scratch of %zu floats needed", need);
  TP_REQUIRE((long)slices * a.max_pieces <= 65535, "ssm_scan: too many pieces");
#define SCAN_LAUNCH(TN_, TP_, GRID) hipLaunchKernelGGL((ssm_scan_kernel<TN_, TP_>), GRID, dim3(256), shmem, s, a)
#define SCAN_DISPATCH(GRID)                                \
  do {                                                     \
    if (TP == 2) {                                         \
      if (tn == 1) SCAN_LAUNCH(1, 2, GRID);                \
      else if (tn == 2) SCAN_LAUNCH(2, 2, GRID);           \
      else if (tn == 4) SCAN_LAUNCH(4, 2, GRID);           \
      else if (tn == 8) SCAN_LAUNCH(8, 2, GRID);           \
      else SCAN_LAUNCH(16, 2, GRID);                       \
    } else {                                               \
      if (tn == 1) SCAN_LAUNCH(1, 1, GRID);                \
      else if (tn == 2) SCAN_LAUNCH(2, 1, GRID);           \
      else if (tn == 4) SCAN_LAUNCH(4, 1, GRID);           \
      else if (tn == 8) SCAN_LAUNCH(8, 1, GRID);           \
      else if (tn == 16) SCAN_LAUNCH(16, 1, GRID);         \
      else SCAN_LAUNCH(32, 1, GRID);                       \
    }                                                      \
  } while (0)
  if (piece == 0) {
    a.mode = SCAN_DIRECT;
    SCAN_DISPATCH(dim3(n_req, heads, slices));
  } else {
    a.mode = SCAN_LOCAL;
    SCAN_DISPATCH(dim3(n_req, heads, slices * a.max_pieces));
    a.mode = SCAN_CARRY;
    SCAN_DISPATCH(dim3(n_req, heads, slices));
    a.mode = SCAN_OUTPUT;
    SCAN_DISPATCH(dim3(n_req, heads, slices * a.max_pieces));
  }
#undef SCAN_DISPATCH
#undef SCAN_LAUNCH
  TP_CHECK_LAUNCH("ssm_scan");
  return 0;
}

// ---- gate, grouped norm, weight ---------------------------------------------------------------
// v = y * silu(z) (z: column z_col0 + j of the projection's rows), normed in `groups` equal parts, each by its own
// root mean square (eps inside the root), times w [inner]; out [n, inner] float32 or bfloat16.
// One block per (token, part).
#define GN_ITEMS 8   // values a thread keeps between the sum and the store (parts up to 8 x the block)
template <typename TO>
__global__ void gated_group_norm_kernel(const float* __restrict__ y, const float* __restrict__ proj, int proj_stride,
                                        int z_col0, const float* __restrict__ w, float eps, TO* __restrict__ out, int inner,
                                        int part) {
  __shared__ float scratch[32];
  const int t = blockIdx.x, q = blockIdx.y;
  const float* yr = y + (size_t)t * inner + (size_t)q * part;
  const float* zr = proj + (size_t)t * proj_stride + z_col0 + (size_t)q * part;
  TO* o = out + (size_t)t * inner + (size_t)q * part;
  const float* wr = w + (size_t)q * part;
  if (part <= GN_ITEMS * (int)blockDim.x) {
    float v[GN_ITEMS];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < GN_ITEMS; ++i) {
      const int j = threadIdx.x + i * blockDim.x;
      v[i] = j < part ? yr[j] * silu_f(zr[j]) : 0.f;
      ss = fmaf(v[i], v[i], ss);
    }
    const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)part + eps);
#pragma unroll
    for (int i = 0; i < GN_ITEMS; ++i) {
      const int j = threadIdx.x + i * blockDim.x;
      if (j < part) from_float(o + j, v[i] * rstd * wr[j]);
    }
    return;
  }
  float ss = 0.f;
  for (int j = threadIdx.x; j < part; j += blockDim.x) {
    const float v = yr[j] * silu_f(zr[j]);
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)part + eps);
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

// hyb_kernels.hip -- the non-GEMM kernels of layer-list ("hybrid") decoders on ragged batches: a step's tokens are ONE flat row range, entry s of the batch owns rows
// [seq_start[s], seq_start[s + 1]) at positions seq_pos0[s] + i, so prompt portions of any length and single decoded tokens run in the same launches.
//
//   embedding gather, RMS norm (plain or one-plus weights; also the per-token 1 / rms for later consumers), grouped RMS norm,
//   short causal convolution + SiLU with carried taps, the state-space-duality recurrence with a carried f32 state,
//   whole-projection query / key norm + interleaved partial rotary + paged K / V write, paged attention with a sliding window and kept first tokens,
//   sigmoid top-k routing, stable expert dispatch, scaled row gather, SiLU-GLU, weighted combine with a gated shared expert.
//   Options that later designs added next to these: the recurrence with fixed decays or with step values from the caller and a column of ones, query / key norms per head,
//   attention inside position chunks with a learned sink and one gate logit per head, a router bias with a softmax over the chosen logits (the delta-rule and
//   exponential-gate kernels are in hyb_recur.hip).
//
// What is f32 regardless of the serving dtype: the residual stream, every norm, positions and angles, scores / softmax / the weighted value sum, router logits and
// scores, decays, step sizes and the recurrent state.  T below is the dtype of GEMM operands and of the K / V pages: bf16, or f32 in the all-f32 mode.
#include "common.cuh"
#include <float.h>

namespace mrs {
namespace hyb {

static thread_local char g_err[256];
static int fail(const char *m) { snprintf(g_err, sizeof g_err, "%s", m); return 1; }
static int ok_or(const char *what) {
  if (hipGetLastError() == hipSuccess) return 0;
  snprintf(g_err, sizeof g_err, "%s: launch failed", what);
  return 1;
}

__device__ __forceinline__ float block_sum_256(float v, float *red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}
__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// ---------------------------------------------------------------------------------- embedding rows -> f32 residual
template <class T> __global__ void __launch_bounds__(256) embed_kernel(const int *__restrict__ tokens, const T *__restrict__ table, float *__restrict__ x, int W, int vocab) {
  const int t = blockIdx.x;
  int id = tokens[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  for (int c = threadIdx.x; c < W; c += 256) x[(size_t)t * W + c] = to_f<T>(table[(size_t)id * W + c]);
}

// ---------------------------------------------------------------------------------- x / sqrt(mean(x^2) + eps) * (w | 1 + w); grid.y = equal parts of the row
// w null: no weight.  gate (optional, [rows, ldg]): gate_after 0: the row is multiplied by silu(gate) BEFORE its root mean square is taken; gate_after 1: the normed row is
// multiplied by silu(gate)
template <class T> __global__ void __launch_bounds__(256) rmsnorm_kernel(const float *__restrict__ x, int ldx, const float *__restrict__ w, T *__restrict__ out, float *__restrict__ out32,
                                                                          float *__restrict__ rstd, int part, float eps, int one_plus, int ldo, const float *__restrict__ gate, int ldg,
                                                                          int gate_after) {
  __shared__ float red[4];
  extern __shared__ float row[];  // the (gated) part, when a gate comes first: silu is evaluated once
  const int t = blockIdx.x, g = blockIdx.y;
  const float *xr = x + (size_t)t * ldx + (size_t)g * part;
  const float *gr = gate ? gate + (size_t)t * ldg + (size_t)g * part : nullptr;
  const bool pre = gr && !gate_after;
  float s = 0.f;
  for (int c = threadIdx.x; c < part; c += 256) {
    float v = xr[c];
    if (pre) { v *= silu_f(gr[c]); row[c] = v; }
    s = fmaf(v, v, s);
  }
  s = block_sum_256(s, red);
  const float inv = 1.0f / sqrtf(s / (float)part + eps);
  if (rstd && threadIdx.x == 0) rstd[(size_t)t * gridDim.y + g] = inv;
  for (int c = threadIdx.x; c < part; c += 256) {
    const float wv = w ? w[(size_t)g * part + c] : (one_plus ? 0.f : 1.0f);
    float v = (pre ? row[c] : xr[c]) * inv * (one_plus ? 1.0f + wv : wv);
    if (gr && gate_after) v *= silu_f(gr[c]);
    if (out) out[(size_t)t * ldo + (size_t)g * part + c] = from_f<T>(v);
    if (out32) out32[(size_t)t * ldo + (size_t)g * part + c] = v;
  }
}

// ---------------------------------------------------------------------------------- short causal convolution (+ SiLU) with carried taps
// u [rows, ldu] (the channels start at column 0 of the pointer handed in), cw [C, taps] (the last column multiplies the current token), state [slots, C, taps - 1]
// (oldest first).  An entry that starts at position 0 reads zeros instead of its slot.  in_bias (nullable, [C]): the bias of the product that made u -- the convolution
// runs over u + in_bias, and that is what the slot carries.  cb (nullable): the convolution's own bias.  act 1: SiLU of the result, 0: the result as it is.
// Where a convolved q | k | v channel goes when the convolution feeds attention directly (ROUTE): query channels times the query temperature
// 1 + coef ln(floor((pos + 1) / every) + 1) to q_out (T), key and value channels into the row's page slot (k_cache null: the rows carry queries only).
struct QkvRoute {
  void *q_out, *k_cache, *v_cache;
  const int *tok_pos;
  const long long *slot_mapping;
  int nq, nk, G, D, Dv, block_size, temp_every;
  float temp_coef;
};
template <class T> __device__ __forceinline__ void qkv_route(const QkvRoute &o, int t, int c, float v) {
  if (c < o.nq) {
    float f = 1.0f;
    if (o.temp_every > 0) f = 1.0f + o.temp_coef * logf((float)((o.tok_pos[t] + 1) / o.temp_every + 1));
    ((T *)o.q_out)[(size_t)t * o.nq + c] = from_f<T>(v * f);
    return;
  }
  if (!o.k_cache) return;
  const long long slot = o.slot_mapping[t];
  if (slot < 0) return;
  const long long blk = slot / o.block_size;
  const int off = (int)(slot % o.block_size);
  c -= o.nq;
  if (c < o.nk) {
    const int g = c / o.D, d = c % o.D;
    ((T *)o.k_cache)[(((size_t)blk * o.G + g) * o.block_size + off) * o.D + d] = from_f<T>(v);
  } else {
    c -= o.nk;
    const int g = c / o.Dv, d = c % o.Dv;
    ((T *)o.v_cache)[(((size_t)blk * o.G + g) * o.block_size + off) * o.Dv + d] = from_f<T>(v);
  }
}
// A thread owns one channel of CONV_ROWS consecutive rows and slides a register window of the last taps - 1 inputs along them (every input is loaded once, the taps' weights
// once); the window is filled afresh at the block's first row and wherever a new entry starts.  Taps in ascending order, as the step kernel adds them.
constexpr int CONV_ROWS = 8;
template <class T, bool ROUTE> __global__ void __launch_bounds__(256) conv_kernel(const float *__restrict__ u, int ldu, const float *__restrict__ in_bias, const float *__restrict__ cw,
                                                   const float *__restrict__ cb,
                                                   const float *__restrict__ state, const int *__restrict__ tok_seq, const int *__restrict__ seq_start, const int *__restrict__ seq_pos0,
                                                   const int *__restrict__ seq_slot, float *__restrict__ out, int C, int taps, int act, QkvRoute o, int rows) {
  const int t0 = blockIdx.x * CONV_ROWS, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int keep = taps - 1;
  const float ib = in_bias ? in_bias[c] : 0.f, b0 = cb ? cb[c] : 0.f;
  float w[16], win[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) w[k] = k < keep ? cw[(size_t)c * taps + k] : 0.f;
  const float w_cur = cw[(size_t)c * taps + keep];
#pragma unroll
  for (int r = 0; r < CONV_ROWS; ++r) {
    const int t = t0 + r;
    if (t >= rows) break;
    const int s = tok_seq[t], r0 = seq_start[s], i = t - r0;
    if (r == 0 || i == 0) {
      const bool carried = seq_pos0[s] > 0;
      const float *st = state + ((size_t)seq_slot[s] * C + c) * keep;
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        if (k >= keep) break;
        const int idx = i - keep + k;
        win[k] = idx >= 0 ? u[(size_t)(r0 + idx) * ldu + c] + ib : (carried ? st[keep + idx] : 0.f);
      }
    }
    const float cur = u[(size_t)t * ldu + c] + ib;
    float acc = b0;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      if (k >= keep) break;
      acc = fmaf(w[k], win[k], acc);
    }
    acc = fmaf(w_cur, cur, acc);
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      if (k >= keep) break;
      win[k] = k + 1 < keep ? win[k + 1] : cur;
    }
    if (ROUTE) qkv_route<T>(o, t, c, acc);
    else out[(size_t)t * C + c] = act ? silu_f(acc) : acc;
  }
}
// decode steps (every entry brings one row): convolution and tap shift in one launch, the thread of (entry, channel) reads its taps, then writes them
template <class T, bool ROUTE> __global__ void __launch_bounds__(256) conv_step_kernel(const float *__restrict__ u, int ldu, const float *__restrict__ in_bias, const float *__restrict__ cw,
                                                        const float *__restrict__ cb,
                                                        float *__restrict__ state, const int *__restrict__ seq_start, const int *__restrict__ seq_pos0, const int *__restrict__ seq_slot,
                                                        float *__restrict__ out, int C, int taps, int act, QkvRoute o) {
  const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int row = seq_start[s], keep = taps - 1;
  if (seq_start[s + 1] - row != 1) return;
  const bool carried = seq_pos0[s] > 0;
  float *st = state + ((size_t)seq_slot[s] * C + c) * keep;
  const float cur = u[(size_t)row * ldu + c] + (in_bias ? in_bias[c] : 0.f);
  float acc = cb ? cb[c] : 0.f, v[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    if (k >= keep) break;
    v[k] = carried ? st[k] : 0.f;
    acc = fmaf(cw[(size_t)c * taps + k], v[k], acc);
  }
  acc = fmaf(cw[(size_t)c * taps + keep], cur, acc);
  if (ROUTE) qkv_route<T>(o, row, c, acc);
  else out[(size_t)row * C + c] = act ? silu_f(acc) : acc;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    if (k >= keep) break;
    st[k] = k + 1 < keep ? v[k + 1] : cur;
  }
}
// the slot's taps after the step: the last taps - 1 inputs of (old taps ++ this step's rows).  One thread per (entry, channel) reads everything before it writes.
__global__ void __launch_bounds__(256) conv_state_kernel(const float *__restrict__ u, int ldu, const float *__restrict__ in_bias, float *__restrict__ state, const int *__restrict__ seq_start,
                                                         const int *__restrict__ seq_pos0, const int *__restrict__ seq_slot, int C, int taps) {
  const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = seq_start[s], len = seq_start[s + 1] - r0, keep = taps - 1;
  if (len <= 0) return;
  const bool carried = seq_pos0[s] > 0;
  float *st = state + ((size_t)seq_slot[s] * C + c) * keep;
  const float ib = in_bias ? in_bias[c] : 0.f;
  float v[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    if (k >= keep) break;
    const int idx = len - keep + k;
    v[k] = idx >= 0 ? u[(size_t)(r0 + idx) * ldu + c] + ib : (carried ? st[keep + idx] : 0.f);
  }
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    if (k >= keep) break;
    st[k] = v[k];
  }
}

// ---------------------------------------------------------------------------------- state-space-duality recurrence, f32 state carried in a slot
//   dt = softplus(dt_raw + dt_bias_h);  S <- exp(-exp(A_log_h) dt) S + dt B x^T  (S: N x P);  y = S^T C + D_h x          (the gate and the norm follow in rmsnorm_kernel)
// Step sizes and decays of all rows first (ssd_steps_kernel: the transcendental functions leave the serial chain).  The rows of an entry are cut into segments (a table
// the host builds); the recurrence is linear in S, so a long portion runs as
//   A  every segment but an entry's last, from a ZERO state: its local end state L_k and the product d_k of its decays          (parallel over segments)
//   B  init_(k+1) = d_k init_k + L_k, init_0 = the slot's state (zero for an entry that starts at position 0)                  (elementwise, serial over an entry's segments)
//   C  every segment from its init state: the outputs; an entry's last segment leaves the slot's new state                     (parallel over segments)
// and an entry of one segment (a decoded token, a short portion) is pass C alone.  Scan kernel: one wave per (segment, head, tile of P): lane = (p, r), r in [0, R) owns the
// state rows n in [r K, r K + K); the sum over n closes with R-lane butterflies.  No LDS, no barrier; DEPTH tokens' operands are in flight in a ring of register stages.
struct ScanArgs {
  const float *xbc;   // [rows, C]: x [heads * P] | B [G * N] | C [G * N] after convolution + SiLU
  const float *u;     // [rows, ldu] projection: dt_raw at column dt_col
  const float *dt_bias, *A_log, *D;   // D nullable (no skip term)
  const float *fixed_decay;  // [heads], nullable: every row steps with dt = 1 and this decay (dt_bias, A_log and the dt column of u are not read): S <- decay_h S + B x^T
  float *steps;       // [rows, heads, 2]: dt, decay
  float *state;       // [slots, heads, N, P]
  float *out;         // [rows, heads * P]
  const int *seq_pos0, *seq_slot;
  const int *seg_entry, *seg_row0, *seg_len, *ent_seg0;  // segment table: entry, first row, rows; first segment of every entry (+ the total)
  float *carry;       // [segments, heads, N, P]: L_k, then init_(k+1)
  float *decay;       // [segments, heads]: d_k
  int C, ldu, dt_col, heads, P, N, G, rows;
  int Pin;            // value columns that xbc carries per head; P - Pin (0 or 1) further columns of the state take x = 1 (a running sum of dt B next to the outer products)
  int ext_steps;      // `steps` was filled by the caller (gates of another form): nothing of dt_bias / A_log / fixed_decay is read
  float c_mult;       // every C value is multiplied by this when it is read (a query scale)
};
__global__ void __launch_bounds__(256) ssd_steps_kernel(ScanArgs a) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= a.rows * a.heads) return;
  const int t = i / a.heads, h = i % a.heads;
  if (a.fixed_decay) {
    a.steps[2 * (size_t)i] = 1.0f;
    a.steps[2 * (size_t)i + 1] = a.fixed_decay[h];
    return;
  }
  const float dt = softplus_f(a.u[(size_t)t * a.ldu + a.dt_col + h] + a.dt_bias[h]);
  a.steps[2 * (size_t)i] = dt;
  a.steps[2 * (size_t)i + 1] = expf(-expf(a.A_log[h]) * dt);
}
__global__ void __launch_bounds__(256) ssd_carry_kernel(ScanArgs a) {
  const int e = blockIdx.x * 256 + threadIdx.x, h = blockIdx.y, s = blockIdx.z;
  const int np = a.N * a.P;
  if (e >= np) return;
  const int z0 = a.ent_seg0[s], z1 = a.ent_seg0[s + 1];
  if (z1 - z0 < 2) return;
  float cur = a.seq_pos0[s] > 0 ? a.state[((size_t)a.seq_slot[s] * a.heads + h) * np + e] : 0.f;
  for (int z = z0; z < z1 - 1; ++z) {
    float *c = a.carry + ((size_t)z * a.heads + h) * np + e;
    cur = fmaf(a.decay[(size_t)z * a.heads + h], cur, *c);
    *c = cur;
  }
}
struct ScanStage {
  float x, dt, dec;
};
// LOCAL: pass A (zero start, no outputs, end state and decay product to `carry` / `decay`), else pass C
template <int R, int K, bool VEC, int DEPTH, bool LOCAL> __global__ void __launch_bounds__(64) ssd_scan_kernel(ScanArgs a) {
  constexpr int PT = 64 / R;
  const int lane = threadIdx.x, r = lane % R, p = blockIdx.x * PT + lane / R;
  const int h = blockIdx.y, z = blockIdx.z;
  const int s = a.seg_entry[z], r0 = a.seg_row0[z], len = a.seg_len[z];
  const bool first = z == a.ent_seg0[s], last = z == a.ent_seg0[s + 1] - 1;
  if (len <= 0 || (LOCAL && last)) return;
  const bool live = p < a.P;
  const int pc = live ? p : a.P - 1;
  const int g = h / (a.heads / a.G), inner = a.heads * a.Pin, inner_out = a.heads * a.P;
  const bool one_col = pc >= a.Pin;
  int nk = a.N - r * K;  // this lane's rows n = r K + k, k < nk
  nk = nk < 0 ? 0 : (nk > K ? K : nk);
  const size_t np = (size_t)a.N * a.P;
  float *st = a.state + ((size_t)a.seq_slot[s] * a.heads + h) * np;
  const float *init = LOCAL ? nullptr : (first ? (a.seq_pos0[s] > 0 ? st : nullptr) : a.carry + ((size_t)(z - 1) * a.heads + h) * np);
  float S[K];
#pragma unroll
  for (int k = 0; k < K; ++k) S[k] = (k < nk && init) ? init[(size_t)(r * K + k) * a.P + pc] : 0.f;
  const float Dh = a.D ? a.D[h] : 0.f;
  const int bcol = inner + g * a.N + r * K, ccol = inner + a.G * a.N + g * a.N + r * K;
  float B[DEPTH][K], Cv[DEPTH][K], prod = 1.0f;
  ScanStage sg[DEPTH];
  // unconditional requests (rows past the end re-read the last row; their step is made a no-op below): the waits before a stage's use then count exactly the
  // requests issued after it
  auto request = [&](int i, float *B_, float *C_, ScanStage &g_) {
    const int row = r0 + (i < len ? i : len - 1);
    const float *xr = a.xbc + (size_t)row * a.C;
    if (VEC) {
#pragma unroll
      for (int k = 0; k < K; k += 4) {
        const int kk = k < nk ? k : 0;  // lanes past the state size re-read a valid group (nk is a multiple of 4 here)
        const float4 b4 = *(const float4 *)(xr + (nk ? bcol : inner) + kk), c4 = *(const float4 *)(xr + (nk ? ccol : inner) + kk);
        const bool on = k < nk;
        B_[k] = on ? b4.x : 0.f; B_[k + 1] = on ? b4.y : 0.f; B_[k + 2] = on ? b4.z : 0.f; B_[k + 3] = on ? b4.w : 0.f;
        C_[k] = on ? c4.x * a.c_mult : 0.f; C_[k + 1] = on ? c4.y * a.c_mult : 0.f; C_[k + 2] = on ? c4.z * a.c_mult : 0.f; C_[k + 3] = on ? c4.w * a.c_mult : 0.f;
      }
    } else {
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const int kk = k < nk ? k : 0;
        const float bv = xr[(nk ? bcol : inner) + kk], cv = xr[(nk ? ccol : inner) + kk];
        B_[k] = k < nk ? bv : 0.f;
        C_[k] = k < nk ? cv * a.c_mult : 0.f;
      }
    }
    g_.x = one_col ? 1.0f : xr[h * a.Pin + pc];
    float d0, d1;
    if (DEPTH == 1 && !LOCAL && !a.ext_steps) {  // decode steps: the step size and decay inline (ssd_steps_kernel's expressions), one launch less
      if (a.fixed_decay) { d0 = 1.0f; d1 = a.fixed_decay[h]; }
      else {
        d0 = softplus_f(a.u[(size_t)row * a.ldu + a.dt_col + h] + a.dt_bias[h]);
        d1 = expf(-expf(a.A_log[h]) * d0);
      }
    } else {
      const float *de = a.steps + 2 * ((size_t)row * a.heads + h);
      d0 = de[0]; d1 = de[1];
    }
    g_.dt = i < len ? d0 : 0.f;    // past the end: S <- 1 S + 0
    g_.dec = i < len ? d1 : 1.f;
  };
#pragma unroll
  for (int j = 0; j < DEPTH; ++j) request(j, B[j], Cv[j], sg[j]);
  for (int i0 = 0; i0 < len; i0 += DEPTH) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      const int i = i0 + j;
      const float dx = sg[j].dt * sg[j].x, dec = sg[j].dec, xv = sg[j].x;
      float part = 0.f;
#pragma unroll
      for (int k = 0; k < K; ++k) {
        S[k] = fmaf(dec, S[k], dx * B[j][k]);
        if (!LOCAL) part = fmaf(S[k], Cv[j][k], part);
      }
      if (LOCAL) prod *= dec;
      if (DEPTH > 1 || i0 + DEPTH < len) request(i + DEPTH, B[j], Cv[j], sg[j]);
      if (!LOCAL) {
#pragma unroll
        for (int m = 1; m < R; m <<= 1) part += __shfl_xor(part, m, 64);
        if (r == 0 && live && i < len) a.out[(size_t)(r0 + i) * inner_out + h * a.P + p] = fmaf(Dh, xv, part);
      }
    }
  }
  if (LOCAL) {
    if (blockIdx.x == 0 && lane == 0) a.decay[(size_t)z * a.heads + h] = prod;
    st = a.carry + ((size_t)z * a.heads + h) * np;
  }
  if (live && (LOCAL || last))
#pragma unroll
    for (int k = 0; k < K; ++k)
      if (k < nk) st[(size_t)(r * K + k) * a.P + p] = S[k];
}

// The same recurrence for portions (segments of many rows), operands through LDS: the waves of one (segment, head) -- one per 64 / R values of P -- share the rows' B, C, x and
// step values.  TC rows are staged at a time with coalesced loads (every value is read from global memory once per head instead of once per lane group), the next TC rows
// are in registers while the current ones are consumed, and a lane reads its K state rows' B / C as broadcast 16-byte LDS reads.
template <int R, int K, bool VEC, bool LOCAL, int NT> __global__ void __launch_bounds__(NT) ssd_scan_lds_kernel(ScanArgs a, int rowpad) {
  constexpr int TC = 8;  // rows per stage; a thread stages columns tid and tid + nthr of every row (16 registers)
  extern __shared__ __attribute__((aligned(16))) float sm[];  // [2][TC][rowpad]: B [N] | C [N] | x [P] | dt | decay
  constexpr int PT = 64 / R;
  const int tid = threadIdx.x, nthr = blockDim.x, wave = tid >> 6, lane = tid & 63, r = lane % R, p = (blockIdx.x * (nthr >> 6) + wave) * PT + lane / R;
  const int h = blockIdx.y, z = blockIdx.z;
  const int s = a.seg_entry[z], r0 = a.seg_row0[z], len = a.seg_len[z];
  const bool first = z == a.ent_seg0[s], last = z == a.ent_seg0[s + 1] - 1;
  if (len <= 0 || (LOCAL && last)) return;
  const bool live = p < a.P;
  const int pc = live ? p : a.P - 1;
  const int g = h / (a.heads / a.G), inner = a.heads * a.Pin, inner_out = a.heads * a.P, N = a.N, P = a.P;
  int nk = N - r * K;
  nk = nk < 0 ? 0 : (nk > K ? K : nk);
  const size_t np = (size_t)N * P;
  float *st = a.state + ((size_t)a.seq_slot[s] * a.heads + h) * np;
  const float *init = LOCAL ? nullptr : (first ? (a.seq_pos0[s] > 0 ? st : nullptr) : a.carry + ((size_t)(z - 1) * a.heads + h) * np);
  float S[K];
#pragma unroll
  for (int k = 0; k < K; ++k) S[k] = (k < nk && init) ? init[(size_t)(r * K + k) * P + pc] : 0.f;
  const float Dh = a.D ? a.D[h] : 0.f;
  const int bcol = inner + g * N, ccol = inner + a.G * N + g * N, per = TC * rowpad, rowlen = 2 * N + P + 2;
  float stg[16], prod = 1.0f;
  auto fetch = [&](int c0) {
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int tok = q >> 1, j = tid + (q & 1) * nthr, i = c0 + tok;
      float v = 0.f;
      if (i < len && j < rowlen) {
        const int row = r0 + i;
        const float *xr = a.xbc + (size_t)row * a.C;
        if (j < N) v = xr[bcol + j];
        else if (j < 2 * N) v = xr[ccol + j - N] * a.c_mult;
        else if (j < 2 * N + P) v = j - 2 * N < a.Pin ? xr[h * a.Pin + j - 2 * N] : 1.0f;
        else v = a.steps[2 * ((size_t)row * a.heads + h) + (j - 2 * N - P)];
      }
      stg[q] = v;
    }
  };
  auto put = [&](float *buf) {
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int j = tid + (q & 1) * nthr;
      if (j < rowpad) buf[(q >> 1) * rowpad + j] = stg[q];
    }
  };
  fetch(0);
  put(sm);
  __syncthreads();
  int flip = 0;
  for (int c0 = 0; c0 < len; c0 += TC, flip ^= 1) {
    const float *cur = sm + flip * per;
    const bool more = c0 + TC < len;
    if (more) fetch(c0 + TC);
    const int cnt = len - c0 < TC ? len - c0 : TC;
    for (int j = 0; j < cnt; ++j) {
      const float *row = cur + j * rowpad;
      const float dt = row[2 * N + P], dec = row[2 * N + P + 1], xv = row[2 * N + pc];
      const float dx = dt * xv;
      float part = 0.f;
      if (VEC) {
#pragma unroll
        for (int k = 0; k < K; k += 4) {
          const int kk = r * K + (k < nk ? k : 0);
          const float4 b4 = *(const float4 *)(row + (nk ? kk : 0)), c4 = *(const float4 *)(row + N + (nk ? kk : 0));
          const bool on = k < nk;
          const float bb[4] = {on ? b4.x : 0.f, on ? b4.y : 0.f, on ? b4.z : 0.f, on ? b4.w : 0.f}, cc[4] = {on ? c4.x : 0.f, on ? c4.y : 0.f, on ? c4.z : 0.f, on ? c4.w : 0.f};
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            S[k + q] = fmaf(dec, S[k + q], dx * bb[q]);
            if (!LOCAL) part = fmaf(S[k + q], cc[q], part);
          }
        }
      } else {
#pragma unroll
        for (int k = 0; k < K; ++k) {
          const int kk = k < nk ? r * K + k : 0;
          const float bv = k < nk ? row[kk] : 0.f, cv = k < nk ? row[N + kk] : 0.f;
          S[k] = fmaf(dec, S[k], dx * bv);
          if (!LOCAL) part = fmaf(S[k], cv, part);
        }
      }
      if (LOCAL) prod *= dec;
      else {
#pragma unroll
        for (int m = 1; m < R; m <<= 1) part += __shfl_xor(part, m, 64);
        if (r == 0 && live) a.out[(size_t)(r0 + c0 + j) * inner_out + h * P + p] = fmaf(Dh, xv, part);
      }
    }
    if (more) put(sm + (flip ^ 1) * per);
    __syncthreads();
  }
  if (LOCAL) {
    if (tid == 0) a.decay[(size_t)z * a.heads + h] = prod;
    st = a.carry + ((size_t)z * a.heads + h) * np;
  }
  if (live && (LOCAL || last))
#pragma unroll
    for (int k = 0; k < K; ++k)
      if (k < nk) st[(size_t)(r * K + k) * P + p] = S[k];
}

// ---------------------------------------------------------------------------------- query / key norm over the whole projection, partial interleaved rotary, K / V page write
struct QkArgs {
  const float *qkv;   // [rows, ld]: q [H * D] | k [G * D] | v [G * Dv]
  const float *qw, *kw;  // plain norm weights over the whole projection (null: no norm)
  const float *freq;  // [rot / 2] angular frequencies
  const int *tok_pos;
  const long long *slot_mapping;  // [rows] page slot = block * block_size + offset
  void *q_out;        // [rows, H * D] in T
  void *k_cache, *v_cache;  // [blocks, G, block_size, D | Dv] in T
  int ld, H, G, D, Dv, rot, block_size;
  float eps;
  int per_head;       // the norm runs over every head's D values with weights [D] shared by the heads, instead of over the whole projection with weights [H * D]
};
template <class T> __global__ void __launch_bounds__(256) qk_norm_rope_cache_kernel(QkArgs a) {
  __shared__ float red[4];
  extern __shared__ float head_inv[];  // per_head: 1 / rms of every query and key head
  const int t = blockIdx.x, tid = threadIdx.x;
  const int nq = a.H * a.D, nk = a.G * a.D, nv = a.G * a.Dv;
  const float *q = a.qkv + (size_t)t * a.ld, *k = q + nq, *v = k + nk;
  float iq = 1.f, ik = 1.f;
  if (a.per_head) {
    for (int j = tid >> 6; j < a.H + a.G; j += 4) {
      const float *src = q + (size_t)j * a.D;  // key heads follow the query heads in the row
      float s = 0.f;
      for (int d = tid & 63; d < a.D; d += 64) s = fmaf(src[d], src[d], s);
      s = wave_sum(s);
      if ((tid & 63) == 0) head_inv[j] = ((j < a.H ? a.qw : a.kw) != nullptr) ? 1.0f / sqrtf(s / (float)a.D + a.eps) : 1.0f;
    }
    __syncthreads();
  } else if (a.qw) {
    float s = 0.f;
    for (int c = tid; c < nq; c += 256) s = fmaf(q[c], q[c], s);
    iq = 1.0f / sqrtf(block_sum_256(s, red) / (float)nq + a.eps);
  }
  if (a.kw && !a.per_head) {
    float s = 0.f;
    for (int c = tid; c < nk; c += 256) s = fmaf(k[c], k[c], s);
    ik = 1.0f / sqrtf(block_sum_256(s, red) / (float)nk + a.eps);
  }
  const float pos = (float)a.tok_pos[t];
  const long long slot = a.slot_mapping[t];
  const long long blk = slot / a.block_size;
  const int off = (int)(slot % a.block_size);
  T *qo = (T *)a.q_out + (size_t)t * nq;
  for (int e2 = tid; e2 < (nq + nk) / 2; e2 += 256) {
    const bool is_q = e2 < nq / 2;
    const int e = is_q ? 2 * e2 : 2 * e2 - nq;
    const float *src = is_q ? q : k;
    const float *w = is_q ? a.qw : a.kw;
    const int d = e % a.D;
    const float inv = a.per_head ? head_inv[(is_q ? 0 : a.H) + e / a.D] : (is_q ? iq : ik);
    float x0 = src[e] * inv, x1 = src[e + 1] * inv;
    if (w) { x0 *= w[a.per_head ? d : e]; x1 *= w[a.per_head ? d + 1 : e + 1]; }
    if (d < a.rot) {
      float sn, cs;
      sincosf(pos * a.freq[d >> 1], &sn, &cs);
      const float y0 = x0 * cs - x1 * sn, y1 = x1 * cs + x0 * sn;
      x0 = y0; x1 = y1;
    }
    if (is_q) { qo[e] = from_f<T>(x0); qo[e + 1] = from_f<T>(x1); }
    else if (slot >= 0) {
      const int g = e / a.D;
      T *kc = (T *)a.k_cache + (((size_t)blk * a.G + g) * a.block_size + off) * a.D + d;
      kc[0] = from_f<T>(x0); kc[1] = from_f<T>(x1);
    }
  }
  if (slot >= 0)
    for (int e = tid; e < nv; e += 256) {
      const int g = e / a.Dv, d = e % a.Dv;
      ((T *)a.v_cache)[(((size_t)blk * a.G + g) * a.block_size + off) * a.Dv + d] = from_f<T>(v[e]);
    }
}

// ---------------------------------------------------------------------------------- paged attention, sliding window with kept first tokens
// Query at position i sees key j <= i when i - j < window or j < keep_first (window <= 0: every j <= i).  One wave per (row, head): keys in passes of 64 (a lane = a key for the
// scores, a lane = value dimensions for the weighted sum), running maximum / sum in f32.  Options: softcap > 0: s <- softcap tanh(s / softcap) after the scale; sink: one
// more term e^0 in the softmax's denominator (a key of score 0 without a value); gate (f32 [rows, ldg], column head * Dv + d): the output is multiplied by sigmoid(gate).
struct AttnArgs {
  const void *q;        // [rows, H * D] in T
  const void *k_cache, *v_cache;
  const int *block_tables;  // [entries, max_blocks]
  const int *tok_seq, *tok_pos;
  void *out;            // [rows, H * Dv] in T
  int H, G, D, Dv, block_size, max_blocks, window, keep_first;
  float scale;
  float softcap;        // 0: none
  int sink;
  const float *gate;    // nullable
  int ldg;
  // single-row steps: `splits` > 1 workgroups (grid.z) share a row's key passes; each leaves its unnormalised sum, running maximum and sum in scratch
  // [splits, rows, H, Dv + 2] (f32) and attn_merge_kernel joins them in split order (the sink, the gate and the rounding happen there)
  float *scratch;
  int splits, rows;
  int token_major;      // K / V rows laid out [block, slot, kv head, dim] (a product's row-major output) instead of [block, kv head, slot, dim]
  int chunk;            // > 0: position i sees j <= i only inside its own chunk, floor(i / chunk) == floor(j / chunk), chunks counted from position 0 (window / keep_first unused)
  const float *sink_logit;  // [H], nullable: with `sink`, the extra term of head h is e^{sink_logit[h]} instead of e^0
  int gate_per_head;    // the gate holds ONE logit per (row, head) at column h (ldg >= H) instead of one per output value
};
__device__ __forceinline__ float sink_of(const AttnArgs &a, int h) { return a.sink_logit ? a.sink_logit[h] : 0.f; }
__device__ __forceinline__ const float *gate_row(const AttnArgs &a, int t, int h) {
  return a.gate ? a.gate + (size_t)t * a.ldg + (a.gate_per_head ? (size_t)h : (size_t)h * a.Dv) : nullptr;
}
__device__ __forceinline__ long long kv_row(const AttnArgs &a, const int *bt, int key, int g) {
  const long long blk = bt[key / a.block_size];
  const int off = key % a.block_size;
  return a.token_major ? (blk * a.block_size + off) * a.G + g : (blk * a.G + g) * a.block_size + off;
}
__device__ __forceinline__ float capped(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }
template <class T> struct Ld;
template <> struct Ld<bf16_t> {
  static __device__ __forceinline__ void v8(const bf16_t *p, float *o) {
    const int4 v = *(const int4 *)p;
    const unsigned u[4] = {(unsigned)v.x, (unsigned)v.y, (unsigned)v.z, (unsigned)v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) { o[2 * j] = __uint_as_float(u[j] << 16); o[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u); }
  }
  static __device__ __forceinline__ void v2(const bf16_t *p, float &x, float &y) {
    const unsigned u = *(const unsigned *)p;
    x = __uint_as_float(u << 16); y = __uint_as_float(u & 0xffff0000u);
  }
};
template <> struct Ld<float> {
  static __device__ __forceinline__ void v8(const float *p, float *o) {
    const float4 x = *(const float4 *)p, y = *(const float4 *)(p + 4);
    o[0] = x.x; o[1] = x.y; o[2] = x.z; o[3] = x.w; o[4] = y.x; o[5] = y.y; o[6] = y.z; o[7] = y.w;
  }
  static __device__ __forceinline__ void v2(const float *p, float &x, float &y) { const float2 v = *(const float2 *)p; x = v.x; y = v.y; }
};
// DVC: 128-wide pieces of the value size (a lane owns the dimension pair 2 lane, 2 lane + 1 of every piece).  VEC: key size a multiple of 8 and value size even: whole
// key rows in 16-byte loads, value pairs in one load.
template <class T, int DVC, bool VEC> __global__ void __launch_bounds__(64) paged_window_attn_kernel(AttnArgs a) {
  extern __shared__ float lds[];  // q [D] | p [64] | key row index [64]
  float *qs = lds, *ps = lds + ((a.D + 3) & ~3);
  long long *rowbase = (long long *)(ps + 64);
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = a.tok_seq[t], i = a.tok_pos[t], g = h / (a.H / a.G);
  const T *q = (const T *)a.q + ((size_t)t * a.H + h) * a.D;
  for (int d = lane; d < a.D; d += 64) qs[d] = to_f<T>(q[d]);
  const int *bt = a.block_tables + (size_t)s * a.max_blocks;
  int w_lo = a.window > 0 ? i - a.window + 1 : 0;
  if (w_lo < 0) w_lo = 0;
  if (a.chunk > 0) w_lo = (i / a.chunk) * a.chunk;
  int n1 = a.keep_first < w_lo ? a.keep_first : w_lo;  // kept first tokens that the window does not already cover
  if (n1 < 0 || a.chunk > 0) n1 = 0;
  int total = n1 + (i - w_lo + 1), v_begin = 0;
  const bool split = a.splits > 1;
  if (split) {  // this workgroup's share of the passes
    const int per = ((total + 63) / 64 + a.splits - 1) / a.splits;
    v_begin = blockIdx.z * per * 64;
    const int v_end = v_begin + per * 64;
    total = total < v_end ? total : v_end;
  }
  float m = (a.sink && !split) ? sink_of(a, h) : -FLT_MAX, l = (a.sink && !split) ? 1.f : 0.f, o[DVC][2];
#pragma unroll
  for (int c = 0; c < DVC; ++c) o[c][0] = o[c][1] = 0.f;
  MRS_WAVE_SYNC();
  for (int v0 = v_begin; v0 < total; v0 += 64) {
    const int vi = v0 + lane;
    float sc = -FLT_MAX;
    long long base = -1;
    if (vi < total) {
      const int key = vi < n1 ? vi : w_lo + (vi - n1);
      base = kv_row(a, bt, key, g);
      const T *kr = (const T *)a.k_cache + (size_t)base * a.D;
      float acc = 0.f;
      if (VEC) {
        for (int d = 0; d < a.D; d += 8) {
          float kv[8];
          Ld<T>::v8(kr + d, kv);
          const float4 qa = *(const float4 *)(qs + d), qb = *(const float4 *)(qs + d + 4);
          acc = fmaf(qa.x, kv[0], acc); acc = fmaf(qa.y, kv[1], acc); acc = fmaf(qa.z, kv[2], acc); acc = fmaf(qa.w, kv[3], acc);
          acc = fmaf(qb.x, kv[4], acc); acc = fmaf(qb.y, kv[5], acc); acc = fmaf(qb.z, kv[6], acc); acc = fmaf(qb.w, kv[7], acc);
        }
      } else {
        for (int d = 0; d < a.D; ++d) acc = fmaf(qs[d], to_f<T>(kr[d]), acc);
      }
      sc = capped(acc * a.scale, a.softcap);
    }
    const float mn = fmaxf(m, wave_max(sc));
    const float alpha = expf(m - mn);
    const float p = vi < total ? expf(sc - mn) : 0.f;  // (a split whose share is empty never gets here)
    l = l * alpha + wave_sum(p);
    m = mn;
    MRS_WAVE_SYNC();
    ps[lane] = p;
    rowbase[lane] = base;
    MRS_WAVE_SYNC();
    const int cnt = total - v0 < 64 ? total - v0 : 64;
#pragma unroll
    for (int c = 0; c < DVC; ++c) {
      const int d = 128 * c + 2 * lane;
      float a0 = o[c][0] * alpha, a1 = o[c][1] * alpha;
      if (d < a.Dv) {
        const T *vb = (const T *)a.v_cache + d;
        if (VEC) {
#pragma unroll 4
          for (int j = 0; j < cnt; ++j) {
            float x, y;
            Ld<T>::v2(vb + (size_t)rowbase[j] * a.Dv, x, y);
            a0 = fmaf(ps[j], x, a0);
            a1 = fmaf(ps[j], y, a1);
          }
        } else {
          const bool two = d + 1 < a.Dv;
          for (int j = 0; j < cnt; ++j) {
            const T *vr = vb + (size_t)rowbase[j] * a.Dv;
            a0 = fmaf(ps[j], to_f<T>(vr[0]), a0);
            if (two) a1 = fmaf(ps[j], to_f<T>(vr[1]), a1);
          }
        }
      }
      o[c][0] = a0; o[c][1] = a1;
    }
  }
  if (split) {
    float *part = a.scratch + (((size_t)blockIdx.z * a.rows + t) * a.H + h) * (a.Dv + 2);
#pragma unroll
    for (int c = 0; c < DVC; ++c) {
      const int d = 128 * c + 2 * lane;
      if (d < a.Dv) part[d] = o[c][0];
      if (d + 1 < a.Dv) part[d + 1] = o[c][1];
    }
    if (lane == 0) { part[a.Dv] = m; part[a.Dv + 1] = l; }
    return;
  }
  const float inv = 1.0f / l;
  T *out = (T *)a.out + ((size_t)t * a.H + h) * a.Dv;
  const float *gr = gate_row(a, t, h);
  const int gs = a.gate_per_head ? 0 : 1;
#pragma unroll
  for (int c = 0; c < DVC; ++c) {
    const int d = 128 * c + 2 * lane;
    if (d < a.Dv) out[d] = from_f<T>(o[c][0] * inv * (gr ? sigmoid_f(gr[gs * d]) : 1.0f));
    if (d + 1 < a.Dv) out[d + 1] = from_f<T>(o[c][1] * inv * (gr ? sigmoid_f(gr[gs * (d + 1)]) : 1.0f));
  }
}
// joins the splits of a row and head: M = max_s m_s (and 0 with the sink), L = sum_s l_s e^{m_s - M} (+ e^{-M}), out = sum_s o_s e^{m_s - M} / L (times sigmoid(gate))
template <class T> __global__ void __launch_bounds__(64) attn_merge_kernel(AttnArgs a) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, stride = a.Dv + 2;
  const float *base = a.scratch + ((size_t)t * a.H + h) * stride;
  const size_t step = (size_t)a.rows * a.H * stride;
  const float sv = sink_of(a, h);
  float M = a.sink ? sv : -FLT_MAX;
  for (int s = 0; s < a.splits; ++s) M = fmaxf(M, base[s * step + a.Dv]);
  float L = a.sink ? expf(sv - M) : 0.f;
  for (int s = 0; s < a.splits; ++s) L += base[s * step + a.Dv + 1] * expf(base[s * step + a.Dv] - M);
  const float inv = 1.0f / L;
  T *out = (T *)a.out + ((size_t)t * a.H + h) * a.Dv;
  const float *gr = gate_row(a, t, h);
  for (int d = lane; d < a.Dv; d += 64) {
    float acc = 0.f;
    for (int s = 0; s < a.splits; ++s) acc = fmaf(base[s * step + d], expf(base[s * step + a.Dv] - M), acc);
    out[d] = from_f<T>(acc * inv * (gr ? sigmoid_f(gr[a.gate_per_head ? 0 : d]) : 1.0f));
  }
}

// Portions: NQ consecutive queries of one entry (a tile of a segment) per wave.  A key row is loaded once and scored against all NQ queries (their vectors sit in LDS),
// a value pair is loaded once and added into NQ accumulators: 1 / NQ of the single-query kernel's loads for the same arithmetic.  Every query keeps its own running
// maximum / sum and its own visibility test (position i sees key j <= i with i - j < window or j < keep_first); the key range of the tile is the union of its queries' ranges.
template <class T, int DVC, int NQ> __global__ void __launch_bounds__(64) paged_window_attn_tile_kernel(AttnArgs a, const int *__restrict__ seg_entry, const int *__restrict__ seg_row0,
                                                                                                        const int *__restrict__ seg_len) {
  extern __shared__ __attribute__((aligned(16))) float lds[];  // q [NQ][Dp] | p [64][NQ] | key row index [64]
  const int z = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
  const int t0 = seg_row0[z] + blockIdx.x * NQ;
  int nq = seg_row0[z] + seg_len[z] - t0;
  if (nq <= 0) return;
  nq = nq > NQ ? NQ : nq;
  const int Dp = (a.D + 3) & ~3;
  float *qs = lds, *ps = lds + NQ * Dp;
  long long *rowbase = (long long *)(ps + 64 * NQ);
  const int s = seg_entry[z], i0 = a.tok_pos[t0], g = h / (a.H / a.G);
  for (int e = lane; e < NQ * Dp; e += 64) {
    const int q = e / Dp, d = e - q * Dp;
    qs[e] = (q < nq && d < a.D) ? to_f<T>(((const T *)a.q)[((size_t)(t0 + q) * a.H + h) * a.D + d]) : 0.f;
  }
  const int *bt = a.block_tables + (size_t)s * a.max_blocks;
  int w_lo = a.window > 0 ? i0 - a.window + 1 : 0;
  if (w_lo < 0) w_lo = 0;
  if (a.chunk > 0) w_lo = (i0 / a.chunk) * a.chunk;   // the first query's chunk; a later query of the tile may start a new one and then sees only part of the range
  int n1 = a.keep_first < w_lo ? a.keep_first : w_lo;
  if (n1 < 0 || a.chunk > 0) n1 = 0;
  const int total = n1 + (i0 + nq - 1 - w_lo + 1);
  float m[NQ], l[NQ], o[NQ][DVC][2];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    m[q] = a.sink ? sink_of(a, h) : -FLT_MAX; l[q] = a.sink ? 1.f : 0.f;
#pragma unroll
    for (int c = 0; c < DVC; ++c) o[q][c][0] = o[q][c][1] = 0.f;
  }
  MRS_WAVE_SYNC();
  for (int v0 = 0; v0 < total; v0 += 64) {
    const int vi = v0 + lane;
    int key = -1;
    long long base = -1;
    float sc[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) sc[q] = 0.f;
    if (vi < total) {
      key = vi < n1 ? vi : w_lo + (vi - n1);
      base = kv_row(a, bt, key, g);
      const T *kr = (const T *)a.k_cache + (size_t)base * a.D;
      for (int d = 0; d < a.D; d += 8) {
        float kv[8];
        Ld<T>::v8(kr + d, kv);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const float4 qa = *(const float4 *)(qs + q * Dp + d), qb = *(const float4 *)(qs + q * Dp + d + 4);
          float acc = sc[q];
          acc = fmaf(qa.x, kv[0], acc); acc = fmaf(qa.y, kv[1], acc); acc = fmaf(qa.z, kv[2], acc); acc = fmaf(qa.w, kv[3], acc);
          acc = fmaf(qb.x, kv[4], acc); acc = fmaf(qb.y, kv[5], acc); acc = fmaf(qb.z, kv[6], acc); acc = fmaf(qb.w, kv[7], acc);
          sc[q] = acc;
        }
      }
    }
    MRS_WAVE_SYNC();  // the previous pass has read p and the row indices
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int iq = i0 + q;
      const bool vis = key >= 0 && q < nq && key <= iq && (a.chunk > 0 ? key >= (iq / a.chunk) * a.chunk : (a.window <= 0 || iq - key < a.window || key < a.keep_first));
      const float sv = vis ? capped(sc[q] * a.scale, a.softcap) : -FLT_MAX;
      const float mn = fmaxf(m[q], wave_max(sv));
      const float alpha = expf(m[q] - mn);
      const float pq = vis ? expf(sv - mn) : 0.f;
      l[q] = l[q] * alpha + wave_sum(pq);
      m[q] = mn;
#pragma unroll
      for (int c = 0; c < DVC; ++c) { o[q][c][0] *= alpha; o[q][c][1] *= alpha; }
      ps[lane * NQ + q] = pq;
    }
    rowbase[lane] = base;
    MRS_WAVE_SYNC();
    const int cnt = total - v0 < 64 ? total - v0 : 64;
#pragma unroll
    for (int c = 0; c < DVC; ++c) {
      const int d = 128 * c + 2 * lane;
      if (d < a.Dv) {
        const T *vb = (const T *)a.v_cache + d;
#pragma unroll 2
        for (int j = 0; j < cnt; ++j) {
          float x, y;
          Ld<T>::v2(vb + (size_t)rowbase[j] * a.Dv, x, y);
          float pj[NQ];
#pragma unroll
          for (int q4 = 0; q4 < NQ; q4 += 4) {
            const float4 p4 = *(const float4 *)(ps + j * NQ + q4);
            pj[q4] = p4.x; pj[q4 + 1] = p4.y; pj[q4 + 2] = p4.z; pj[q4 + 3] = p4.w;
          }
#pragma unroll
          for (int q = 0; q < NQ; ++q) {
            o[q][c][0] = fmaf(pj[q], x, o[q][c][0]);
            o[q][c][1] = fmaf(pj[q], y, o[q][c][1]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    if (q >= nq) break;
    const float inv = 1.0f / l[q];
    T *out = (T *)a.out + ((size_t)(t0 + q) * a.H + h) * a.Dv;
    const float *gr = gate_row(a, t0 + q, h);
    const int gs = a.gate_per_head ? 0 : 1;
#pragma unroll
    for (int c = 0; c < DVC; ++c) {
      const int d = 128 * c + 2 * lane;
      if (d < a.Dv) {
        out[d] = from_f<T>(o[q][c][0] * inv * (gr ? sigmoid_f(gr[gs * d]) : 1.0f));
        out[d + 1] = from_f<T>(o[q][c][1] * inv * (gr ? sigmoid_f(gr[gs * (d + 1)]) : 1.0f));
      }
    }
  }
}

// ---------------------------------------------------------------------------------- mixture of experts: routing, dispatch, gather, GLU, combine
// Router: one workgroup per row.  logits z_e = w_e . h in f32 (a wave per expert, lanes over the width, butterfly sum); the `top` largest (ties: the lower index).
// SOFTMAX false: score = sigmoid(z), weights = the scores, un-renormalised; row E of the weight (when has_gate) is the shared expert's gate: gate[t] = sigmoid(w_E . h).
// SOFTMAX true: score = softmax(z) over ALL experts, weights = out_scale * the chosen scores, un-renormalised; with `chosen_only` the softmax runs over the chosen logits
// alone (the weights of a row sum to out_scale).  bias (nullable, [E]) is added to the logits.
template <bool SOFTMAX> __global__ void __launch_bounds__(1024) route_topk_kernel(const float *__restrict__ h, const float *__restrict__ wr, int W, int E, int top, int has_gate,
                                                                                  int *__restrict__ ids, float *__restrict__ wts, float *__restrict__ gate, float out_scale,
                                                                                  const float *__restrict__ bias, int chosen_only) {
  extern __shared__ float z[];  // [E + 1]
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float *hr = h + (size_t)t * W;
  const bool vec = (W & 3) == 0;
  for (int e = wave; e < E + (has_gate ? 1 : 0); e += 16) {
    const float *w = wr + (size_t)e * W;
    float acc = 0.f;
    if (vec) {
#pragma unroll 4
      for (int k = lane * 4; k < W; k += 256) {
        const float4 x4 = *(const float4 *)(hr + k), w4 = *(const float4 *)(w + k);
        acc = fmaf(x4.x, w4.x, acc); acc = fmaf(x4.y, w4.y, acc); acc = fmaf(x4.z, w4.z, acc); acc = fmaf(x4.w, w4.w, acc);
      }
    } else {
      for (int k = lane; k < W; k += 64) acc = fmaf(hr[k], w[k], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) z[e] = (bias && e < E) ? acc + bias[e] : acc;
  }
  __syncthreads();
  if (wave != 0) return;
  if (has_gate && lane == 0) gate[t] = sigmoid_f(z[E]);
  float zmax = 0.f, zden = 1.f;
  if (SOFTMAX && !chosen_only) {
    float mx = -FLT_MAX;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    zmax = wave_max(mx);
    float den = 0.f;
    for (int e = lane; e < E; e += 64) den += expf(z[e] - zmax);
    zden = wave_sum(den);
  }
  for (int k = 0; k < top; ++k) {
    float bv = -FLT_MAX;
    int be = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (z[e] > bv) { bv = z[e]; be = e; }  // ascending e: the first of equals stays
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) {
      const float ov = __shfl_xor(bv, m, 64);
      const int oe = __shfl_xor(be, m, 64);
      if (ov > bv || (ov == bv && oe < be)) { bv = ov; be = oe; }
    }
    if (SOFTMAX && chosen_only && k == 0) zmax = bv;  // the largest logit comes first
    if (lane == 0) {
      ids[(size_t)t * top + k] = be;
      wts[(size_t)t * top + k] = SOFTMAX ? (chosen_only ? expf(bv - zmax) : out_scale * (expf(bv - zmax) / zden)) : sigmoid_f(bv);
    }
    if ((be & 63) == lane) z[be] = -FLT_MAX;  // taken: written by the lane that reads this entry in the next round (every lane holds the same `be` after the butterfly)
  }
  if (SOFTMAX && chosen_only && lane == 0) {
    float den = 0.f;
    for (int k = 0; k < top; ++k) den += wts[(size_t)t * top + k];
    for (int k = 0; k < top; ++k) wts[(size_t)t * top + k] = out_scale * (wts[(size_t)t * top + k] / den);
  }
}
// stable counting sort of the routes by expert, one workgroup per expert: bounds [E + 1], sorted_route [R] (route index = token * top + k), route_pos [R] (its inverse),
// sorted_expert [R].  Every workgroup counts the routes below its expert (its base) and its own, then places its routes in ascending route order.
__global__ void __launch_bounds__(256) moe_dispatch_kernel(const int *__restrict__ ids, int R, int E, int *__restrict__ bounds, int *__restrict__ sorted_route,
                                                          int *__restrict__ route_pos, int *__restrict__ sorted_expert) {
  __shared__ int red[2][4];
  __shared__ int wcnt[4];
  const int e = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  int less = 0, eq = 0;
  for (int r = tid; r < R; r += 256) {
    const int id = ids[r];
    less += id < e;
    eq += id == e;
  }
  less = wave_sum(less);
  eq = wave_sum(eq);
  if (lane == 0) { red[0][wave] = less; red[1][wave] = eq; }
  __syncthreads();
  const int base = red[0][0] + red[0][1] + red[0][2] + red[0][3], cnt = red[1][0] + red[1][1] + red[1][2] + red[1][3];
  if (tid == 0) {
    bounds[e] = base;
    if (e == E - 1) bounds[E] = base + cnt;
  }
  if (cnt == 0) return;
  int running = base;
  for (int r0 = 0; r0 < R; r0 += 256) {
    const int r = r0 + tid;
    const bool mine = r < R && ids[r] == e;
    const unsigned long long bal = __ballot(mine);
    if (lane == 0) wcnt[wave] = __popcll(bal);
    __syncthreads();
    int off = running;
    for (int w = 0; w < wave; ++w) off += wcnt[w];
    if (mine) {
      const int at = off + __popcll(bal & ((1ull << lane) - 1ull));
      sorted_route[at] = r;
      route_pos[r] = at;
      sorted_expert[at] = e;
    }
    running += wcnt[0] + wcnt[1] + wcnt[2] + wcnt[3];
    __syncthreads();
  }
}
// row i of the expert-sorted operand = weight of its route * the token's normed row (f32), rounded once to T
template <class T> __global__ void __launch_bounds__(256) moe_gather_kernel(const float *__restrict__ h32, const int *__restrict__ sorted_route, const float *__restrict__ wts, int top,
                                                                            T *__restrict__ out, int W) {
  const int i = blockIdx.x, r = sorted_route[i], t = r / top;
  const float w = wts ? wts[r] : 1.0f;  // no weights: the rows are gathered as they are (the route's weight multiplies the expert's output instead)
  for (int c = threadIdx.x; c < W; c += 256) out[(size_t)i * W + c] = from_f<T>(w * h32[(size_t)t * W + c]);
}
// silu(gate) * up; gu [rows, 2 ff] = gate | up
template <class T> __global__ void __launch_bounds__(256) glu_silu_kernel(const float *__restrict__ gu, T *__restrict__ out, int rows, int ff) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)rows * ff) return;
  const size_t r = i / ff, c = i % ff;
  const float gv = gu[r * 2 * ff + c], uv = gu[r * 2 * ff + ff + c];
  out[i] = from_f<T>(silu_f(gv) * uv);
}
// g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha g) * (u + 1); gu [rows, 2 ff] = gate | up
__device__ __forceinline__ float glu_clamped_f(float gv, float uv, float limit, float alpha) {
  const float g = fminf(gv, limit), u = fminf(fmaxf(uv, -limit), limit);
  return g * sigmoid_f(alpha * g) * (u + 1.0f);
}
template <class T> __global__ void __launch_bounds__(256) glu_clamped_kernel(const float *__restrict__ gu, T *__restrict__ out, int rows, int ff, float limit, float alpha) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)rows * ff) return;
  const size_t r = i / ff, c = i % ff;
  out[i] = from_f<T>(glu_clamped_f(gu[r * 2 * ff + c], gu[r * 2 * ff + ff + c], limit, alpha));
}
// xIELU of (u + bias): z > 0: ap z^2 + z / 2;  z <= 0: an (e^z - 1 - z) + z / 2      (ap = softplus(p), an = 1 / 2 + softplus(q), both evaluated by the caller)
__device__ __forceinline__ float xielu_f(float z, float ap, float an) { return z > 0.f ? fmaf(ap * z, z, 0.5f * z) : fmaf(an, expm1f(z) - z, 0.5f * z); }
template <class T> __global__ void __launch_bounds__(256) bias_xielu_kernel(const float *__restrict__ u, int ldu, const float *__restrict__ bias, T *__restrict__ out, int rows, int ff,
                                                                            float ap, float an) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)rows * ff) return;
  const size_t r = i / ff, c = i % ff;
  out[i] = from_f<T>(xielu_f(u[r * ldu + c] + (bias ? bias[c] : 0.f), ap, an));
}
// out[t] (+)= sum_k w_k d[route_pos[t top + k]] + gate[t] * shared[t]        (w_k = wts[t top + k], or 1 without weights: the experts' inputs were scaled instead)
__global__ void __launch_bounds__(256) moe_combine_kernel(float *__restrict__ x, const float *__restrict__ d, const int *__restrict__ route_pos, int top, const float *__restrict__ shared,
                                                          const float *__restrict__ gate, int W, const float *__restrict__ wts, int accumulate) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const float v = d[(size_t)route_pos[(size_t)t * top + k] * W + c];
      acc = wts ? fmaf(wts[(size_t)t * top + k], v, acc) : acc + v;
    }
    if (shared) acc += (gate ? gate[t] : 1.0f) * shared[(size_t)t * W + c];
    x[(size_t)t * W + c] = accumulate ? x[(size_t)t * W + c] + acc : acc;
  }
}

// ---------------------------------------------------------------------------------- layer norm with weight and bias: (v - mean) / sqrt(mean((v - mean)^2) + eps) * w + b
// v = x (+ in_bias): the bias of the product that made x.  The result goes to out (T) and / or out32, and / or is ADDED to resid (the f32 residual stream: norms after a sublayer).
// With w2: the updated residual row is normed once more (weights w2, b2: the norm in front of the NEXT sublayer) and THAT goes to out / out32 -- two launches and a pass
// over the stream less per sublayer.
template <class T> __global__ void __launch_bounds__(256) layernorm_kernel(const float *__restrict__ x, int ldx, const float *__restrict__ in_bias, const float *__restrict__ w,
                                                                           const float *__restrict__ b, T *__restrict__ out, float *__restrict__ out32, float *__restrict__ resid, int ldr,
                                                                           int width, float eps, const float *__restrict__ w2, const float *__restrict__ b2) {
  __shared__ float red[4];
  extern __shared__ float row[];
  const int t = blockIdx.x;
  const float *xr = x + (size_t)t * ldx;
  float s = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = xr[c] + (in_bias ? in_bias[c] : 0.f);
    row[c] = v;
    s += v;
  }
  const float mean = block_sum_256(s, red) / (float)width;
  float q = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    const float dv = row[c] - mean;
    q = fmaf(dv, dv, q);
  }
  const float inv = 1.0f / sqrtf(block_sum_256(q, red) / (float)width + eps);
  if (w2) {
    float s2 = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) {
      const float r = resid[(size_t)t * ldr + c] + ((row[c] - mean) * inv * w[c] + (b ? b[c] : 0.f));
      resid[(size_t)t * ldr + c] = r;
      row[c] = r;
      s2 += r;
    }
    const float mean2 = block_sum_256(s2, red) / (float)width;
    float q2 = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) {
      const float dv = row[c] - mean2;
      q2 = fmaf(dv, dv, q2);
    }
    const float inv2 = 1.0f / sqrtf(block_sum_256(q2, red) / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += 256) {
      const float y = (row[c] - mean2) * inv2 * w2[c] + (b2 ? b2[c] : 0.f);
      if (out) out[(size_t)t * width + c] = from_f<T>(y);
      if (out32) out32[(size_t)t * width + c] = y;
    }
    return;
  }
  for (int c = threadIdx.x; c < width; c += 256) {
    const float y = (row[c] - mean) * inv * w[c] + (b ? b[c] : 0.f);
    if (out) out[(size_t)t * width + c] = from_f<T>(y);
    if (out32) out32[(size_t)t * width + c] = y;
    if (resid) resid[(size_t)t * ldr + c] += y;
  }
}

// ---------------------------------------------------------------------------------- projection biases, query temperature, K / V page write (no norm, no rotation)
// q <- (q + qb) * (1 + coef ln(floor((pos + 1) / every) + 1)) in f32, rounded once to T; k + kb and v + vb go to the page slot of the row (no k_cache: the layer reads another
// layer's pages and has no key / value columns)
struct QkvBiasArgs {
  const float *qkv;   // [rows, ld]: q [H * D] | k [G * D] | v [G * Dv] | ...
  const float *qb, *kb, *vb;  // nullable
  const int *tok_pos;
  const long long *slot_mapping;
  void *q_out, *k_cache, *v_cache;
  int ld, H, G, D, Dv, block_size, temp_every;
  float temp_coef;
};
template <class T> __global__ void __launch_bounds__(256) qkv_bias_temp_cache_kernel(QkvBiasArgs a) {
  const int t = blockIdx.x, tid = threadIdx.x;
  const int nq = a.H * a.D, nk = a.G * a.D, nv = a.G * a.Dv;
  const float *q = a.qkv + (size_t)t * a.ld;
  float f = 1.0f;
  if (a.temp_every > 0) f = 1.0f + a.temp_coef * logf((float)((a.tok_pos[t] + 1) / a.temp_every + 1));
  T *qo = (T *)a.q_out + (size_t)t * nq;
  for (int c = tid; c < nq; c += 256) qo[c] = from_f<T>((q[c] + (a.qb ? a.qb[c] : 0.f)) * f);
  if (!a.k_cache) return;
  const long long slot = a.slot_mapping[t];
  if (slot < 0) return;
  const long long blk = slot / a.block_size;
  const int off = (int)(slot % a.block_size);
  const float *k = q + nq, *v = k + nk;
  for (int e = tid; e < nk; e += 256) {
    const int g = e / a.D, d = e % a.D;
    ((T *)a.k_cache)[(((size_t)blk * a.G + g) * a.block_size + off) * a.D + d] = from_f<T>(k[e] + (a.kb ? a.kb[e] : 0.f));
  }
  for (int e = tid; e < nv; e += 256) {
    const int g = e / a.Dv, d = e % a.Dv;
    ((T *)a.v_cache)[(((size_t)blk * a.G + g) * a.block_size + off) * a.Dv + d] = from_f<T>(v[e] + (a.vb ? a.vb[e] : 0.f));
  }
}
// ---------------------------------------------------------------------------------- half-split rotary on f32 rows, in place (queries and keys of a recurrence)
// u [rows, ld]: `heads` heads of D values from column col.  In the first `rot` dimensions of a head, (x_i, x_{i + rot / 2}) turns by position * freq[i]; then every value of
// the head is multiplied by mult.  grid.y = 0: the range at q_col (mult 1), 1: the range at k_col (mult k_mult).
__global__ void __launch_bounds__(256) rotary_half_kernel(float *__restrict__ u, int ld, int q_col, int k_col, int heads, int D, int rot, const float *__restrict__ freq,
                                                          const int *__restrict__ tok_pos, float k_mult) {
  const int t = blockIdx.x, half = rot >> 1;
  float *row = u + (size_t)t * ld + (blockIdx.y ? k_col : q_col);
  const float mult = blockIdx.y ? k_mult : 1.0f, pos = (float)tok_pos[t];
  const int per = D - half;  // items of a head: `half` pairs, then the D - rot values that pass
  for (int e = threadIdx.x; e < heads * per; e += 256) {
    const int h = e / per, i = e - h * per;
    float *x = row + (size_t)h * D;
    if (i < half) {
      float sn, cs;
      sincosf(pos * freq[i], &sn, &cs);
      const float a = x[i], b = x[i + half];
      x[i] = (a * cs - b * sn) * mult;
      x[i + half] = (b * cs + a * sn) * mult;
    } else {
      x[i + half] *= mult;
    }
  }
}

// ---------------------------------------------------------------------------------- latent attention: the query rounded, the latent row normed and paged
// u [rows, ld] = q [nq] | c [R] (f32, one product): q goes to q_out (T) as it is; c / rms(c) * w (plain weight) goes to the row's page slot of c_cache [blocks, 1, block_size, R]
template <class T> __global__ void __launch_bounds__(256) latent_norm_cache_kernel(const float *__restrict__ u, int ld, int nq, int R, const float *__restrict__ w,
                                                                                   const long long *__restrict__ slot_mapping, T *__restrict__ q_out, T *__restrict__ c_cache, float eps) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float *q = u + (size_t)t * ld, *c = q + nq;
  for (int e = tid; e < nq; e += 256) q_out[(size_t)t * nq + e] = from_f<T>(q[e]);
  float s = 0.f;
  for (int e = tid; e < R; e += 256) s = fmaf(c[e], c[e], s);
  const float inv = 1.0f / sqrtf(block_sum_256(s, red) / (float)R + eps);
  const long long slot = slot_mapping[t];
  if (slot < 0) return;
  for (int e = tid; e < R; e += 256) c_cache[(size_t)slot * R + e] = from_f<T>(c[e] * inv * w[e]);
}

// ---------------------------------------------------------------------------------- several residual streams (hyper-connections)
// x [rows, S, W] f32.  One launch closes a sublayer and opens the next:
//   write  (y given): new_r = sum_s mix[s, r] x_s + outw[r] y for every stream r, all from the old streams (mix null: new_r = outw[r] y -- the streams' start)
//   read   (inw given): v = sum_s inw[s] x_s of the updated streams; norm_w given: v / rms(v) * (1 + norm_w | norm_w) to out (T) and / or out32; norm_w null: v itself to out32
template <class T, int S> __global__ void __launch_bounds__(256) hyper_step_kernel(float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ mix,
                                                                                   const float *__restrict__ outw, const float *__restrict__ inw, const float *__restrict__ norm_w,
                                                                                   T *__restrict__ out, float *__restrict__ out32, int W, float eps, int one_plus) {
  __shared__ float red[4];
  __shared__ float cm[S * S], co[S], ci[S];
  extern __shared__ float row[];  // the read sum, until its norm is known
  const int t = blockIdx.x, tid = threadIdx.x;
  if (tid < S * S) cm[tid] = mix ? mix[tid] : 0.f;
  if (tid < S) { co[tid] = outw ? outw[tid] : 0.f; ci[tid] = inw ? inw[tid] : 0.f; }
  __syncthreads();
  float *xr = x + (size_t)t * S * W;
  float ss = 0.f;
  for (int c = tid; c < W; c += 256) {
    float v[S];
    if (y) {
      const float yv = y[(size_t)t * W + c];
      float old[S];
      if (mix) {
#pragma unroll
        for (int s = 0; s < S; ++s) old[s] = xr[(size_t)s * W + c];
      }
#pragma unroll
      for (int r = 0; r < S; ++r) {
        float acc = 0.f;
        if (mix) {
#pragma unroll
          for (int s = 0; s < S; ++s) acc = fmaf(cm[s * S + r], old[s], acc);
        }
        v[r] = fmaf(co[r], yv, acc);
        xr[(size_t)r * W + c] = v[r];
      }
    } else {
#pragma unroll
      for (int s = 0; s < S; ++s) v[s] = xr[(size_t)s * W + c];
    }
    if (inw) {
      float uv = 0.f;
#pragma unroll
      for (int s = 0; s < S; ++s) uv = fmaf(ci[s], v[s], uv);
      if (norm_w) { row[c] = uv; ss = fmaf(uv, uv, ss); }
      else if (out32) out32[(size_t)t * W + c] = uv;
    }
  }
  if (!inw || !norm_w) return;
  const float inv = 1.0f / sqrtf(block_sum_256(ss, red) / (float)W + eps);
  for (int c = tid; c < W; c += 256) {
    const float v = row[c] * inv * (one_plus ? 1.0f + norm_w[c] : norm_w[c]);
    if (out) out[(size_t)t * W + c] = from_f<T>(v);
    if (out32) out32[(size_t)t * W + c] = v;
  }
}

__global__ void __launch_bounds__(256) gather_rows_kernel(const float *__restrict__ x, const int *__restrict__ idx, float *__restrict__ out, int W) {
  const int i = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) out[(size_t)i * W + c] = x[(size_t)idx[i] * W + c];
}

}  // namespace hyb
}  // namespace mrs

using namespace mrs::hyb;
#define S_(s) ((hipStream_t)(s))

extern "C" const char *mrs_hyb_last_error() { return g_err; }

extern "C" int mrs_hyb_embed(const int *tokens, const void *table, float *x, int rows, int W, int vocab, int dtype, void *stream) {
  if (rows <= 0) return 0;
  if (dtype == 1) hipLaunchKernelGGL(embed_kernel<mrs::bf16_t>, dim3(rows), dim3(256), 0, S_(stream), tokens, (const mrs::bf16_t *)table, x, W, vocab);
  else if (dtype == 2) hipLaunchKernelGGL(embed_kernel<float>, dim3(rows), dim3(256), 0, S_(stream), tokens, (const float *)table, x, W, vocab);
  else return fail("mrs_hyb_embed: dtype");
  return ok_or("mrs_hyb_embed");
}

// parts > 1: every row is normed in `parts` equal pieces, each by its own root mean square.  out (dtype) and / or out32 (f32) receive the result, rstd [rows, parts] the 1 / rms.
extern "C" int mrs_hyb_rmsnorm(const float *x, int ldx, const float *w, void *out, float *out32, float *rstd, int rows, int width, int parts, float eps, int one_plus, int dtype,
                               const float *gate, int ldg, int gate_after, void *stream) {
  if (rows <= 0) return 0;
  if (parts <= 0 || width % parts) return fail("mrs_hyb_rmsnorm: the row does not split into equal parts");
  dim3 grid(rows, parts);
  const size_t lds = gate && !gate_after ? (size_t)(width / parts) * 4 : 0;
  if (lds > 60000) return fail("mrs_hyb_rmsnorm: a gated part above 15000 values");
  if (dtype == 1) hipLaunchKernelGGL(rmsnorm_kernel<mrs::bf16_t>, grid, dim3(256), lds, S_(stream), x, ldx, w, (mrs::bf16_t *)out, out32, rstd, width / parts, eps, one_plus, width, gate, ldg, gate_after);
  else if (dtype == 2) hipLaunchKernelGGL(rmsnorm_kernel<float>, grid, dim3(256), lds, S_(stream), x, ldx, w, (float *)out, out32, rstd, width / parts, eps, one_plus, width, gate, ldg, gate_after);
  else return fail("mrs_hyb_rmsnorm: dtype");
  return ok_or("mrs_hyb_rmsnorm");
}

/* out [rows, C] = act(conv(u + in_bias) + cb): in_bias, cb nullable; act 1 = SiLU, 0 = none.  The slots carry the last taps - 1 rows of u + in_bias.  With a route (dtype
 * 1 | 2) the result goes to the query buffer / the K and V pages instead of `out`. */
static int conv_launch(const float *u, int ldu, const float *in_bias, const float *cw, const float *cb, float *state, const int *tok_seq, const int *seq_start,
                       const int *seq_pos0, const int *seq_slot, float *out, int rows, int entries, int C, int taps, int act, const QkvRoute &o, int dtype, void *stream) {
  if (rows <= 0) return 0;
  if (taps < 1 || taps > 17) return fail("mrs_hyb_conv: 1 .. 17 taps");
  if (taps > 1 && !state) return fail("mrs_hyb_conv: carried taps need their slots");
  dim3 g_rows((rows + CONV_ROWS - 1) / CONV_ROWS, (C + 255) / 256), g_ent(entries, (C + 255) / 256);
  const bool step = rows == entries;  // one row per entry (an entry without rows cannot occur then)
#define MRS_CONV(T, R) do { if (step) hipLaunchKernelGGL((conv_step_kernel<T, R>), g_ent, dim3(256), 0, S_(stream), u, ldu, in_bias, cw, cb, state, seq_start, seq_pos0, seq_slot, out, C, taps, act, o); \
                            else hipLaunchKernelGGL((conv_kernel<T, R>), g_rows, dim3(256), 0, S_(stream), u, ldu, in_bias, cw, cb, state, tok_seq, seq_start, seq_pos0, seq_slot, out, C, taps, act, o, rows); } while (0)
  if (dtype == 0) MRS_CONV(float, false);
  else if (dtype == 1) MRS_CONV(mrs::bf16_t, true);
  else if (dtype == 2) MRS_CONV(float, true);
  else return fail("mrs_hyb_conv: dtype");
#undef MRS_CONV
  if (!step && taps > 1)
    hipLaunchKernelGGL(conv_state_kernel, g_ent, dim3(256), 0, S_(stream), u, ldu, in_bias, state, seq_start, seq_pos0, seq_slot, C, taps);
  return ok_or("mrs_hyb_conv");
}
extern "C" int mrs_hyb_conv(const float *u, int ldu, const float *in_bias, const float *cw, const float *cb, float *state, const int *tok_seq, const int *seq_start,
                            const int *seq_pos0, const int *seq_slot, float *out, int rows, int entries, int C, int taps, int act, void *stream) {
  return conv_launch(u, ldu, in_bias, cw, cb, state, tok_seq, seq_start, seq_pos0, seq_slot, out, rows, entries, C, taps, act, QkvRoute{}, 0, stream);
}
/* The convolution over the q | k | v columns of u (+ in_bias, no activation) feeding attention in the same launch: q times the query temperature (temp_every <= 0: none) to
 * q_out (dtype), k and v into the rows' page slots.  k_cache null: u carries H * D query columns only. */
extern "C" int mrs_hyb_conv_qkv_cache(const float *u, int ldu, const float *in_bias, const float *cw, float *state, const int *tok_seq, const int *seq_start, const int *seq_pos0,
                                      const int *seq_slot, const int *tok_pos, const long long *slot_mapping, void *q_out, void *k_cache, void *v_cache, int rows, int entries, int H,
                                      int G, int D, int Dv, int block_size, int taps, float temp_coef, int temp_every, int dtype, void *stream) {
  if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || (k_cache && !v_cache) || !q_out) return fail("mrs_hyb_conv_qkv_cache: head sizes (heads % kv_heads == 0)");
  if (dtype != 1 && dtype != 2) return fail("mrs_hyb_conv_qkv_cache: dtype");
  const QkvRoute o{q_out, k_cache, v_cache, tok_pos, slot_mapping, H * D, G * D, G, D, Dv, block_size, temp_every, temp_coef};
  const int C = H * D + (k_cache ? G * D + G * Dv : 0);
  return conv_launch(u, ldu, in_bias, cw, nullptr, state, tok_seq, seq_start, seq_pos0, seq_slot, nullptr, rows, entries, C, taps, 0, o, dtype, stream);
}
extern "C" int mrs_hyb_conv_silu(const float *u, int ldu, const float *cw, const float *cb, float *state, const int *tok_seq, const int *seq_start, const int *seq_pos0,
                                 const int *seq_slot, float *out, int rows, int entries, int C, int taps, void *stream) {
  return mrs_hyb_conv(u, ldu, nullptr, cw, cb, state, tok_seq, seq_start, seq_pos0, seq_slot, out, rows, entries, C, taps, 1, stream);
}

/* steps: scratch [rows, heads, 2] f32.  Segment table (host-built): seg_entry / seg_row0 / seg_len [segments], ent_seg0 [entries + 1]; carry [segments, heads, N, P] and
 * decay [segments, heads] are scratch that is only touched when some entry has more than one segment (segments > entries). */
static int scan_launch(const float *xbc, const float *u, const float *dt_bias, const float *A_log, const float *D, const float *fixed_decay, float *state, float *out,
                       const int *seq_pos0, const int *seq_slot, const int *seg_entry, const int *seg_row0, const int *seg_len, const int *ent_seg0, float *steps, float *carry,
                       float *decay, int rows, int entries, int segments, int C, int ldu, int dt_col, int heads, int P, int N, int G, void *stream, int ones = 0,
                       int ext_steps = 0, float c_mult = 1.0f) {
  if (entries <= 0 || rows <= 0 || segments <= 0) return 0;
  if (heads <= 0 || G <= 0 || heads % G || P <= 0 || N <= 0) return fail("mrs_hyb_ssd_scan: bad head / group sizes");
  if (segments > 65535 || entries > 65535) return fail("mrs_hyb_ssd_scan: more than 65535 segments in one step");
  if (segments > entries && (!carry || !decay)) return fail("mrs_hyb_ssd_scan: segmented entries need the carry scratch");
  const int Pin = P;  // value columns the rows carry; the state has `ones` more
  P += ones ? 1 : 0;
  ScanArgs a{xbc, u, dt_bias, A_log, D, fixed_decay, steps, state, out, seq_pos0, seq_slot, seg_entry, seg_row0, seg_len, ent_seg0, carry, decay, C, ldu, dt_col, heads, P, N, G, rows,
             Pin, ext_steps ? 1 : 0, c_mult};
  const bool vec = C % 4 == 0 && (heads * Pin) % 4 == 0 && N % 4 == 0 && ((uintptr_t)xbc % 16) == 0;
  const bool single = rows == segments;  // one row per segment (decode steps): no ring, step sizes inline
  if (!single && !ext_steps) hipLaunchKernelGGL(ssd_steps_kernel, dim3((rows * heads + 255) / 256), dim3(256), 0, S_(stream), a);
  const bool split = segments > entries;
#define MRS_SCAN_(R, K, V, DP, L) hipLaunchKernelGGL((ssd_scan_kernel<R, K, V, DP, L>), dim3((P + 64 / R - 1) / (64 / R), heads, segments), dim3(64), 0, S_(stream), a)
#define MRS_SCAN_LDS_(R, K, V, L) do { if (nw <= 4) hipLaunchKernelGGL((ssd_scan_lds_kernel<R, K, V, L, 256>), dim3(nblk, heads, segments), dim3(64 * nw), lds_bytes, S_(stream), a, rowpad); \
                                       else hipLaunchKernelGGL((ssd_scan_lds_kernel<R, K, V, L, 1024>), dim3(nblk, heads, segments), dim3(64 * nw), lds_bytes, S_(stream), a, rowpad); } while (0)
  // portions: the LDS-staged kernel when two columns per thread cover a staged row; a head's P columns take workgroups of at most 16 waves (each stages the rows for itself)
  int nw = 0, nblk = 1;
  const int rowpad = (2 * N + P + 2 + 3) & ~3;
  const size_t lds_bytes = (size_t)2 * 8 * rowpad * 4;
  auto plan_lds = [&](int R_) {
    const int all = (P + 64 / R_ - 1) / (64 / R_);
    nblk = (all + 15) / 16;
    nw = (all + nblk - 1) / nblk;
    if (single || rowpad > 2 * 64 * nw || lds_bytes > 65536) nw = 0;
  };
#define MRS_SCAN(R, K, DP) do { \
    plan_lds(R); \
    if (split) { if (nw) { if (vec) MRS_SCAN_LDS_(R, K, true, true); else MRS_SCAN_LDS_(R, K, false, true); } \
                 else { if (vec) MRS_SCAN_(R, K, true, DP, true); else MRS_SCAN_(R, K, false, DP, true); } \
                 hipLaunchKernelGGL(ssd_carry_kernel, dim3((N * P + 255) / 256, heads, entries), dim3(256), 0, S_(stream), a); } \
    if (single) { if (vec) MRS_SCAN_(R, K, true, 1, false); else MRS_SCAN_(R, K, false, 1, false); } \
    else if (nw) { if (vec) MRS_SCAN_LDS_(R, K, true, false); else MRS_SCAN_LDS_(R, K, false, false); } \
    else { if (vec) MRS_SCAN_(R, K, true, DP, false); else MRS_SCAN_(R, K, false, DP, false); } } while (0)
  // (a head whose columns need more than sixteen waves -- a value size of 256 and the column of ones -- runs as two workgroups that each stage the rows; two lanes per
  // column with 64 state rows each, which would keep it in one, measured 1.8x slower, pieces of eight waves 1.1x slower)
  if (N <= 16) MRS_SCAN(2, 8, 8);
  else if (N <= 64) MRS_SCAN(4, 16, 6);
  else if (N <= 128) MRS_SCAN(4, 32, 4);
  else if (N <= 256) MRS_SCAN(8, 32, 4);
  else if (N <= 512) MRS_SCAN(16, 32, 4);
  else return fail("mrs_hyb_ssd_scan: state size above 512");
#undef MRS_SCAN_LDS_
#undef MRS_SCAN
#undef MRS_SCAN_
  return ok_or("mrs_hyb_ssd_scan");
}

extern "C" int mrs_hyb_ssd_scan(const float *xbc, const float *u, const float *dt_bias, const float *A_log, const float *D, float *state, float *out, const int *seq_pos0,
                                const int *seq_slot, const int *seg_entry, const int *seg_row0, const int *seg_len, const int *ent_seg0, float *steps, float *carry,
                                float *decay, int rows, int entries, int segments, int C, int ldu, int dt_col, int heads, int P, int N, int G, void *stream) {
  if (!dt_bias || !A_log || !D || !u) return fail("mrs_hyb_ssd_scan: step-size bias, decay rate and skip weight are needed");
  return scan_launch(xbc, u, dt_bias, A_log, D, nullptr, state, out, seq_pos0, seq_slot, seg_entry, seg_row0, seg_len, ent_seg0, steps, carry, decay, rows, entries, segments, C, ldu,
                     dt_col, heads, P, N, G, stream);
}
/* The same recurrence with one fixed decay per head and unit steps, S <- decay_h S + k v^T, o = S^T q (retention / decayed linear attention): xkq [rows, ld] holds
 * v [heads * P] | k [G * N] | q [G * N] from column 0; state [slots, heads, N, P] */
extern "C" int mrs_hyb_decay_scan(const float *xkq, int ld, const float *fixed_decay, float *state, float *out, const int *seq_pos0, const int *seq_slot, const int *seg_entry,
                                  const int *seg_row0, const int *seg_len, const int *ent_seg0, float *steps, float *carry, float *decay, int rows, int entries, int segments,
                                  int heads, int P, int N, int G, void *stream) {
  if (!fixed_decay) return fail("mrs_hyb_decay_scan: the heads' decays are needed");
  if (ld < heads * P + 2 * G * N) return fail("mrs_hyb_decay_scan: rows shorter than v | k | q");
  return scan_launch(xkq, nullptr, nullptr, nullptr, nullptr, fixed_decay, state, out, seq_pos0, seq_slot, seg_entry, seg_row0, seg_len, ent_seg0, steps, carry, decay, rows,
                     entries, segments, ld, 0, 0, heads, P, N, G, stream);
}

/* The same recurrence with step values the caller computed: steps [rows, heads, 2] = (what the state takes in, what it keeps) per row and head, S <- keep S + take k v^T,
 * o = S^T q; xkq [rows, ld] holds v [heads * P] | k [G * N] | q [G * N] from column 0.  ones != 0: the state has one more column per head that takes v = 1 (the running sum
 * of take * k beside the outer products): state [slots, heads, N, P + 1], out [rows, heads * (P + 1)], the last value of every head being that column's read-out.
 * q_mult: the queries are multiplied by it as they are read. */
extern "C" int mrs_hyb_gated_scan(const float *xkq, int ld, float *steps, float *state, float *out, const int *seq_pos0, const int *seq_slot, const int *seg_entry,
                                  const int *seg_row0, const int *seg_len, const int *ent_seg0, float *carry, float *decay, int rows, int entries, int segments,
                                  int heads, int P, int N, int G, int ones, float q_mult, void *stream) {
  if (!steps) return fail("mrs_hyb_gated_scan: the rows' step values are needed");
  if (ld < heads * P + 2 * G * N) return fail("mrs_hyb_gated_scan: rows shorter than v | k | q");
  return scan_launch(xkq, nullptr, nullptr, nullptr, nullptr, nullptr, state, out, seq_pos0, seq_slot, seg_entry, seg_row0, seg_len, ent_seg0, steps, carry, decay, rows,
                     entries, segments, ld, 0, 0, heads, P, N, G, stream, ones, 1, q_mult);
}

static int qk_launch(const float *qkv, int ld, const float *qw, const float *kw, const float *freq, const int *tok_pos, const long long *slot_mapping, void *q_out,
                     void *k_cache, void *v_cache, int rows, int H, int G, int D, int Dv, int rot, int block_size, float eps, int dtype, int per_head, void *stream) {
  if (rows <= 0) return 0;
  if ((D & 1) || (rot & 1) || rot > D || rot < 0 || H <= 0 || G <= 0 || H % G) return fail("mrs_hyb_qk_norm_rope_cache: head sizes (even dim, even rot <= dim, heads % kv_heads == 0)");
  QkArgs a{qkv, qw, kw, freq, tok_pos, slot_mapping, q_out, k_cache, v_cache, ld, H, G, D, Dv, rot, block_size, eps, per_head ? 1 : 0};
  const size_t lds = per_head ? (size_t)(H + G) * 4 : 0;
  if (lds > 32768) return fail("mrs_hyb_qk_norm_rope_cache: more than 8192 heads");
  if (dtype == 1) hipLaunchKernelGGL(qk_norm_rope_cache_kernel<mrs::bf16_t>, dim3(rows), dim3(256), lds, S_(stream), a);
  else if (dtype == 2) hipLaunchKernelGGL(qk_norm_rope_cache_kernel<float>, dim3(rows), dim3(256), lds, S_(stream), a);
  else return fail("mrs_hyb_qk_norm_rope_cache: dtype");
  return ok_or("mrs_hyb_qk_norm_rope_cache");
}
extern "C" int mrs_hyb_qk_norm_rope_cache(const float *qkv, int ld, const float *qw, const float *kw, const float *freq, const int *tok_pos, const long long *slot_mapping,
                                          void *q_out, void *k_cache, void *v_cache, int rows, int H, int G, int D, int Dv, int rot, int block_size, float eps, int dtype,
                                          void *stream) {
  return qk_launch(qkv, ld, qw, kw, freq, tok_pos, slot_mapping, q_out, k_cache, v_cache, rows, H, G, D, Dv, rot, block_size, eps, dtype, 0, stream);
}
/* the same with the query / key norm per head: every head's D values are divided by their own root mean square and multiplied by qw / kw [D], shared by the heads */
extern "C" int mrs_hyb_qk_headnorm_rope_cache(const float *qkv, int ld, const float *qw, const float *kw, const float *freq, const int *tok_pos, const long long *slot_mapping,
                                              void *q_out, void *k_cache, void *v_cache, int rows, int H, int G, int D, int Dv, int rot, int block_size, float eps, int dtype,
                                              void *stream) {
  return qk_launch(qkv, ld, qw, kw, freq, tok_pos, slot_mapping, q_out, k_cache, v_cache, rows, H, G, D, Dv, rot, block_size, eps, dtype, 1, stream);
}

/* seg_entry / seg_row0 / seg_len [segments] (nullable): the batch's segment table (rows of one entry in pieces); with it, batches that bring portions run the
 * query-tiled kernel */
static int attn_launch(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_seq, const int *tok_pos, void *out,
                       int rows, int H, int G, int D, int Dv, int block_size, int max_blocks, int window, int keep_first, float scale, int dtype,
                       const int *seg_entry, const int *seg_row0, const int *seg_len, int segments, int seg_rows, float softcap, int sink, const float *gate, int ldg,
                       float *scratch, int splits, int token_major, void *stream, int chunk = 0, const float *sink_logit = nullptr, int gate_per_head = 0) {
  if (rows <= 0) return 0;
  if (Dv > 512 || H % G) return fail("mrs_hyb_paged_window_attn: value size above 512 / heads % kv_heads");
  if (gate && ldg < (gate_per_head ? H : H * Dv)) return fail("mrs_hyb_paged_window_attn: gate rows shorter than heads (* value size)");
  if (chunk > 0 && (window > 0 || keep_first > 0)) return fail("mrs_hyb_paged_window_attn: chunks and a sliding window exclude each other");
  AttnArgs a{q, k_cache, v_cache, block_tables, tok_seq, tok_pos, out, H, G, D, Dv, block_size, max_blocks, window, keep_first, scale, softcap > 0.f ? softcap : 0.f, sink ? 1 : 0, gate, ldg, nullptr, 0, rows, token_major ? 1 : 0,
             chunk > 0 ? chunk : 0, sink ? sink_logit : nullptr, gate_per_head ? 1 : 0};
  const bool vec = D % 8 == 0 && Dv % 2 == 0 && ((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)v_cache % 8) == 0;
  const int c = (Dv + 127) / 128;
  if (vec && seg_entry && segments > 0 && rows > segments && segments <= 65535 && seg_rows > 0) {
    constexpr int NQ = 8;
    const size_t lds = (size_t)(NQ * ((D + 3) & ~3) + 64 * NQ) * 4 + 64 * 8;
    if (lds <= 65536) {
      dim3 grid((seg_rows + NQ - 1) / NQ, H, segments);
#define MRS_ATTN_T(T, C) hipLaunchKernelGGL((paged_window_attn_tile_kernel<T, C, NQ>), grid, dim3(64), lds, S_(stream), a, seg_entry, seg_row0, seg_len)
      if (dtype == 1) { if (c <= 1) MRS_ATTN_T(mrs::bf16_t, 1); else if (c <= 2) MRS_ATTN_T(mrs::bf16_t, 2); else MRS_ATTN_T(mrs::bf16_t, 4); }
      else if (dtype == 2) { if (c <= 1) MRS_ATTN_T(float, 1); else if (c <= 2) MRS_ATTN_T(float, 2); else MRS_ATTN_T(float, 4); }
      else return fail("mrs_hyb_paged_window_attn: dtype");
#undef MRS_ATTN_T
      return ok_or("mrs_hyb_paged_window_attn");
    }
  }
  const size_t lds = (size_t)(((D + 3) & ~3) + 64) * 4 + 64 * 8;
  if (scratch && splits > 1) {
    if (splits > 256) return fail("mrs_hyb_paged_window_attn: more than 256 key splits");
    a.scratch = scratch;
    a.splits = splits;
  }
  dim3 grid(rows, H, a.splits > 1 ? a.splits : 1);
#define MRS_ATTN(T, C) do { if (vec) hipLaunchKernelGGL((paged_window_attn_kernel<T, C, true>), grid, dim3(64), lds, S_(stream), a); \
                            else hipLaunchKernelGGL((paged_window_attn_kernel<T, C, false>), grid, dim3(64), lds, S_(stream), a); } while (0)
  if (dtype == 1) { if (c <= 1) MRS_ATTN(mrs::bf16_t, 1); else if (c <= 2) MRS_ATTN(mrs::bf16_t, 2); else MRS_ATTN(mrs::bf16_t, 4); }
  else if (dtype == 2) { if (c <= 1) MRS_ATTN(float, 1); else if (c <= 2) MRS_ATTN(float, 2); else MRS_ATTN(float, 4); }
  else return fail("mrs_hyb_paged_window_attn: dtype");
#undef MRS_ATTN
  if (a.splits > 1) {
    if (dtype == 1) hipLaunchKernelGGL(attn_merge_kernel<mrs::bf16_t>, dim3(rows, H), dim3(64), 0, S_(stream), a);
    else hipLaunchKernelGGL(attn_merge_kernel<float>, dim3(rows, H), dim3(64), 0, S_(stream), a);
  }
  return ok_or("mrs_hyb_paged_window_attn");
}

extern "C" int mrs_hyb_paged_window_attn(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_seq, const int *tok_pos, void *out,
                                         int rows, int H, int G, int D, int Dv, int block_size, int max_blocks, int window, int keep_first, float scale, int dtype,
                                         const int *seg_entry, const int *seg_row0, const int *seg_len, int segments, int seg_rows, void *stream) {
  return attn_launch(q, k_cache, v_cache, block_tables, tok_seq, tok_pos, out, rows, H, G, D, Dv, block_size, max_blocks, window, keep_first, scale, dtype, seg_entry, seg_row0, seg_len,
                     segments, seg_rows, 0.f, 0, nullptr, 0, nullptr, 0, 0, stream);
}
/* the same attention with its options: softcap (0: none), sink (a zero-score term in the denominator), gate (nullable f32 [rows, ldg]: output times sigmoid(gate)).
 * scratch (nullable, f32 [splits, rows, H, Dv + 2]) with splits > 1: a step of single rows deals every row's key passes to that many workgroups (steps with portions ignore it).
 * token_major: k_cache / v_cache hold rows [block, slot, kv head, dim], the row-major output of a product over the blocks' tokens */
extern "C" int mrs_hyb_paged_attn_opts(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_seq, const int *tok_pos, void *out,
                                       int rows, int H, int G, int D, int Dv, int block_size, int max_blocks, int window, int keep_first, float scale, int dtype,
                                       const int *seg_entry, const int *seg_row0, const int *seg_len, int segments, int seg_rows, float softcap, int sink, const float *gate, int ldg,
                                       float *scratch, int splits, int token_major, void *stream) {
  return attn_launch(q, k_cache, v_cache, block_tables, tok_seq, tok_pos, out, rows, H, G, D, Dv, block_size, max_blocks, window, keep_first, scale, dtype, seg_entry, seg_row0, seg_len,
                     segments, seg_rows, softcap, sink, gate, ldg, scratch, splits, token_major, stream);
}

/* the same attention inside position chunks (chunk > 0: query i reads the keys j <= i with floor(j / chunk) == floor(i / chunk)), with a learned sink (sink_logit [H], nullable:
 * the softmax's extra term of head h is e^{sink_logit[h]}) and a gate of one logit per (row, head) (gate_per_head != 0: gate[t * ldg + h]) */
extern "C" int mrs_hyb_paged_attn_chunked(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_seq, const int *tok_pos, void *out,
                                          int rows, int H, int G, int D, int Dv, int block_size, int max_blocks, int chunk, float scale, int dtype, const int *seg_entry,
                                          const int *seg_row0, const int *seg_len, int segments, int seg_rows, float softcap, int sink, const float *sink_logit, const float *gate,
                                          int ldg, int gate_per_head, float *scratch, int splits, void *stream) {
  return attn_launch(q, k_cache, v_cache, block_tables, tok_seq, tok_pos, out, rows, H, G, D, Dv, block_size, max_blocks, 0, 0, scale, dtype, seg_entry, seg_row0, seg_len,
                     segments, seg_rows, softcap, sink, gate, ldg, scratch, splits, 0, stream, chunk, sink_logit, gate_per_head);
}

/* h [rows, W] f32 (contiguous), wr [E (+ 1), W] f32 */
extern "C" int mrs_hyb_route_sigmoid_topk(const float *h, const float *wr, int rows, int W, int E, int top, int has_gate, int *ids, float *wts, float *gate, void *stream) {
  if (rows <= 0) return 0;
  if (top < 1 || top > E || E > 8192) return fail("mrs_hyb_route_sigmoid_topk: 1 <= top <= experts <= 8192");
  hipLaunchKernelGGL(route_topk_kernel<false>, dim3(rows), dim3(1024), (size_t)(E + 1) * 4, S_(stream), h, wr, W, E, top, has_gate, ids, wts, gate, 1.0f, (const float *)nullptr, 0);
  return ok_or("mrs_hyb_route_sigmoid_topk");
}

/* softmax over all experts, the `top` largest, weights = scale * score (not renormalised over the chosen) */
extern "C" int mrs_hyb_route_softmax_topk(const float *h, const float *wr, int rows, int W, int E, int top, float scale, int *ids, float *wts, void *stream) {
  if (rows <= 0) return 0;
  if (top < 1 || top > E || E > 8192) return fail("mrs_hyb_route_softmax_topk: 1 <= top <= experts <= 8192");
  hipLaunchKernelGGL(route_topk_kernel<true>, dim3(rows), dim3(1024), (size_t)(E + 1) * 4, S_(stream), h, wr, W, E, top, 0, ids, wts, (float *)nullptr, scale, (const float *)nullptr, 0);
  return ok_or("mrs_hyb_route_softmax_topk");
}

/* logits = wr h + bias (bias nullable); the `top` largest; weights = scale * softmax over the chosen logits only */
extern "C" int mrs_hyb_route_topk_softmax(const float *h, const float *wr, const float *bias, int rows, int W, int E, int top, float scale, int *ids, float *wts, void *stream) {
  if (rows <= 0) return 0;
  if (top < 1 || top > E || E > 8192) return fail("mrs_hyb_route_topk_softmax: 1 <= top <= experts <= 8192");
  hipLaunchKernelGGL(route_topk_kernel<true>, dim3(rows), dim3(1024), (size_t)(E + 1) * 4, S_(stream), h, wr, W, E, top, 0, ids, wts, (float *)nullptr, scale, bias, 1);
  return ok_or("mrs_hyb_route_topk_softmax");
}

extern "C" int mrs_hyb_moe_dispatch(const int *ids, int R, int E, int *bounds, int *sorted_route, int *route_pos, int *sorted_expert, void *stream) {
  if (E <= 0 || E > 8192) return fail("mrs_hyb_moe_dispatch: 1 .. 8192 experts");
  if (R <= 0) return 0;
  hipLaunchKernelGGL(moe_dispatch_kernel, dim3(E), dim3(256), 0, S_(stream), ids, R, E, bounds, sorted_route, route_pos, sorted_expert);
  return ok_or("mrs_hyb_moe_dispatch");
}

extern "C" int mrs_hyb_moe_gather(const float *h32, const int *sorted_route, const float *wts, int top, void *out, int R, int W, int dtype, void *stream) {
  if (R <= 0) return 0;
  if (dtype == 1) hipLaunchKernelGGL(moe_gather_kernel<mrs::bf16_t>, dim3(R), dim3(256), 0, S_(stream), h32, sorted_route, wts, top, (mrs::bf16_t *)out, W);
  else if (dtype == 2) hipLaunchKernelGGL(moe_gather_kernel<float>, dim3(R), dim3(256), 0, S_(stream), h32, sorted_route, wts, top, (float *)out, W);
  else return fail("mrs_hyb_moe_gather: dtype");
  return ok_or("mrs_hyb_moe_gather");
}

extern "C" int mrs_hyb_glu_silu(const float *gu, void *out, int rows, int ff, int dtype, void *stream) {
  if (rows <= 0) return 0;
  const unsigned blocks = (unsigned)(((size_t)rows * ff + 255) / 256);
  if (dtype == 1) hipLaunchKernelGGL(glu_silu_kernel<mrs::bf16_t>, dim3(blocks), dim3(256), 0, S_(stream), gu, (mrs::bf16_t *)out, rows, ff);
  else if (dtype == 2) hipLaunchKernelGGL(glu_silu_kernel<float>, dim3(blocks), dim3(256), 0, S_(stream), gu, (float *)out, rows, ff);
  else return fail("mrs_hyb_glu_silu: dtype");
  return ok_or("mrs_hyb_glu_silu");
}

extern "C" int mrs_hyb_moe_combine(float *x, const float *d, const int *route_pos, int top, const float *shared, const float *gate, int rows, int W, void *stream) {
  if (rows <= 0) return 0;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(rows), dim3(256), 0, S_(stream), x, d, route_pos, top, shared, gate, W, (const float *)nullptr, 1);
  return ok_or("mrs_hyb_moe_combine");
}

/* out[t] (+)= sum_k wts[t top + k] * d[route_pos[t top + k]] + shared[t] (shared nullable) */
extern "C" int mrs_hyb_moe_combine_weighted(float *out, const float *d, const int *route_pos, const float *wts, int top, const float *shared, int rows, int W, int accumulate,
                                            void *stream) {
  if (rows <= 0) return 0;
  if (!wts) return fail("mrs_hyb_moe_combine_weighted: the route weights are missing");
  hipLaunchKernelGGL(moe_combine_kernel, dim3(rows), dim3(256), 0, S_(stream), out, d, route_pos, top, shared, (const float *)nullptr, W, wts, accumulate);
  return ok_or("mrs_hyb_moe_combine_weighted");
}

extern "C" int mrs_hyb_glu_clamped(const float *gu, void *out, int rows, int ff, float limit, float alpha, int dtype, void *stream) {
  if (rows <= 0) return 0;
  const unsigned blocks = (unsigned)(((size_t)rows * ff + 255) / 256);
  if (dtype == 1) hipLaunchKernelGGL(glu_clamped_kernel<mrs::bf16_t>, dim3(blocks), dim3(256), 0, S_(stream), gu, (mrs::bf16_t *)out, rows, ff, limit, alpha);
  else if (dtype == 2) hipLaunchKernelGGL(glu_clamped_kernel<float>, dim3(blocks), dim3(256), 0, S_(stream), gu, (float *)out, rows, ff, limit, alpha);
  else return fail("mrs_hyb_glu_clamped: dtype");
  return ok_or("mrs_hyb_glu_clamped");
}

/* out (dtype) = xIELU(u + bias); ap = softplus(p), an = 1 / 2 + softplus(q) of the layer's two activation numbers */
extern "C" int mrs_hyb_bias_xielu(const float *u, int ldu, const float *bias, void *out, int rows, int ff, float ap, float an, int dtype, void *stream) {
  if (rows <= 0) return 0;
  const unsigned blocks = (unsigned)(((size_t)rows * ff + 255) / 256);
  if (dtype == 1) hipLaunchKernelGGL(bias_xielu_kernel<mrs::bf16_t>, dim3(blocks), dim3(256), 0, S_(stream), u, ldu, bias, (mrs::bf16_t *)out, rows, ff, ap, an);
  else if (dtype == 2) hipLaunchKernelGGL(bias_xielu_kernel<float>, dim3(blocks), dim3(256), 0, S_(stream), u, ldu, bias, (float *)out, rows, ff, ap, an);
  else return fail("mrs_hyb_bias_xielu: dtype");
  return ok_or("mrs_hyb_bias_xielu");
}

/* Layer norm of every row of x (+ in_bias): out (dtype, nullable), out32 (nullable), resid (nullable, f32 [rows, ldr]): resid += the normed row */
extern "C" int mrs_hyb_layernorm(const float *x, int ldx, const float *in_bias, const float *w, const float *b, void *out, float *out32, float *resid, int ldr, int rows, int width,
                                 float eps, int dtype, void *stream) {
  if (rows <= 0) return 0;
  if (width <= 0 || width > 15000) return fail("mrs_hyb_layernorm: 1 .. 15000 values per row");
  const size_t lds = (size_t)width * 4;
  if (dtype == 1) hipLaunchKernelGGL(layernorm_kernel<mrs::bf16_t>, dim3(rows), dim3(256), lds, S_(stream), x, ldx, in_bias, w, b, (mrs::bf16_t *)out, out32, resid, ldr, width, eps,
                                     (const float *)nullptr, (const float *)nullptr);
  else if (dtype == 2) hipLaunchKernelGGL(layernorm_kernel<float>, dim3(rows), dim3(256), lds, S_(stream), x, ldx, in_bias, w, b, (float *)out, out32, resid, ldr, width, eps,
                                          (const float *)nullptr, (const float *)nullptr);
  else return fail("mrs_hyb_layernorm: dtype");
  return ok_or("mrs_hyb_layernorm");
}

/* resid += norm(y + in_bias; w, b), then out (dtype) / out32 = norm(resid; w2, b2): the norm behind a sublayer and the norm in front of the next one in one pass */
extern "C" int mrs_hyb_layernorm_pair(const float *y, int ldy, const float *in_bias, const float *w, const float *b, float *resid, int ldr, const float *w2, const float *b2,
                                      void *out, float *out32, int rows, int width, float eps, int dtype, void *stream) {
  if (rows <= 0) return 0;
  if (width <= 0 || width > 15000) return fail("mrs_hyb_layernorm_pair: 1 .. 15000 values per row");
  if (!resid || !w2 || !w) return fail("mrs_hyb_layernorm_pair: the residual stream and both norms' weights are needed");
  const size_t lds = (size_t)width * 4;
  if (dtype == 1) hipLaunchKernelGGL(layernorm_kernel<mrs::bf16_t>, dim3(rows), dim3(256), lds, S_(stream), y, ldy, in_bias, w, b, (mrs::bf16_t *)out, out32, resid, ldr, width, eps, w2, b2);
  else if (dtype == 2) hipLaunchKernelGGL(layernorm_kernel<float>, dim3(rows), dim3(256), lds, S_(stream), y, ldy, in_bias, w, b, (float *)out, out32, resid, ldr, width, eps, w2, b2);
  else return fail("mrs_hyb_layernorm_pair: dtype");
  return ok_or("mrs_hyb_layernorm_pair");
}

/* temp_every <= 0: no query temperature.  k_cache null: the rows carry no key / value columns (a layer that reads another layer's pages) */
extern "C" int mrs_hyb_qkv_bias_temp_cache(const float *qkv, int ld, const float *qb, const float *kb, const float *vb, const int *tok_pos, const long long *slot_mapping, void *q_out,
                                           void *k_cache, void *v_cache, int rows, int H, int G, int D, int Dv, int block_size, float temp_coef, int temp_every, int dtype,
                                           void *stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || (k_cache && !v_cache)) return fail("mrs_hyb_qkv_bias_temp_cache: head sizes (heads % kv_heads == 0)");
  QkvBiasArgs a{qkv, qb, kb, vb, tok_pos, slot_mapping, q_out, k_cache, v_cache, ld, H, G, D, Dv, block_size, temp_every, temp_coef};
  if (dtype == 1) hipLaunchKernelGGL(qkv_bias_temp_cache_kernel<mrs::bf16_t>, dim3(rows), dim3(256), 0, S_(stream), a);
  else if (dtype == 2) hipLaunchKernelGGL(qkv_bias_temp_cache_kernel<float>, dim3(rows), dim3(256), 0, S_(stream), a);
  else return fail("mrs_hyb_qkv_bias_temp_cache: dtype");
  return ok_or("mrs_hyb_qkv_bias_temp_cache");
}

extern "C" int mrs_hyb_gather_rows(const float *x, const int *idx, float *out, int n, int W, void *stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(n), dim3(256), 0, S_(stream), x, idx, out, W);
  return ok_or("mrs_hyb_gather_rows");
}

/* In place on u [rows, ld]: heads x D values at q_col and at k_col; the first rot dimensions of every head turn in half-split pairs (i, i + rot / 2) by tok_pos * freq[i];
 * the key range is then multiplied by k_mult.  k_col < 0: queries only. */
extern "C" int mrs_hyb_rotary_half(float *u, int ld, int q_col, int k_col, int heads, int D, int rot, const float *freq, const int *tok_pos, float k_mult, int rows, void *stream) {
  if (rows <= 0) return 0;
  if (heads <= 0 || D <= 0 || rot < 0 || (rot & 1) || rot > D || (rot > 0 && !freq)) return fail("mrs_hyb_rotary_half: even rot <= dim");
  hipLaunchKernelGGL(rotary_half_kernel, dim3(rows, k_col >= 0 ? 2 : 1), dim3(256), 0, S_(stream), u, ld, q_col, k_col, heads, D, rot, freq, tok_pos, k_mult);
  return ok_or("mrs_hyb_rotary_half");
}

/* u [rows, ld] = q [nq] | c [R]: q_out [rows, nq] (dtype) = q; c_cache[slot] (dtype, rows of R) = c / rms(c) * w */
extern "C" int mrs_hyb_latent_norm_cache(const float *u, int ld, int nq, int R, const float *w, const long long *slot_mapping, void *q_out, void *c_cache, float eps, int rows, int dtype,
                                         void *stream) {
  if (rows <= 0) return 0;
  if (nq <= 0 || R <= 0 || ld < nq + R || !w) return fail("mrs_hyb_latent_norm_cache: rows shorter than q | latent, or no norm weight");
  if (dtype == 1) hipLaunchKernelGGL(latent_norm_cache_kernel<mrs::bf16_t>, dim3(rows), dim3(256), 0, S_(stream), u, ld, nq, R, w, slot_mapping, (mrs::bf16_t *)q_out, (mrs::bf16_t *)c_cache, eps);
  else if (dtype == 2) hipLaunchKernelGGL(latent_norm_cache_kernel<float>, dim3(rows), dim3(256), 0, S_(stream), u, ld, nq, R, w, slot_mapping, (float *)q_out, (float *)c_cache, eps);
  else return fail("mrs_hyb_latent_norm_cache: dtype");
  return ok_or("mrs_hyb_latent_norm_cache");
}

/* x [rows, S, W] f32 residual streams.  y (nullable, [rows, W]): x_r <- sum_s mix[s, r] x_s + outw[r] y (mix null: x_r <- outw[r] y).  inw (nullable, [S]): v = sum_s inw[s] x_s of
 * the updated streams; with norm_w the RMS-normed v goes to out (dtype, nullable) / out32 (nullable), without it v goes to out32. */
extern "C" int mrs_hyb_hyper_step(float *x, const float *y, const float *mix, const float *outw, const float *inw, const float *norm_w, void *out, float *out32, int rows, int S, int W,
                                  float eps, int one_plus, int dtype, void *stream) {
  if (rows <= 0) return 0;
  if (S < 1 || S > 8) return fail("mrs_hyb_hyper_step: 1 .. 8 streams");
  if (W <= 0 || W > 15000) return fail("mrs_hyb_hyper_step: 1 .. 15000 values per row");
  if (y && !outw) return fail("mrs_hyb_hyper_step: writing needs the streams' output weights");
  if (dtype != 1 && dtype != 2) return fail("mrs_hyb_hyper_step: dtype");
  const size_t lds = inw && norm_w ? (size_t)W * 4 : 0;
#define MRS_HC(S_N) do { if (dtype == 1) hipLaunchKernelGGL((hyper_step_kernel<mrs::bf16_t, S_N>), dim3(rows), dim3(256), lds, S_(stream), x, y, mix, outw, inw, norm_w, (mrs::bf16_t *)out, out32, W, eps, one_plus); \
                         else hipLaunchKernelGGL((hyper_step_kernel<float, S_N>), dim3(rows), dim3(256), lds, S_(stream), x, y, mix, outw, inw, norm_w, (float *)out, out32, W, eps, one_plus); } while (0)
  switch (S) {
    case 1: MRS_HC(1); break;
    case 2: MRS_HC(2); break;
    case 3: MRS_HC(3); break;
    case 4: MRS_HC(4); break;
    case 5: MRS_HC(5); break;
    case 6: MRS_HC(6); break;
    case 7: MRS_HC(7); break;
    default: MRS_HC(8); break;
  }
#undef MRS_HC
  return ok_or("mrs_hyb_hyper_step");
}

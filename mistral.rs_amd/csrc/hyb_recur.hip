// hyb_recur.hip -- kernels of the recurrent mixers that write their state with a correction (delta rule) or through exponential gates with a running stabiliser, and
// of layers whose two sublayers read two norms of the same residual row.  Same conventions as hyb_kernels.hip: a step's rows are one flat range, entry s owns rows
// [seq_start[s], seq_start[s + 1]) at positions seq_pos0[s] + i and state slot seq_slot[s]; an entry whose first position is 0 reads its slot as zero.
//
//   norm pair            one root mean square, two weights: the inputs of a layer's mixer and feed-forward in one pass over the residual row
//   delta prep           unit-length queries and keys per head, write strengths, decays per head or per (head, key channel)
//   delta step prep      the same behind the short convolution and its tap shift, for steps of single rows: one launch
//   delta scan           S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q            (f32 state [slot, head, D, Dv])
//                        every entry one chain, or the segments of long portions side by side (end states and transitions from zero | identity, a carry, the outputs)
//   exponential gates    capped log gates, the running maximum m, the step values e^{i - m'}, e^{f + m - m'} and e^{-m'} of every row
//   head norm + gate     per-head output norm (optionally behind a normaliser column), shared or full weight, sigmoid / SiLU gate, rounded once for the out-projection
//   normed average       x (+)= c (y1 / rms(y1) w1 + y2 / rms(y2) w2)
//   squared ReLU, rounded column blocks
//
// Everything here is f32 arithmetic on f32 operands; T is only the type the results are rounded to for the next product.
#include "common.cuh"
#include <float.h>

namespace mrs {
namespace hybr {

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

// Sum over groups of R consecutive lanes (R = 4 or 16, groups aligned to R) with data-parallel-primitive moves: each step is one add whose second operand comes from another
// lane of the same row of 16 (quad permutations, rotations inside the row) -- no trip through the LDS crossbar on the serial chain of a recurrence.
template <int CTRL> __device__ __forceinline__ float dpp_add(float x) {
  return x + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
template <int R> __device__ __forceinline__ float group_sum(float x) {
  static_assert(R == 4 || R == 16, "groups of 4 or 16 lanes");
  x = dpp_add<0xB1>(x);               // quad_perm [1, 0, 3, 2]
  x = dpp_add<0x4E>(x);               // quad_perm [2, 3, 0, 1]
  if (R == 16) {
    x = dpp_add<0x124>(x);            // row_ror 4
    x = dpp_add<0x128>(x);            // row_ror 8
  }
  return x;
}

// ---------------------------------------------------------------------------------- x / rms(x) times two weights
template <class T> __global__ void __launch_bounds__(256) rmsnorm_pair_kernel(const float *__restrict__ x, int ldx, const float *__restrict__ w1, const float *__restrict__ w2,
                                                                               T *__restrict__ out1, T *__restrict__ out2, float *__restrict__ out2_32, int W, float eps, int one_plus) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float *xr = x + (size_t)t * ldx;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) s = fmaf(xr[c], xr[c], s);
  const float inv = 1.0f / sqrtf(block_sum_256(s, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = xr[c] * inv, a = v * (one_plus ? 1.0f + w1[c] : w1[c]), b = v * (one_plus ? 1.0f + w2[c] : w2[c]);
    out1[(size_t)t * W + c] = from_f<T>(a);
    out2[(size_t)t * W + c] = from_f<T>(b);
    if (out2_32) out2_32[(size_t)t * W + c] = b;
  }
}

// ---------------------------------------------------------------------------------- delta rule: operands of the recurrence
// c [rows, ldc]: q [G * D] | k [G * D] | v ... after convolution + SiLU; q and k are made unit vectors per head in place (x / sqrt(sum x^2 + 1e-6)), q times D^(-1/2).
// beta [rows, H] = sigmoid(u[b_col + h]).  Decays [rows, ndec], ndec = H * per: exp(-exp(A_log[c / per]) softplus(a[c] + dt_bias[c])), the rows of `a` being a [rows, lda]
// (per = 1: one decay per head; per = D: one per head and key channel).
__device__ __forceinline__ void delta_prep_row(float *cr, const float *ur, int b_col, const float *ar, const float *__restrict__ A_log, const float *__restrict__ dt_bias,
                                               float *betar, float *decr, int H, int G, int D, int per) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float qmul = 1.0f / sqrtf((float)D);
  for (int j = wave; j < 2 * G; j += 4) {  // head j of q | k
    float *v = cr + (size_t)j * D;
    float s = 0.f;
    for (int d = lane; d < D; d += 64) s = fmaf(v[d], v[d], s);
    const float inv = (1.0f / sqrtf(wave_sum(s) + 1e-6f)) * (j < G ? qmul : 1.0f);
    for (int d = lane; d < D; d += 64) v[d] *= inv;
  }
  for (int h = threadIdx.x; h < H; h += 256) betar[h] = sigmoid_f(ur[b_col + h]);
  const int ndec = H * per;
  for (int e = threadIdx.x; e < ndec; e += 256) decr[e] = expf(-expf(A_log[e / per]) * softplus_f(ar[e] + dt_bias[e]));
}
__global__ void __launch_bounds__(256) delta_prep_kernel(float *__restrict__ c, int ldc, const float *__restrict__ u, int ldu, int b_col, const float *__restrict__ a, int lda,
                                                         const float *__restrict__ A_log, const float *__restrict__ dt_bias, float *__restrict__ beta, float *__restrict__ dec,
                                                         int H, int G, int D, int per) {
  const int t = blockIdx.x;
  delta_prep_row(c + (size_t)t * ldc, u + (size_t)t * ldu, b_col, a + (size_t)t * lda, A_log, dt_bias, beta + (size_t)t * H, dec + (size_t)t * H * per, H, G, D, per);
}
// Steps in which every entry brings one row: the short convolution (+ SiLU) over the q | k | v columns of u with its carried taps (read, then shifted: state [slots, C,
// taps - 1], oldest first; an entry at position 0 reads zeros) and the operands above, in one launch.  grid.y: one workgroup per q / k head (convolution, then the unit
// vector from the workgroup's sum of squares), one per 256 value channels, and one for write strengths and decays.
__global__ void __launch_bounds__(256) delta_step_prep_kernel(const float *__restrict__ u, int ldu, const float *__restrict__ cw, float *__restrict__ state, float *__restrict__ c,
                                                              int ldc, int C, int taps, int b_col, const float *__restrict__ a, int lda, const float *__restrict__ A_log,
                                                              const float *__restrict__ dt_bias, float *__restrict__ beta, float *__restrict__ dec, const int *__restrict__ seq_start,
                                                              const int *__restrict__ seq_pos0, const int *__restrict__ seq_slot, int H, int G, int D, int per) {
  __shared__ float red[4];
  const int s = blockIdx.x, y = blockIdx.y, t = seq_start[s], keep = taps - 1;
  if (seq_start[s + 1] - t != 1) return;
  const bool carried = seq_pos0[s] > 0;
  auto conv = [&](int ch) {
    float *st = state + ((size_t)seq_slot[s] * C + ch) * (keep > 0 ? keep : 1);
    const float cur = u[(size_t)t * ldu + ch];
    float acc = 0.f, v[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      if (k >= keep) break;
      v[k] = carried ? st[k] : 0.f;
      acc = fmaf(cw[(size_t)ch * taps + k], v[k], acc);
    }
    acc = fmaf(cw[(size_t)ch * taps + keep], cur, acc);
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      if (k >= keep) break;
      st[k] = k + 1 < keep ? v[k + 1] : cur;
    }
    return silu_f(acc);
  };
  float *cr = c + (size_t)t * ldc;
  const int nqk = 2 * G * D, nvb = (C - nqk + 255) / 256;
  if (y < 2 * G) {   // head y of q | k
    float ss = 0.f;
    for (int d = threadIdx.x; d < D; d += 256) {
      const float v = conv(y * D + d);
      cr[y * D + d] = v;   // re-read below by the thread that wrote it
      ss = fmaf(v, v, ss);
    }
    const float inv = (1.0f / sqrtf(block_sum_256(ss, red) + 1e-6f)) * (y < G ? 1.0f / sqrtf((float)D) : 1.0f);
    for (int d = threadIdx.x; d < D; d += 256) cr[y * D + d] *= inv;
  } else if (y < 2 * G + nvb) {
    const int ch = nqk + (y - 2 * G) * 256 + threadIdx.x;
    if (ch < C) cr[ch] = conv(ch);
  } else {
    for (int h = threadIdx.x; h < H; h += 256) beta[(size_t)t * H + h] = sigmoid_f(u[(size_t)t * ldu + b_col + h]);
    const int ndec = H * per;
    for (int e = threadIdx.x; e < ndec; e += 256) dec[(size_t)t * ndec + e] = expf(-expf(A_log[e / per]) * softplus_f(a[(size_t)t * lda + e] + dt_bias[e]));
  }
}

// ---------------------------------------------------------------------------------- delta rule: the recurrence
// The value columns of S are independent: lane (p, r) of a wave owns the rows n in [r K, r K + K) of column p, the two sums over n (S^T k before the write, S^T q after it)
// close with R-lane butterflies.  The waves of one (entry, head) share the rows' operands through LDS: TC rows are staged at a time with coalesced loads, the next TC rows
// are in registers while the current ones are consumed.  An entry's rows run in order (the write depends on the state), entries / heads / columns in parallel.
struct DeltaArgs {
  const float *c;      // [rows, ldc]: q [G * D] | k [G * D] | v [H * Dv]
  const float *beta;   // [rows, H]
  const float *dec;    // [rows, H * per]
  float *state;        // [slots, H, D, Dv]
  float *out;          // [rows, H * Dv]
  const int *seq_pos0, *seq_slot;
  const int *seg_entry, *seg_row0, *seg_len, *ent_seg0;  // segment table: entry, first row, rows; first segment of every entry (+ the total)
  float *carry;        // [segments, H, D, Dv]: a segment's end state from zero, then the state the next segment starts from
  float *trans;        // [segments, H, D, D]: what a segment does to a state it is handed (the product of its rows' transitions)
  int ldc, H, G, D, Dv, per;
};
// The recurrence is linear in S: a row maps S -> (I - beta k k^T) diag(g) S + beta k v^T, the matrix in front being the same for every value column.  A long portion can
// therefore run its segments side by side like the other scans of this library:
//   A  every segment but an entry's last, from the state [0 | I] with the values [v | 0]: D further columns carry the identity through the same steps, so the segment leaves its
//      end state from zero L_k and its transition P_k                                                                                      (parallel over segments; LOCAL)
//   B  init_(k+1) = P_k init_k + L_k, init_0 = the slot's state (zero for an entry that starts at position 0)                              (delta_carry_kernel)
//   C  every segment from its init state: the outputs; an entry's last segment leaves the slot's new state                                (parallel over segments)
// An entry of one segment is pass C alone; the host runs A and B only when the step's entries alone would leave most of the chip idle.
template <int R, int K, bool VEC, int MAXREG, bool LOCAL> __global__ void __launch_bounds__(512) delta_scan_kernel(DeltaArgs a, int rowpad, int TC) {
  extern __shared__ __attribute__((aligned(16))) float sm[];  // [2][TC][rowpad]: k [D] | q [D] | decay [per] (padded to 4) | v [Dv] | beta
  constexpr int PT = 64 / R;
  const int tid = threadIdx.x, nthr = blockDim.x, wave = tid >> 6, lane = tid & 63, r = lane % R, p = (blockIdx.x * (nthr >> 6) + wave) * PT + lane / R;
  const int h = blockIdx.y, z = blockIdx.z;
  const int s = a.seg_entry[z], r0 = a.seg_row0[z], len = a.seg_len[z];
  const bool first = z == a.ent_seg0[s], last = z == a.ent_seg0[s + 1] - 1;
  if (len <= 0 || (LOCAL && last)) return;
  const int D = a.D, Dv = a.Dv, per = a.per, g = h / (a.H / a.G);
  const int ncol = LOCAL ? Dv + D : Dv;
  const bool live = p < ncol;
  const int pa = live ? p : ncol - 1;
  const bool ident = LOCAL && pa >= Dv;      // a column of the identity: no value, no output
  const int pc = ident ? 0 : pa, idc = pa - Dv;
  int nk = D - r * K;
  nk = nk < 0 ? 0 : (nk > K ? K : nk);
  float *st = a.state + ((size_t)a.seq_slot[s] * a.H + h) * D * Dv;
  const float *init = LOCAL ? nullptr : (first ? (a.seq_pos0[s] > 0 ? st : nullptr) : a.carry + ((size_t)(z - 1) * a.H + h) * D * Dv);
  float S[K];
#pragma unroll
  for (int k = 0; k < K; ++k) S[k] = k < nk ? (LOCAL ? ((ident && r * K + k == idc) ? 1.0f : 0.f) : (init ? init[(size_t)(r * K + k) * Dv + pc] : 0.f)) : 0.f;
  const int perp = (per + 3) & ~3, o_q = D, o_g = 2 * D, o_v = 2 * D + perp, o_b = o_v + Dv, rowlen = o_b + 1, stage = TC * rowpad;
  const int qcol = g * D, kcol = a.G * D + g * D, vcol = 2 * a.G * D + h * Dv;
  // this lane's operands of one staged row: k, decay and q of its K state rows (zeros / ones past the key size), the column's value and the write strength
  constexpr bool PREFETCH = K <= 16;
  const int base = nk ? r * K : 0;
  auto ops = [&](const float *row, float *kv, float *gv, float *qv, float *sv) {
    sv[0] = ident ? 0.f : row[o_v + pc];
    sv[1] = row[o_b];
    const float g1 = row[o_g];
    if (VEC) {
#pragma unroll
      for (int k = 0; k < K; k += 4) {
        const int kk = base + (k < nk ? k : 0);
        const float4 k4 = *(const float4 *)(row + kk), q4 = *(const float4 *)(row + o_q + kk);
        float4 g4 = make_float4(g1, g1, g1, g1);
        if (per > 1) g4 = *(const float4 *)(row + o_g + kk);
        const bool on = k < nk;
        kv[k] = on ? k4.x : 0.f; kv[k + 1] = on ? k4.y : 0.f; kv[k + 2] = on ? k4.z : 0.f; kv[k + 3] = on ? k4.w : 0.f;
        qv[k] = on ? q4.x : 0.f; qv[k + 1] = on ? q4.y : 0.f; qv[k + 2] = on ? q4.z : 0.f; qv[k + 3] = on ? q4.w : 0.f;
        gv[k] = g4.x; gv[k + 1] = g4.y; gv[k + 2] = g4.z; gv[k + 3] = g4.w;
      }
    } else {
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const int kk = k < nk ? base + k : 0;
        kv[k] = k < nk ? row[kk] : 0.f;
        qv[k] = k < nk ? row[o_q + kk] : 0.f;
        gv[k] = per > 1 ? row[o_g + kk] : g1;
      }
    }
  };
  // a stage = TC rows of rowpad values, dealt to the threads flat: element e = tid + m nthr (m < MAXREG) is value e % rowpad of row e / rowpad.  Where an element comes from
  // (its place in the first stage and how far one row moves it) is worked out once; a stage's loads are then one compare and one address each.
  float stg[MAXREG];
  const float *src[MAXREG];
  int rstride[MAXREG], irow[MAXREG];
  const int stage_n = TC * rowpad;
#pragma unroll
  for (int m = 0; m < MAXREG; ++m) {
    const int e = tid + m * nthr;
    src[m] = nullptr;
    rstride[m] = 0;
    irow[m] = 0;
    if (e < stage_n) {
      const int i = e / rowpad, j = e - i * rowpad;
      irow[m] = i;
      const size_t row = (size_t)r0 + i;
      if (j < o_q) { src[m] = a.c + row * a.ldc + kcol + j; rstride[m] = a.ldc; }
      else if (j < o_g) { src[m] = a.c + row * a.ldc + qcol + j - o_q; rstride[m] = a.ldc; }
      else if (j < o_v) { if (j - o_g < per) { src[m] = a.dec + (row * a.H + h) * per + j - o_g; rstride[m] = a.H * per; } }
      else if (j < o_b) { src[m] = a.c + row * a.ldc + vcol + j - o_v; rstride[m] = a.ldc; }
      else if (j < rowlen) { src[m] = a.beta + row * a.H + h; rstride[m] = a.H; }
    }
  }
  auto fetch = [&](int c0) {
#pragma unroll
    for (int m = 0; m < MAXREG; ++m) stg[m] = (src[m] && c0 + irow[m] < len) ? src[m][(size_t)c0 * rstride[m]] : 0.f;
  };
  auto put = [&](float *buf) {
#pragma unroll
    for (int m = 0; m < MAXREG; ++m) {
      const int e = tid + m * nthr;
      if (e < stage_n) buf[e] = stg[m];
    }
  };
  fetch(0);
  put(sm);
  __syncthreads();
  int flip = 0;
  for (int c0 = 0; c0 < len; c0 += TC, flip ^= 1) {
    const float *cur = sm + flip * stage;
    const bool more = c0 + TC < len;
    if (more) fetch(c0 + TC);
    const int cnt = len - c0 < TC ? len - c0 : TC;
    // a row's operands leave LDS one row ahead of their use (they do not depend on the state), into one of two register sets in turn: the serial chain per row is the
    // two sums and the write between them
    float ka[K], ga[K], qa[K], kb[K], gb[K], qb[K], sa[2], sb[2];
    float *op = a.out + (size_t)(r0 + c0) * a.H * Dv + (size_t)h * Dv + pc;
    const size_t ostep = (size_t)a.H * Dv;
    auto step = [&](const float *kc, const float *gc, const float *qc, const float *sc) {
      float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
      for (int k = 0; k < K; k += 2) {
        S[k] *= gc[k];
        acc0 = fmaf(S[k], kc[k], acc0);
        if (k + 1 < K) {
          S[k + 1] *= gc[k + 1];
          acc1 = fmaf(S[k + 1], kc[k + 1], acc1);
        }
      }
      const float uw = sc[1] * (sc[0] - group_sum<R>(acc0 + acc1));
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int k = 0; k < K; k += 2) {
        S[k] = fmaf(kc[k], uw, S[k]);
        o0 = fmaf(S[k], qc[k], o0);
        if (k + 1 < K) {
          S[k + 1] = fmaf(kc[k + 1], uw, S[k + 1]);
          o1 = fmaf(S[k + 1], qc[k + 1], o1);
        }
      }
      if (!LOCAL) {
        const float o = group_sum<R>(o0 + o1);
        if (r == 0 && live) *op = o;
        op += ostep;
      }
    };
    if (PREFETCH) {
      ops(cur, ka, ga, qa, sa);
      for (int i = 0; i < cnt; i += 2) {
        if (i + 1 < cnt) ops(cur + (i + 1) * rowpad, kb, gb, qb, sb);
        step(ka, ga, qa, sa);
        if (i + 1 < cnt) {
          if (i + 2 < cnt) ops(cur + (i + 2) * rowpad, ka, ga, qa, sa);
          step(kb, gb, qb, sb);
        }
      }
    } else {
      for (int i = 0; i < cnt; ++i) {
        ops(cur + i * rowpad, ka, ga, qa, sa);
        step(ka, ga, qa, sa);
      }
    }
    if (more) put(sm + (flip ^ 1) * stage);
    __syncthreads();
  }
  if (LOCAL) {
    float *dst = ident ? a.trans + ((size_t)z * a.H + h) * D * D + idc : a.carry + ((size_t)z * a.H + h) * D * Dv + pc;
    const int ld = ident ? D : Dv;
    if (live)
#pragma unroll
      for (int k = 0; k < K; ++k)
        if (k < nk) dst[(size_t)(r * K + k) * ld] = S[k];
  } else if (live && last) {
#pragma unroll
    for (int k = 0; k < K; ++k)
      if (k < nk) st[(size_t)(r * K + k) * Dv + p] = S[k];
  }
}
// pass B: one workgroup per (4 value columns, head, entry); thread n owns state row n of the four columns.  Serial over the entry's segments:
// new[n][:] = sum_m P[n][m] cur[m][:] + L[n][:], cur in LDS; carry[z] (L on entry) leaves as the state segment z + 1 starts from.
__global__ void __launch_bounds__(256) delta_carry_kernel(DeltaArgs a) {
  __shared__ __attribute__((aligned(16))) float cur[256][4];
  const int n = threadIdx.x, p0 = blockIdx.x * 4, h = blockIdx.y, s = blockIdx.z;
  const int z0 = a.ent_seg0[s], z1 = a.ent_seg0[s + 1], D = a.D, Dv = a.Dv;
  if (z1 - z0 < 2) return;
  const float *st = a.state + ((size_t)a.seq_slot[s] * a.H + h) * D * Dv;
  const bool carried = a.seq_pos0[s] > 0;
  float v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = (carried && n < D && p0 + j < Dv) ? st[(size_t)n * Dv + p0 + j] : 0.f;
  for (int z = z0; z < z1 - 1; ++z) {
    __syncthreads();   // the previous round has read cur
    if (n < D) *(float4 *)cur[n] = make_float4(v[0], v[1], v[2], v[3]);
    __syncthreads();
    if (n < D) {
      const float *P = a.trans + (((size_t)z * a.H + h) * D + n) * D;
      float *L = a.carry + (((size_t)z * a.H + h) * D + n) * Dv + p0;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = p0 + j < Dv ? L[j] : 0.f;
      for (int m = 0; m < D; ++m) {
        const float pm = P[m];
        const float4 c4 = *(const float4 *)cur[m];
        v[0] = fmaf(pm, c4.x, v[0]); v[1] = fmaf(pm, c4.y, v[1]); v[2] = fmaf(pm, c4.z, v[2]); v[3] = fmaf(pm, c4.w, v[3]);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (p0 + j < Dv) L[j] = v[j];
    }
  }
}

// ---------------------------------------------------------------------------------- exponential gates with a running stabiliser
// u [rows, ldu]: raw input-gate logits at i_col + h, forget-gate logits at f_col + h.
//   i = cap tanh((raw_i + bi) / cap);  f = logsigmoid(cap tanh((raw_f + bf) / cap));  m' = max(f + m, i)   (m carried per slot and head, 0 for a fresh sequence)
//   steps [rows, H, 2] = (e^{i - m'}, e^{f + m - m'}): what the state takes in and what it keeps;  mexp [rows, H] = e^{-m'}
// The chain m' = max(f + m, i) composes: a run of rows acts as m -> max(m + F, I) with F = sum f and I = the chain's result from minus infinity.  An entry's rows are cut
// into 256 / H pieces; every (piece, head) thread folds its piece, one thread per head chains the pieces, then every thread replays its piece from the right start.
// mbuf [rows + entries, H]: m' of every row, then the m every entry started from.
__device__ __forceinline__ void log_gates(const float *ur, int i_col, int f_col, int h, const float *bi, const float *bf, float cap, float &ig, float &fg) {
  ig = cap * tanhf((ur[i_col + h] + bi[h]) / cap);
  fg = -softplus_f(-(cap * tanhf((ur[f_col + h] + bf[h]) / cap)));
}
__global__ void __launch_bounds__(256) exp_gates_log_kernel(const float *__restrict__ u, int ldu, int i_col, int f_col, const float *__restrict__ bi, const float *__restrict__ bf,
                                                            float cap, float *__restrict__ steps, int H, int n) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  float ig, fg;
  log_gates(u + (size_t)(e / H) * ldu, i_col, f_col, e % H, bi, bf, cap, ig, fg);
  steps[2 * (size_t)e] = ig;
  steps[2 * (size_t)e + 1] = fg;
}
// one workgroup per entry.  FUSED (steps of single rows): the log gates before and the exponentials after the chain in the same launch.
template <bool FUSED> __global__ void __launch_bounds__(256) exp_gates_chain_kernel(const float *__restrict__ u, int ldu, int i_col, int f_col, const float *__restrict__ bi,
                                                                                    const float *__restrict__ bf, float cap, float *__restrict__ m_state, float *__restrict__ steps,
                                                                                    float *__restrict__ mbuf, float *__restrict__ mexp, const int *__restrict__ seq_start,
                                                                                    const int *__restrict__ seq_pos0, const int *__restrict__ seq_slot, int H, int rows) {
  __shared__ float pF[256], pI[256], pM[256];
  const int s = blockIdx.x, r0 = seq_start[s], len = seq_start[s + 1] - r0;
  if (len <= 0) return;
  if (FUSED) {
    for (int e = threadIdx.x; e < len * H; e += 256) {
      float ig, fg;
      log_gates(u + (size_t)(r0 + e / H) * ldu, i_col, f_col, e % H, bi, bf, cap, ig, fg);
      steps[2 * ((size_t)r0 * H + e)] = ig;
      steps[2 * ((size_t)r0 * H + e) + 1] = fg;
    }
    __syncthreads();
  }
  float *ms = m_state + (size_t)seq_slot[s] * H;
  const bool carried = seq_pos0[s] > 0;
  const int pieces = 256 / H, per = (len + pieces - 1) / pieces;
  const int pc = threadIdx.x / H, ph = threadIdx.x % H;
  const int i0 = pc * per, i1 = (i0 + per < len) ? i0 + per : len;
  const bool mine = pc < pieces && i0 < len;
  if (mine) {
    float F = 0.f, I = -FLT_MAX;
    for (int i = i0; i < i1; ++i) {
      const float *g = steps + 2 * ((size_t)(r0 + i) * H + ph);
      F += g[1];
      I = fmaxf(I + g[1], g[0]);
    }
    pF[threadIdx.x] = F;
    pI[threadIdx.x] = I;
  }
  __syncthreads();
  if (threadIdx.x < H) {
    float m = carried ? ms[threadIdx.x] : 0.f;
    mbuf[((size_t)rows + s) * H + threadIdx.x] = m;
    for (int c = 0; c < pieces && c * per < len; ++c) {
      pM[c * H + threadIdx.x] = m;
      m = fmaxf(m + pF[c * H + threadIdx.x], pI[c * H + threadIdx.x]);
    }
    ms[threadIdx.x] = m;   // the entry's last m'
  }
  __syncthreads();
  if (mine) {
    float m = pM[threadIdx.x];
    for (int i = i0; i < i1; ++i) {
      const float *g = steps + 2 * ((size_t)(r0 + i) * H + ph);
      m = fmaxf(g[1] + m, g[0]);
      mbuf[(size_t)(r0 + i) * H + ph] = m;
    }
  }
  if (!FUSED) return;
  __syncthreads();
  for (int e = threadIdx.x; e < len * H; e += 256) {
    const int i = e / H, h = e % H, t = r0 + i;
    const float m_old = i ? mbuf[(size_t)(t - 1) * H + h] : mbuf[((size_t)rows + s) * H + h], m_new = mbuf[(size_t)t * H + h];
    float *g = steps + 2 * ((size_t)t * H + h);
    const float ig = g[0], fg = g[1];
    g[0] = expf(ig - m_new);
    g[1] = expf(fg + m_old - m_new);
    mexp[(size_t)t * H + h] = expf(-m_new);
  }
}
__global__ void __launch_bounds__(256) exp_gates_exp_kernel(float *__restrict__ steps, const float *__restrict__ mbuf, float *__restrict__ mexp, const int *__restrict__ tok_seq,
                                                            const int *__restrict__ seq_start, int H, int rows) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= rows * H) return;
  const int t = e / H, h = e % H, s = tok_seq[t];
  const float m_old = t > seq_start[s] ? mbuf[(size_t)(t - 1) * H + h] : mbuf[((size_t)rows + s) * H + h], m_new = mbuf[(size_t)e];
  const float ig = steps[2 * (size_t)e], fg = steps[2 * (size_t)e + 1];
  steps[2 * (size_t)e] = expf(ig - m_new);
  steps[2 * (size_t)e + 1] = expf(fg + m_old - m_new);
  mexp[e] = expf(-m_new);
}

// ---------------------------------------------------------------------------------- per-head output norm with a gate
// y [rows, H * ldp] f32 (head h's Dv values start at h * ldp).  mexp (nullable, [rows, H]): the values are first divided by max(|y[h * ldp + Dv]|, mexp) + 1e-6 (the
// normaliser column of a matrix memory).  Then o / sqrt(mean(o^2) + eps) times w (w_full: [H * Dv], else [Dv] shared by the heads) times the gate: gate_mode 1 = sigmoid,
// 2 = SiLU of gate[t * ldg + h * Dv + d]; 0 = none.  One wave per (row, head).
template <class T> __global__ void __launch_bounds__(64) head_norm_gate_kernel(const float *__restrict__ y, int ldp, const float *__restrict__ mexp, const float *__restrict__ w,
                                                                               int w_full, const float *__restrict__ gate, int ldg, int gate_mode, T *__restrict__ out, int H, int Dv,
                                                                               float eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float *yr = y + ((size_t)t * H + h) * ldp;
  float den = 1.0f;
  if (mexp) den = 1.0f / (fmaxf(fabsf(yr[Dv]), mexp[(size_t)t * H + h]) + 1e-6f);
  float s = 0.f;
  for (int d = lane; d < Dv; d += 64) {
    const float v = mexp ? yr[d] * den : yr[d];
    s = fmaf(v, v, s);
  }
  const float inv = 1.0f / sqrtf(wave_sum(s) / (float)Dv + eps);
  for (int d = lane; d < Dv; d += 64) {
    float v = (mexp ? yr[d] * den : yr[d]) * inv * w[(w_full ? h * Dv : 0) + d];
    if (gate_mode) {
      const float gv = gate[(size_t)t * ldg + (size_t)h * Dv + d];
      v *= gate_mode == 1 ? sigmoid_f(gv) : silu_f(gv);
    }
    out[((size_t)t * H + h) * Dv + d] = from_f<T>(v);
  }
}

// ---------------------------------------------------------------------------------- x (+)= c (y1 / rms(y1) w1 + y2 / rms(y2) w2)
__global__ void __launch_bounds__(256) norm_pair_add_kernel(float *__restrict__ x, int ldx, const float *__restrict__ y1, const float *__restrict__ w1, const float *__restrict__ y2,
                                                            const float *__restrict__ w2, int W, float eps, float c, int accumulate) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float *a = y1 + (size_t)t * W, *b = y2 + (size_t)t * W;
  float s1 = 0.f, s2 = 0.f;
  for (int k = threadIdx.x; k < W; k += 256) { s1 = fmaf(a[k], a[k], s1); s2 = fmaf(b[k], b[k], s2); }
  const float i1 = 1.0f / sqrtf(block_sum_256(s1, red) / (float)W + eps);
  const float i2 = 1.0f / sqrtf(block_sum_256(s2, red) / (float)W + eps);
  for (int k = threadIdx.x; k < W; k += 256) {
    const float v = c * (a[k] * i1 * w1[k] + b[k] * i2 * w2[k]);
    float *xp = x + (size_t)t * ldx + k;
    *xp = accumulate ? *xp + v : v;
  }
}

// out [rows, n] (T, contiguous) = the first n columns of u [rows, ldu], rounded once: a column block of a product's f32 result as the operand of the next product
template <class T> __global__ void __launch_bounds__(256) round_cols_kernel(const float *__restrict__ u, int ldu, T *__restrict__ out, int n, size_t total) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  out[i] = from_f<T>(u[(i / n) * ldu + i % n]);
}

template <class T> __global__ void __launch_bounds__(256) relu_sq_kernel(const float *__restrict__ u, T *__restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = fmaxf(u[i], 0.f);
  out[i] = from_f<T>(v * v);
}

}  // namespace hybr
}  // namespace mrs

using namespace mrs::hybr;
#define S_(s) ((hipStream_t)(s))

extern "C" const char *mrs_hyb_recur_last_error() { return g_err; }

/* out1 = x / rms(x) * w1, out2 = x / rms(x) * w2 (one_plus: 1 + w) in dtype; out2_32 (nullable): the second one in f32 too */
extern "C" int mrs_hyb_rmsnorm_pair(const float *x, int ldx, const float *w1, const float *w2, void *out1, void *out2, float *out2_32, int rows, int W, float eps, int one_plus,
                                    int dtype, void *stream) {
  if (rows <= 0) return 0;
  if (dtype == 1) hipLaunchKernelGGL(rmsnorm_pair_kernel<mrs::bf16_t>, dim3(rows), dim3(256), 0, S_(stream), x, ldx, w1, w2, (mrs::bf16_t *)out1, (mrs::bf16_t *)out2, out2_32, W, eps, one_plus);
  else if (dtype == 2) hipLaunchKernelGGL(rmsnorm_pair_kernel<float>, dim3(rows), dim3(256), 0, S_(stream), x, ldx, w1, w2, (float *)out1, (float *)out2, out2_32, W, eps, one_plus);
  else return fail("mrs_hyb_rmsnorm_pair: dtype");
  return ok_or("mrs_hyb_rmsnorm_pair");
}

extern "C" int mrs_hyb_delta_prep(float *c, int ldc, const float *u, int ldu, int b_col, const float *a, int lda, const float *A_log, const float *dt_bias, float *beta, float *dec,
                                  int rows, int H, int G, int D, int per, void *stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || (per != 1 && per != D)) return fail("mrs_hyb_delta_prep: head sizes (heads % kv_heads == 0; decays per head or per key channel)");
  hipLaunchKernelGGL(delta_prep_kernel, dim3(rows), dim3(256), 0, S_(stream), c, ldc, u, ldu, b_col, a, lda, A_log, dt_bias, beta, dec, H, G, D, per);
  return ok_or("mrs_hyb_delta_prep");
}

/* single-row steps: convolution + SiLU over the C = 2 G D + (value channels) columns of u with the slots' taps, then the operands of mrs_hyb_delta_prep, one launch */
extern "C" int mrs_hyb_delta_step_prep(const float *u, int ldu, const float *cw, float *state, float *c, int ldc, int C, int taps, int b_col, const float *a, int lda,
                                       const float *A_log, const float *dt_bias, float *beta, float *dec, const int *seq_start, const int *seq_pos0, const int *seq_slot,
                                       int rows, int entries, int H, int G, int D, int per, void *stream) {
  if (rows <= 0) return 0;
  if (rows != entries) return fail("mrs_hyb_delta_step_prep: one row per entry");
  if (H <= 0 || G <= 0 || H % G || D <= 0 || (per != 1 && per != D) || taps < 1 || taps > 17 || C < 2 * G * D || ldc < C) return fail("mrs_hyb_delta_step_prep: head sizes / 1 .. 17 taps");
  if (entries > 65535 || 2 * G + (C - 2 * G * D + 255) / 256 + 1 > 65535) return fail("mrs_hyb_delta_step_prep: too many entries / heads for one launch");
  hipLaunchKernelGGL(delta_step_prep_kernel, dim3(entries, 2 * G + (C - 2 * G * D + 255) / 256 + 1), dim3(256), 0, S_(stream), u, ldu, cw, state, c, ldc, C, taps, b_col, a, lda, A_log, dt_bias, beta, dec, seq_start, seq_pos0,
                     seq_slot, H, G, D, per);
  return ok_or("mrs_hyb_delta_step_prep");
}

/* c [rows, ldc] = q [G * D] | k [G * D] | v [H * Dv] (unit q / k), beta [rows, H], dec [rows, H * per] (per 1 or D), state [slots, H, D, Dv], out [rows, H * Dv].
 * Segment table as for the other scans.  carry [segments, H, D, Dv] and trans [segments, H, D, D] (nullable scratch): with them, a step whose entries alone would leave most of
 * the chip idle runs the segments of its long portions side by side (three passes); without them, or when entries x heads x columns fill the chip, every entry is one chain.
 * lanes_per_column 0: chosen from the step's parallelism (4, or 16 for shorter serial chains). */
extern "C" int mrs_hyb_delta_scan(const float *c, int ldc, const float *beta, const float *dec, float *state, float *out, const int *seq_pos0, const int *seq_slot,
                                  const int *seg_entry, const int *seg_row0, const int *seg_len, const int *ent_seg0, float *carry, float *trans, int rows, int entries,
                                  int segments, int H, int G, int D, int Dv, int per, int lanes_per_column, void *stream) {
  if (rows <= 0 || entries <= 0 || segments <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || (per != 1 && per != D)) return fail("mrs_hyb_delta_scan: head sizes (heads % kv_heads == 0; decays per head or per key channel)");
  if (D > 256) return fail("mrs_hyb_delta_scan: key size above 256");
  if (entries > 65535 || segments > 65535 || H > 65535) return fail("mrs_hyb_delta_scan: more than 65535 entries, segments or heads");
  if (ldc < 2 * G * D + H * Dv) return fail("mrs_hyb_delta_scan: rows shorter than q | k | v");
  if (segments > entries && (!carry || !trans)) return fail("mrs_hyb_delta_scan: segmented entries need the carry scratch");
  DeltaArgs a{c, beta, dec, state, out, seq_pos0, seq_slot, seg_entry, seg_row0, seg_len, ent_seg0, carry, trans, ldc, H, G, D, Dv, per};
  const bool split = segments > entries;
  const long long par = (long long)segments * H * ((Dv + 15) / 16);   // waves at four lanes per column
  int R = lanes_per_column;
  if (R != 4 && R != 16) R = (par >= 2048 || D < 64) ? 4 : 16;
  const int PT = 64 / R;
  const int perp = (per + 3) & ~3, rowlen = 2 * D + perp + Dv + 1, rowpad = (rowlen + 3) & ~3;
  constexpr int MAXREG = 12, TC_MAX = 16;
  const bool vec = D % 4 == 0;
  auto launch = [&](bool local) {
    const int ncol = local ? Dv + D : Dv;
    // waves for the columns; waves whose registers can stage eight rows of operands at a time (a stage must outlast the latency of the loads for the next one)
    const int nw_all = (ncol + PT - 1) / PT, nw_stage = (8 * rowpad + MAXREG * 64 - 1) / (MAXREG * 64);
    int nw = nw_all > 8 ? 8 : nw_all;   // (four-wave workgroups, one chain per SIMD, measured no faster: the chain is bound by its own instruction count)
    const int nblk = (nw_all + nw - 1) / nw;
    if (nw < nw_stage) nw = nw_stage > 8 ? 8 : nw_stage;  // few value columns next to long keys: further waves only help to stage (their columns lie past the last one and are never written)
    int TC = (MAXREG * 64 * nw) / rowpad;
    TC = TC > TC_MAX ? TC_MAX : TC;
    if (TC > 65536 / (8 * rowpad)) TC = 65536 / (8 * rowpad);
    if (TC < 1) return fail("mrs_hyb_delta_scan: a row of operands does not fit the staging registers / 64 KB of LDS");
    const size_t lds = (size_t)2 * TC * rowpad * 4;
    dim3 grid(nblk, H, segments), block(64 * nw);
#define MRS_DELTA__(R_, K_, V_, L_) hipLaunchKernelGGL((delta_scan_kernel<R_, K_, V_, MAXREG, L_>), grid, block, lds, S_(stream), a, rowpad, TC)
#define MRS_DELTA_(R_, K_, V_) do { if (local) MRS_DELTA__(R_, K_, V_, true); else MRS_DELTA__(R_, K_, V_, false); } while (0)
#define MRS_DELTA(R_, K_) do { if (vec) MRS_DELTA_(R_, K_, true); else MRS_DELTA_(R_, K_, false); } while (0)
    if (R == 4) {
      if (D <= 32) MRS_DELTA(4, 8); else if (D <= 64) MRS_DELTA(4, 16); else if (D <= 128) MRS_DELTA(4, 32); else MRS_DELTA(4, 64);
    } else {
      if (D <= 64) MRS_DELTA(16, 4); else if (D <= 128) MRS_DELTA(16, 8); else MRS_DELTA(16, 16);
    }
#undef MRS_DELTA
#undef MRS_DELTA_
#undef MRS_DELTA__
    return 0;
  };
  if (split) {
    if (launch(true)) return 1;
    hipLaunchKernelGGL(delta_carry_kernel, dim3((Dv + 3) / 4, H, entries), dim3(256), 0, S_(stream), a);
  }
  if (launch(false)) return 1;
  return ok_or("mrs_hyb_delta_scan");
}

/* steps [rows, H, 2], mbuf [rows + entries, H] (scratch), mexp [rows, H]; m_state [slots, H].  Steps of single rows run one launch, steps with portions three (the log
 * gates and the exponentials of all rows in parallel around the per-entry chain). */
extern "C" int mrs_hyb_exp_gates(const float *u, int ldu, int i_col, int f_col, const float *bi, const float *bf, float cap, float *m_state, float *steps, float *mbuf,
                                 float *mexp, const int *tok_seq, const int *seq_start, const int *seq_pos0, const int *seq_slot, int rows, int entries, int H, void *stream) {
  if (rows <= 0 || entries <= 0) return 0;
  if (H <= 0 || H > 256 || !(cap > 0.f)) return fail("mrs_hyb_exp_gates: 1 .. 256 heads, a positive gate cap");
  if (rows == entries) {
    hipLaunchKernelGGL(exp_gates_chain_kernel<true>, dim3(entries), dim3(256), 0, S_(stream), u, ldu, i_col, f_col, bi, bf, cap, m_state, steps, mbuf, mexp, seq_start, seq_pos0,
                       seq_slot, H, rows);
    return ok_or("mrs_hyb_exp_gates");
  }
  const int n = rows * H;
  hipLaunchKernelGGL(exp_gates_log_kernel, dim3((n + 255) / 256), dim3(256), 0, S_(stream), u, ldu, i_col, f_col, bi, bf, cap, steps, H, n);
  hipLaunchKernelGGL(exp_gates_chain_kernel<false>, dim3(entries), dim3(256), 0, S_(stream), u, ldu, i_col, f_col, bi, bf, cap, m_state, steps, mbuf, mexp, seq_start, seq_pos0,
                     seq_slot, H, rows);
  hipLaunchKernelGGL(exp_gates_exp_kernel, dim3((n + 255) / 256), dim3(256), 0, S_(stream), steps, mbuf, mexp, tok_seq, seq_start, H, rows);
  return ok_or("mrs_hyb_exp_gates");
}

extern "C" int mrs_hyb_head_norm_gate(const float *y, int ldp, const float *mexp, const float *w, int w_full, const float *gate, int ldg, int gate_mode, void *out, int rows,
                                      int H, int Dv, float eps, int dtype, void *stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || H > 65535 || Dv <= 0 || ldp < Dv + (mexp ? 1 : 0) || gate_mode < 0 || gate_mode > 2 || (gate_mode && !gate)) return fail("mrs_hyb_head_norm_gate: head sizes / gate mode");
  if (dtype == 1) hipLaunchKernelGGL(head_norm_gate_kernel<mrs::bf16_t>, dim3(rows, H), dim3(64), 0, S_(stream), y, ldp, mexp, w, w_full, gate, ldg, gate_mode, (mrs::bf16_t *)out, H, Dv, eps);
  else if (dtype == 2) hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3(rows, H), dim3(64), 0, S_(stream), y, ldp, mexp, w, w_full, gate, ldg, gate_mode, (float *)out, H, Dv, eps);
  else return fail("mrs_hyb_head_norm_gate: dtype");
  return ok_or("mrs_hyb_head_norm_gate");
}

extern "C" int mrs_hyb_norm_pair_add(float *x, int ldx, const float *y1, const float *w1, const float *y2, const float *w2, int rows, int W, float eps, float c, int accumulate,
                                     void *stream) {
  if (rows <= 0) return 0;
  hipLaunchKernelGGL(norm_pair_add_kernel, dim3(rows), dim3(256), 0, S_(stream), x, ldx, y1, w1, y2, w2, W, eps, c, accumulate);
  return ok_or("mrs_hyb_norm_pair_add");
}

extern "C" int mrs_hyb_round_cols(const float *u, int ldu, void *out, int rows, int n, int dtype, void *stream) {
  const size_t total = (size_t)rows * n;
  if (total == 0) return 0;
  dim3 grid((unsigned)((total + 255) / 256));
  if (dtype == 1) hipLaunchKernelGGL(round_cols_kernel<mrs::bf16_t>, grid, dim3(256), 0, S_(stream), u, ldu, (mrs::bf16_t *)out, n, total);
  else if (dtype == 2) hipLaunchKernelGGL(round_cols_kernel<float>, grid, dim3(256), 0, S_(stream), u, ldu, (float *)out, n, total);
  else return fail("mrs_hyb_round_cols: dtype");
  return ok_or("mrs_hyb_round_cols");
}

extern "C" int mrs_hyb_relu_sq(const float *u, void *out, int rows, int ff, int dtype, void *stream) {
  const size_t n = (size_t)rows * ff;
  if (n == 0) return 0;
  dim3 grid((unsigned)((n + 255) / 256));
  if (dtype == 1) hipLaunchKernelGGL(relu_sq_kernel<mrs::bf16_t>, grid, dim3(256), 0, S_(stream), u, (mrs::bf16_t *)out, n);
  else if (dtype == 2) hipLaunchKernelGGL(relu_sq_kernel<float>, grid, dim3(256), 0, S_(stream), u, (float *)out, n);
  else return fail("mrs_hyb_relu_sq: dtype");
  return ok_or("mrs_hyb_relu_sq");
}

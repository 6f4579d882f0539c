// hyb_gemm.hip -- plain dense products for models whose weights stay in their checkpoint dtype (bf16, or f32 for the all-f32 serving mode):
//   C[M, N] (f32)  (+)=  A[M, K] . W[N, K]^T          A, W in T = bf16 | f32, both K-contiguous ("x W^T": weights stored [out, in])
// Two kernels per dtype:
//   * gemm_tile_kernel: 64 x 64 output tile per workgroup of four waves, K in steps of 32 through LDS; bf16 operands go to v_mfma_f32_32x32x16_bf16 (one 32 x 32
//     quadrant per wave), f32 operands to a 4 x 4 register block per thread on the vector ALU (true f32: products and sums in f32, k ascending).  Grouped form: the rows
//     are sorted by group, group g owns rows [bounds[g], bounds[g + 1]) and the weight slab W + g * wstride (mixture-of-experts layers: one launch for all experts,
//     the bounds are read on the device, tiles past a group's rows leave).
//   * gemv_rows_kernel: M <= 8 rows (decode steps): one wave per output column streams the weight row with 16-byte loads, f32 accumulation per activation row,
//     butterfly sum.  Grouped form: every activation row has its own weight slab (row_group[m]).
// f32 results only: the consumers (residual sum, norms, recurrences, routers) are f32 anyway; what a consumer feeds into the next product it rounds itself, once.
#include "common.cuh"

namespace mrs {
namespace hyb {

typedef short bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct GemmArgs {
  const void *A;
  const void *W;
  float *C;
  int M, N, K, lda, ldw, ldc;
  int accumulate;            // C += instead of C =
  const int *bounds;         // grouped: [groups + 1] row bounds (device), else null
  long long wstride;         // elements between the groups' weight slabs
  int vec_ok;                // K, lda, ldw multiples of 8 (bf16) / 4 (f32) and 16-byte aligned bases: vector loads
  // batched form (bounds null, batch > 0): blockIdx.z = b multiplies A + b * a_bstride with the slab W + b * wstride into C + b * c_bstride (per-head products: the
  // heads' operands are column blocks of one row-major buffer)
  int batch;
  long long a_bstride, c_bstride;
  int c_is_T;                // C holds T (bf16 | f32 as the operands), rounded once in the epilogue, instead of f32 (no accumulate then): the consumer is another product
};
template <class T> __device__ __forceinline__ void store_c(const GemmArgs &a, size_t idx, float v) {
  if (a.c_is_T) ((T *)a.C)[idx] = from_f<T>(v);
  else a.C[idx] = a.accumulate ? a.C[idx] + v : v;
}

constexpr int BM = 64, BN = 64, BK = 32;

template <class T> struct TileLoad;
template <> struct TileLoad<bf16_t> {
  // 64 rows x 32 k of bf16 = 256 threads x 8 values
  static __device__ __forceinline__ void load(const bf16_t *base, int ld, int row0, int rows_end, int k0, int K, int vec_ok, int tid, uint16_t (*dst)[BK + 8]) {
    const int r = tid >> 2, kc = (tid & 3) * 8;
    const int row = row0 + r;
    int4 v = make_int4(0, 0, 0, 0);
    if (row < rows_end) {
      const bf16_t *p = base + (size_t)row * ld + k0 + kc;
      if (vec_ok && k0 + kc + 8 <= K) v = *(const int4 *)p;
      else {
        uint16_t t[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) t[j] = (k0 + kc + j < K) ? p[j].v : (uint16_t)0;
        v = make_int4((int)(t[0] | ((unsigned)t[1] << 16)), (int)(t[2] | ((unsigned)t[3] << 16)), (int)(t[4] | ((unsigned)t[5] << 16)), (int)(t[6] | ((unsigned)t[7] << 16)));
      }
    }
    *(int4 *)&dst[r][kc] = v;
  }
};
template <> struct TileLoad<float> {
  // 64 rows x 32 k of f32 = 256 threads x 8 values (two float4)
  static __device__ __forceinline__ void load(const float *base, int ld, int row0, int rows_end, int k0, int K, int vec_ok, int tid, float (*dst)[BK + 4]) {
    const int r = tid >> 2, kc = (tid & 3) * 8;
    const int row = row0 + r;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
    if (row < rows_end) {
      const float *p = base + (size_t)row * ld + k0 + kc;
      if (vec_ok && k0 + kc + 8 <= K) { a = *(const float4 *)p; b = *(const float4 *)(p + 4); }
      else {
        float t[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) t[j] = (k0 + kc + j < K) ? p[j] : 0.f;
        a = make_float4(t[0], t[1], t[2], t[3]); b = make_float4(t[4], t[5], t[6], t[7]);
      }
    }
    *(float4 *)&dst[r][kc] = a;
    *(float4 *)&dst[r][kc + 4] = b;
  }
};

__global__ void __launch_bounds__(256) gemm_tile_bf16_kernel(GemmArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t As[BM][BK + 8];
  __shared__ __attribute__((aligned(16))) uint16_t Ws[BN][BK + 8];
  int row_lo = 0, row_hi = a.M;
  const bf16_t *W = (const bf16_t *)a.W;
  if (a.bounds) {
    row_lo = a.bounds[blockIdx.z];
    row_hi = a.bounds[blockIdx.z + 1];
    W += (size_t)blockIdx.z * a.wstride;
  }
  const bf16_t *A = (const bf16_t *)a.A;
  size_t c_off = 0;
  if (a.batch > 0) { A += (size_t)blockIdx.z * a.a_bstride; W += (size_t)blockIdx.z * a.wstride; c_off = (size_t)blockIdx.z * a.c_bstride; }
  const int m0 = row_lo + blockIdx.y * BM, n0 = blockIdx.x * BN;
  if (m0 >= row_hi) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ql = lane & 31, kh = lane >> 5;
  const int wm = (wave & 1) * 32, wn = (wave >> 1) * 32;
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  for (int k0 = 0; k0 < a.K; k0 += BK) {
    TileLoad<bf16_t>::load(A, a.lda, m0, row_hi, k0, a.K, a.vec_ok, tid, As);
    TileLoad<bf16_t>::load(W, a.ldw, n0, a.N, k0, a.K, a.vec_ok, tid, Ws);
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      const bf16x8 af = __builtin_bit_cast(bf16x8, *(const int4 *)&As[wm + ql][ks + 8 * kh]);
      const bf16x8 wf = __builtin_bit_cast(bf16x8, *(const int4 *)&Ws[wn + ql][ks + 8 * kh]);
      // D[i][j] = sum_k X[i][k] Y[k][j] with X = activations (i = row m) and Y = weights (j = column n): lane (ql, kh) ends up with column n = ql and the rows
      // (r & 3) + 8 (r >> 2) + 4 kh, so the stores of a register are 32 consecutive floats of one output row
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, wf, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  const int n = n0 + wn + ql;
  if (n < a.N) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + wm + (r & 3) + 8 * (r >> 2) + 4 * kh;
      if (m < row_hi) store_c<bf16_t>(a, c_off + (size_t)m * a.ldc + n, acc[r]);
    }
  }
}

// 128 x 128 tile for prompt-sized products: every wave owns a 64 x 64 quadrant (2 x 2 MFMA tiles: each operand fragment read from LDS feeds two MFMAs), and the next
// K-step's global loads are in registers while the current one multiplies (one LDS buffer, two barriers per step).
__global__ void __launch_bounds__(256) gemm_tile128_bf16_kernel(GemmArgs a) {
  constexpr int TM = 128, TN = 128;
  __shared__ __attribute__((aligned(16))) uint16_t As[TM][BK + 8];
  __shared__ __attribute__((aligned(16))) uint16_t Ws[TN][BK + 8];
  int row_lo = 0, row_hi = a.M;
  const bf16_t *W = (const bf16_t *)a.W;
  if (a.bounds) {
    row_lo = a.bounds[blockIdx.z];
    row_hi = a.bounds[blockIdx.z + 1];
    W += (size_t)blockIdx.z * a.wstride;
  }
  const int m0 = row_lo + blockIdx.y * TM, n0 = blockIdx.x * TN;
  if (m0 >= row_hi) return;
  const bf16_t *A = (const bf16_t *)a.A;
  size_t c_off = 0;
  if (a.batch > 0) { A += (size_t)blockIdx.z * a.a_bstride; W += (size_t)blockIdx.z * a.wstride; c_off = (size_t)blockIdx.z * a.c_bstride; }
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ql = lane & 31, kh = lane >> 5;
  const int wm = (wave & 1) * 64, wn = (wave >> 1) * 64;
  const int lr = tid >> 2, kc = (tid & 3) * 8;  // this thread stages rows lr and lr + 64 of both operands, 8 values at kc
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  auto fetch = [&](const bf16_t *base, int ld, int row, int rows_end, int k0) -> int4 {
    int4 v = make_int4(0, 0, 0, 0);
    if (row < rows_end) {
      const bf16_t *p = base + (size_t)row * ld + k0 + kc;
      if (a.vec_ok && k0 + kc + 8 <= a.K) v = *(const int4 *)p;
      else {
        uint16_t t[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) t[j] = (k0 + kc + j < a.K) ? p[j].v : (uint16_t)0;
        v = make_int4((int)(t[0] | ((unsigned)t[1] << 16)), (int)(t[2] | ((unsigned)t[3] << 16)), (int)(t[4] | ((unsigned)t[5] << 16)), (int)(t[6] | ((unsigned)t[7] << 16)));
      }
    }
    return v;
  };
  int4 ra[2], rw[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) { ra[i] = fetch(A, a.lda, m0 + lr + 64 * i, row_hi, 0); rw[i] = fetch(W, a.ldw, n0 + lr + 64 * i, a.N, 0); }
  for (int k0 = 0; k0 < a.K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 2; ++i) { *(int4 *)&As[lr + 64 * i][kc] = ra[i]; *(int4 *)&Ws[lr + 64 * i][kc] = rw[i]; }
    __syncthreads();
    if (k0 + BK < a.K) {
#pragma unroll
      for (int i = 0; i < 2; ++i) { ra[i] = fetch(A, a.lda, m0 + lr + 64 * i, row_hi, k0 + BK); rw[i] = fetch(W, a.ldw, n0 + lr + 64 * i, a.N, k0 + BK); }
    }
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      bf16x8 af[2], wf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = __builtin_bit_cast(bf16x8, *(const int4 *)&As[wm + 32 * i + ql][ks + 8 * kh]);
        wf[i] = __builtin_bit_cast(bf16x8, *(const int4 *)&Ws[wn + 32 * i + ql][ks + 8 * kh]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn + 32 * j + ql;
    if (n >= a.N) continue;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + 32 * i + (r & 3) + 8 * (r >> 2) + 4 * kh;
        if (m < row_hi) store_c<bf16_t>(a, c_off + (size_t)m * a.ldc + n, acc[i][j][r]);
      }
  }
}

__global__ void __launch_bounds__(256) gemm_tile_f32_kernel(GemmArgs a) {
  __shared__ __attribute__((aligned(16))) float As[BM][BK + 4];
  __shared__ __attribute__((aligned(16))) float Ws[BN][BK + 4];
  int row_lo = 0, row_hi = a.M;
  const float *W = (const float *)a.W;
  if (a.bounds) {
    row_lo = a.bounds[blockIdx.z];
    row_hi = a.bounds[blockIdx.z + 1];
    W += (size_t)blockIdx.z * a.wstride;
  }
  const float *A = (const float *)a.A;
  size_t c_off = 0;
  if (a.batch > 0) { A += (size_t)blockIdx.z * a.a_bstride; W += (size_t)blockIdx.z * a.wstride; c_off = (size_t)blockIdx.z * a.c_bstride; }
  const int m0 = row_lo + blockIdx.y * BM, n0 = blockIdx.x * BN;
  if (m0 >= row_hi) return;
  const int tid = threadIdx.x, tn = tid & 15, tm = tid >> 4;  // thread: rows tm + 16 i, columns tn + 16 j
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < a.K; k0 += BK) {
    TileLoad<float>::load(A, a.lda, m0, row_hi, k0, a.K, a.vec_ok, tid, As);
    TileLoad<float>::load(W, a.ldw, n0, a.N, k0, a.K, a.vec_ok, tid, Ws);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; k += 4) {
      float4 x[4], y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = *(const float4 *)&As[tm + 16 * i][k];
#pragma unroll
      for (int j = 0; j < 4; ++j) y[j] = *(const float4 *)&Ws[tn + 16 * j][k];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(x[i].x, y[j].x, acc[i][j]);
          acc[i][j] = fmaf(x[i].y, y[j].y, acc[i][j]);
          acc[i][j] = fmaf(x[i].z, y[j].z, acc[i][j]);
          acc[i][j] = fmaf(x[i].w, y[j].w, acc[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + tm + 16 * i;
    if (m >= row_hi) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tn + 16 * j;
      if (n < a.N) store_c<float>(a, c_off + (size_t)m * a.ldc + n, acc[i][j]);
    }
  }
}

// ---------------------------------------------------------------------------------- M <= 8 rows
// The activation operand of a row kernel can be produced on the fly (decode steps: one launch less per use):
//   IN_PLAIN   A [M, K] in T
//   IN_GLU     A = f32 [M, 2 K] = gate | up of the previous product: x_k = round_T(silu(gate_k) * up_k)
//   IN_SCALED  A = f32 [rows, K] normed rows: row m reads source row src_row[m] / src_div times src_scale[src_row[m]] (1 without scales), rounded to T (expert-sorted
//              routed inputs)
//   IN_GLU_CLAMP  A = f32 [M, 2 K] = gate | up: g = min(gate, p0), u = clamp(up, -p0, p0): x_k = round_T(g sigmoid(p1 g) (u + 1))
//   IN_BIAS_XIELU A = f32 [M, K]: z = A + in_bias: x_k = round_T(z > 0 ? p0 z^2 + z / 2 : p1 (e^z - 1 - z) + z / 2)
//   IN_RELU_SQ A = f32 [M, K]: x_k = round_T(max(A, 0)^2)
// The batched form offsets A by columns: only IN_PLAIN reads it there.
enum { IN_PLAIN = 0, IN_GLU = 1, IN_SCALED = 2, IN_GLU_CLAMP = 3, IN_BIAS_XIELU = 4, IN_RELU_SQ = 5 };
struct GemvArgs {
  const void *A;
  const void *W;
  float *C;
  int M, N, K, lda, ldw, ldc;
  int accumulate;
  const int *row_group;      // grouped: row m multiplies W + row_group[m] * wstride (grid.y = M, one row per workgroup row), else null
  long long wstride;
  int vec_ok;
  const int *src_row;        // IN_SCALED
  const float *src_scale;
  int src_div;
  const float *in_bias;      // IN_BIAS_XIELU
  float p0, p1;              // IN_GLU_CLAMP: limit, sigmoid factor; IN_BIAS_XIELU: the two coefficients
  int batch;                 // batched form (row_group null): blockIdx.z = b reads A at column offset b * a_bstride, the slab W + b * wstride, writes C at column offset b * c_bstride
  long long a_bstride, c_bstride;
  int c_is_T;                // C holds T instead of f32 (no accumulate)
};

template <class T> struct Vec8;
template <> struct Vec8<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t *p, float *o) {
    const int4 v = *(const int4 *)p;
    const unsigned u[4] = {(unsigned)v.x, (unsigned)v.y, (unsigned)v.z, (unsigned)v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) { o[2 * j] = __uint_as_float(u[j] << 16); o[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u); }
  }
  static __device__ __forceinline__ void load_nt(const bf16_t *p, float *o) {
    const int4 v = ld16nt_a4(p);
    const unsigned u[4] = {(unsigned)v.x, (unsigned)v.y, (unsigned)v.z, (unsigned)v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) { o[2 * j] = __uint_as_float(u[j] << 16); o[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u); }
  }
};
template <> struct Vec8<float> {
  static __device__ __forceinline__ void load(const float *p, float *o) {
    const float4 a = *(const float4 *)p, b = *(const float4 *)(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
  static __device__ __forceinline__ void load_nt(const float *p, float *o) { load(p, o); }
};
__device__ __forceinline__ float silu_in(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float glu_clamp_in(float gv, float uv, float limit, float alpha) {
  const float g = fminf(gv, limit), u = fminf(fmaxf(uv, -limit), limit);
  return g * (1.0f / (1.0f + expf(-(alpha * g)))) * (u + 1.0f);
}
__device__ __forceinline__ float xielu_in(float z, float ap, float an) { return z > 0.f ? fmaf(ap * z, z, 0.5f * z) : fmaf(an, expm1f(z) - z, 0.5f * z); }

// one activation value (element path) / eight (vector path) of row m at column k, as the product sees it
template <class T, int IN> __device__ __forceinline__ float act1(const GemvArgs &a, int m, int k) {
  if (IN == IN_PLAIN) return to_f<T>(((const T *)a.A)[(size_t)blockIdx.z * a.a_bstride + (size_t)m * a.lda + k]);
  const float *A = (const float *)a.A;
  if (IN == IN_GLU) return round_to<T>(silu_in(A[(size_t)m * a.lda + k]) * A[(size_t)m * a.lda + a.K + k]);
  if (IN == IN_GLU_CLAMP) return round_to<T>(glu_clamp_in(A[(size_t)m * a.lda + k], A[(size_t)m * a.lda + a.K + k], a.p0, a.p1));
  if (IN == IN_BIAS_XIELU) return round_to<T>(xielu_in(A[(size_t)m * a.lda + k] + (a.in_bias ? a.in_bias[k] : 0.f), a.p0, a.p1));
  if (IN == IN_RELU_SQ) { const float v = fmaxf(A[(size_t)m * a.lda + k], 0.f); return round_to<T>(v * v); }
  const int r = a.src_row[m];
  return round_to<T>((a.src_scale ? a.src_scale[r] : 1.0f) * A[(size_t)(r / a.src_div) * a.lda + k]);
}
template <class T, int IN> __device__ __forceinline__ void act8(const GemvArgs &a, int m, int k, float *x) {
  if (IN == IN_PLAIN) { Vec8<T>::load((const T *)a.A + (size_t)blockIdx.z * a.a_bstride + (size_t)m * a.lda + k, x); return; }
  const float *A = (const float *)a.A;
  if (IN == IN_GLU) {
    float g[8], u[8];
    Vec8<float>::load(A + (size_t)m * a.lda + k, g);
    Vec8<float>::load(A + (size_t)m * a.lda + a.K + k, u);
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = round_to<T>(silu_in(g[j]) * u[j]);
    return;
  }
  if (IN == IN_GLU_CLAMP) {
    float g[8], u[8];
    Vec8<float>::load(A + (size_t)m * a.lda + k, g);
    Vec8<float>::load(A + (size_t)m * a.lda + a.K + k, u);
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = round_to<T>(glu_clamp_in(g[j], u[j], a.p0, a.p1));
    return;
  }
  if (IN == IN_BIAS_XIELU) {
    float bv[8];
    Vec8<float>::load(A + (size_t)m * a.lda + k, x);
    if (a.in_bias) Vec8<float>::load(a.in_bias + k, bv);
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = round_to<T>(xielu_in(x[j] + (a.in_bias ? bv[j] : 0.f), a.p0, a.p1));
    return;
  }
  if (IN == IN_RELU_SQ) {
    Vec8<float>::load(A + (size_t)m * a.lda + k, x);
#pragma unroll
    for (int j = 0; j < 8; ++j) { const float v = fmaxf(x[j], 0.f); x[j] = round_to<T>(v * v); }
    return;
  }
  const int r = a.src_row[m];
  const float w = a.src_scale ? a.src_scale[r] : 1.0f;
  Vec8<float>::load(A + (size_t)(r / a.src_div) * a.lda + k, x);
#pragma unroll
  for (int j = 0; j < 8; ++j) x[j] = round_to<T>(w * x[j]);
}

template <class T, int MR, int IN> __global__ void __launch_bounds__(256) gemv_rows_kernel(GemvArgs a) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + wave;
  if (n >= a.N) return;
  const T *W = (const T *)a.W;
  int m_lo = 0, m_cnt = a.M;
  if (a.row_group) {
    m_lo = blockIdx.y;
    m_cnt = 1;
    W += (size_t)a.row_group[m_lo] * a.wstride;
  } else if (a.batch > 0) {
    W += (size_t)blockIdx.z * a.wstride;
  }
  const T *wr = W + (size_t)n * a.ldw;
  float acc[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) acc[m] = 0.f;
  if (a.vec_ok) {
    for (int k = lane * 8; k < a.K; k += 512) {
      float w[8], x[8];
      Vec8<T>::load_nt(wr + k, w);
#pragma unroll
      for (int m = 0; m < MR; ++m)
        if (m < m_cnt) {
          act8<T, IN>(a, m_lo + m, k, x);
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[m] = fmaf(w[j], x[j], acc[m]);
        }
    }
  } else {
    for (int k = lane; k < a.K; k += 64) {
      const float w = to_f<T>(wr[k]);
#pragma unroll
      for (int m = 0; m < MR; ++m)
        if (m < m_cnt) acc[m] = fmaf(w, act1<T, IN>(a, m_lo + m, k), acc[m]);
    }
  }
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    if (m >= m_cnt) break;
    const float s = wave_sum(acc[m]);
    if (lane == 0) {
      const size_t idx = (size_t)blockIdx.z * a.c_bstride + (size_t)(m_lo + m) * a.ldc + n;
      if (a.c_is_T) ((T *)a.C)[idx] = from_f<T>(s);
      else a.C[idx] = a.accumulate ? a.C[idx] + s : s;
    }
  }
}

static thread_local char g_err[256];
static int fail(const char *m) { snprintf(g_err, sizeof g_err, "%s", m); return 1; }

}  // namespace hyb
}  // namespace mrs

using namespace mrs::hyb;

extern "C" const char *mrs_hyb_gemm_last_error() { return g_err; }

// dtype: 1 bf16, 2 f32.  groups > 0: grouped form (bounds [groups + 1] on the device, max_rows = the largest number of rows a group can have).
static int gemm_launch(const void *A, const void *W, void *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int accumulate,
                       const int *bounds, int groups, long long wstride, int max_rows, int batch, long long a_bstride, long long c_bstride, int c_is_T, void *stream) {
  if (M <= 0 || N <= 0) return 0;
  if (batch > 0 && groups > 0) return fail("mrs_hyb_gemm: grouped and batched at once");
  if (c_is_T && accumulate) return fail("mrs_hyb_gemm: a product that writes operands does not accumulate");
  if (batch > 65535) return fail("mrs_hyb_gemm: more than 65535 products in one batch");
  if (K <= 0 || lda < K || ldw < K || ldc < N || (dtype != 1 && dtype != 2)) return fail("mrs_hyb_gemm: bad shape / dtype");
  const int esz = dtype == 1 ? 2 : 4, vq = 8;
  GemmArgs a{A, W, (float *)C, M, N, K, lda, ldw, ldc, accumulate, groups > 0 ? bounds : nullptr, wstride,
             (K % vq == 0 && lda % vq == 0 && ldw % vq == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && (wstride * esz) % 16 == 0 &&
              (batch <= 0 || (a_bstride * esz) % 16 == 0)) ? 1 : 0, batch > 0 ? batch : 0, a_bstride, c_bstride, c_is_T};
  const int gz = groups > 0 ? groups : (batch > 0 ? batch : 1);
  const int rows = groups > 0 ? max_rows : M;
  if (rows <= 0) return 0;
  // prompt-sized bf16 products take the 128 x 128 tile: dense from 256 rows, grouped when a group averages a full tile of rows
  if (dtype == 1 && N >= 128 && (groups > 0 ? M / groups >= 128 : M >= 256)) {
    dim3 g2((N + 127) / 128, (rows + 127) / 128, gz);
    if (g2.y > 65535 || g2.z > 65535) return fail("mrs_hyb_gemm: too many row tiles / groups for one launch");
    hipLaunchKernelGGL(gemm_tile128_bf16_kernel, g2, dim3(256), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? 0 : fail("mrs_hyb_gemm: launch failed");
  }
  dim3 grid((N + BN - 1) / BN, (rows + BM - 1) / BM, gz);
  if (grid.y > 65535 || grid.z > 65535) return fail("mrs_hyb_gemm: too many row tiles / groups for one launch");
  if (dtype == 1) hipLaunchKernelGGL(gemm_tile_bf16_kernel, grid, dim3(256), 0, (hipStream_t)stream, a);
  else hipLaunchKernelGGL(gemm_tile_f32_kernel, grid, dim3(256), 0, (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? 0 : fail("mrs_hyb_gemm: launch failed");
}

extern "C" int mrs_hyb_gemm(const void *A, const void *W, float *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int accumulate,
                            const int *bounds, int groups, long long wstride, int max_rows, void *stream) {
  return gemm_launch(A, W, C, M, N, K, lda, ldw, ldc, dtype, accumulate, bounds, groups, wstride, max_rows, 0, 0, 0, 0, stream);
}
/* `batch` products in one launch: product b multiplies A + b * a_bstride [M, K] (row stride lda) with W + b * wstride [N, K] into C + b * c_bstride (row stride ldc): the heads'
 * operands as column blocks of row-major buffers.  c_is_T: C holds dtype values (rounded once) instead of f32.  batch 0: one product.  At most 8 rows take the row kernel. */
extern "C" int mrs_hyb_gemm_batched(const void *A, const void *W, void *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int batch, long long a_bstride,
                                    long long wstride, long long c_bstride, int c_is_T, void *stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || ldc < N || (dtype != 1 && dtype != 2) || batch < 0) return fail("mrs_hyb_gemm_batched: bad shape / dtype");
  if (M > 8) return gemm_launch(A, W, C, M, N, K, lda, ldw, ldc, dtype, 0, nullptr, 0, wstride, 0, batch, a_bstride, c_bstride, c_is_T, stream);
  const int esz = dtype == 1 ? 2 : 4;
  GemvArgs a{A, W, (float *)C, M, N, K, lda, ldw, ldc, 0, nullptr, wstride,
             (K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && (wstride * esz) % 16 == 0 && (a_bstride * esz) % 16 == 0) ? 1 : 0,
             nullptr, nullptr, 1, nullptr, 0.f, 0.f, batch > 0 ? batch : 0, a_bstride, c_bstride, c_is_T};
  if (batch > 65535) return fail("mrs_hyb_gemm_batched: more than 65535 products in one batch");
  dim3 grid((N + 3) / 4, 1, batch > 0 ? batch : 1);
  hipStream_t s = (hipStream_t)stream;
#define MRS_GEMVB(T) do { if (M <= 1) hipLaunchKernelGGL((gemv_rows_kernel<T, 1, IN_PLAIN>), grid, dim3(256), 0, s, a); else if (M <= 2) hipLaunchKernelGGL((gemv_rows_kernel<T, 2, IN_PLAIN>), grid, dim3(256), 0, s, a); \
                          else if (M <= 4) hipLaunchKernelGGL((gemv_rows_kernel<T, 4, IN_PLAIN>), grid, dim3(256), 0, s, a); else hipLaunchKernelGGL((gemv_rows_kernel<T, 8, IN_PLAIN>), grid, dim3(256), 0, s, a); } while (0)
  if (dtype == 1) MRS_GEMVB(mrs::bf16_t); else MRS_GEMVB(float);
#undef MRS_GEMVB
  return hipGetLastError() == hipSuccess ? 0 : fail("mrs_hyb_gemm_batched: launch failed");
}

/* in_mode: 0 plain (A in dtype), 1 GLU (A = f32 [M, 2 K] gate | up), 2 scaled rows (A = f32 source rows; row m = src_scale[r] * A[r / src_div], r = src_row[m]; no
 * src_scale: the rows are gathered as they are), 3 clamped GLU (A = f32 [M, 2 K]; p0 = limit, p1 = the sigmoid's factor), 4 xIELU(A + in_bias) (p0, p1 = its coefficients), 5 max(A, 0)^2 (A = f32 [M, K]) */
extern "C" int mrs_hyb_gemv_act(const void *A, const void *W, float *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int accumulate, const int *row_group,
                                long long wstride, int in_mode, const int *src_row, const float *src_scale, int src_div, const float *in_bias, float p0, float p1, void *stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || ldc < N || (dtype != 1 && dtype != 2) || in_mode < 0 || in_mode > 5) return fail("mrs_hyb_gemv: bad shape / dtype / input mode");
  if ((in_mode == 1 || in_mode == 3) && lda < 2 * K) return fail("mrs_hyb_gemv: the gate | up operand needs rows of 2 K values");
  if (in_mode == 2 && (!src_row || src_div <= 0)) return fail("mrs_hyb_gemv: gathered rows need their source table");
  if (!row_group && M > 8) return fail("mrs_hyb_gemv: at most 8 rows share a weight");
  if (row_group && M > 65535) return fail("mrs_hyb_gemv: too many rows");
  const int esz = dtype == 1 ? 2 : 4;
  GemvArgs a{A, W, C, M, N, K, lda, ldw, ldc, accumulate, row_group, wstride,
             (K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && (wstride * esz) % 16 == 0 &&
              (!in_bias || ((uintptr_t)in_bias % 16) == 0)) ? 1 : 0, src_row, src_scale, src_div, in_bias, p0, p1, 0, 0, 0, 0};
  dim3 grid((N + 3) / 4, row_group ? M : 1);
  hipStream_t s = (hipStream_t)stream;
#define MRS_GEMV_(T, MR, IN) hipLaunchKernelGGL((gemv_rows_kernel<T, MR, IN>), grid, dim3(256), 0, s, a)
#define MRS_GEMV(T, MR) do { if (in_mode == 0) MRS_GEMV_(T, MR, IN_PLAIN); else if (in_mode == 1) MRS_GEMV_(T, MR, IN_GLU); else if (in_mode == 2) MRS_GEMV_(T, MR, IN_SCALED); \
                             else if (in_mode == 3) MRS_GEMV_(T, MR, IN_GLU_CLAMP); else if (in_mode == 4) MRS_GEMV_(T, MR, IN_BIAS_XIELU); else MRS_GEMV_(T, MR, IN_RELU_SQ); } while (0)
  const int mr = row_group ? 1 : M;
  if (dtype == 1) { if (mr <= 1) MRS_GEMV(mrs::bf16_t, 1); else if (mr <= 2) MRS_GEMV(mrs::bf16_t, 2); else if (mr <= 4) MRS_GEMV(mrs::bf16_t, 4); else MRS_GEMV(mrs::bf16_t, 8); }
  else { if (mr <= 1) MRS_GEMV(float, 1); else if (mr <= 2) MRS_GEMV(float, 2); else if (mr <= 4) MRS_GEMV(float, 4); else MRS_GEMV(float, 8); }
#undef MRS_GEMV
#undef MRS_GEMV_
  return hipGetLastError() == hipSuccess ? 0 : fail("mrs_hyb_gemv: launch failed");
}

extern "C" int mrs_hyb_gemv(const void *A, const void *W, float *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int accumulate,
                            const int *row_group, long long wstride, int in_mode, const int *src_row, const float *src_scale, int src_div, void *stream) {
  if (in_mode < 0 || in_mode > 2) return fail("mrs_hyb_gemv: bad shape / dtype / input mode");
  if (in_mode == 2 && !src_scale) return fail("mrs_hyb_gemv: scaled rows need their source table");
  return mrs_hyb_gemv_act(A, W, C, M, N, K, lda, ldw, ldc, dtype, accumulate, row_group, wstride, in_mode, src_row, src_scale, src_div, nullptr, 0.f, 0.f, stream);
}

// Kernels around attention through a cached latent: an RMS norm over a run of columns of a wider row, and a
// rotation by position of a part of every head's vector with a choice of pairing.  Both read 32-bit results of a
// product and write in the dtype of whatever reads them next, into a place of the caller's (a run of columns of a
// wider row), so that a norm, a rotation and the assembly of a cached row or of a query need no copies.
#include "common.h"

namespace {

// out[r, :] = src[r, :] / sqrt(mean(src[r, :]^2) + eps) * w; one workgroup a row
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_cols_kernel(const float* __restrict__ src, int lds_, const float* __restrict__ w,
                                                           float eps, T* __restrict__ out, int ldo, int n) {
  __shared__ float red[16];
  const float* s = src + (long long)blockIdx.x * lds_;
  T* o = out + (long long)blockIdx.x * ldo;
  float acc = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) acc = fmaf(s[i], s[i], acc);
  const float inv = 1.f / sqrtf(block_sum(acc, red) / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += 256) o[i] = from_f32<T>(s[i] * inv * w[i]);
}

// Row r, head h: the vector src[r, h * size .. + size) goes to out[r, h * ohs .. + size); its first `dims` entries
// are rotated by the angles row_pos[r] * freqs[j], in pairs (j, j + dims / 2) or (2 j, 2 j + 1): (u, v) ->
// (u c - v s, v c + u s) with c and s times `mag`; the rest pass.  Angles in double, reduced to [-pi, pi] before
// the 32-bit sine and cosine.
template <typename T>
__global__ __launch_bounds__(128) void rotary_kernel(const float* __restrict__ src, int lds_, T* __restrict__ out, int ldo,
                                                     int heads, int size, int ohs, int dims, int interleaved,
                                                     const double* __restrict__ freqs, float mag,
                                                     const int* __restrict__ row_pos) {
  extern __shared__ float cs[];  // cos[dims / 2], sin[dims / 2]
  const int r = blockIdx.x, half = dims / 2;
  const int p = row_pos[r];
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    const double a = (double)p * freqs[j];
    const double n = rint(a * 0.15915494309189533577);
    double rem = fma(-n, 6.283185307179586232, a);
    rem = fma(-n, 2.4492935982947064e-16, rem);
    float sn, c;
    sincosf((float)rem, &sn, &c);
    cs[j] = c * mag;
    cs[half + j] = sn * mag;
  }
  __syncthreads();
  const float* s = src + (long long)r * lds_;
  T* o = out + (long long)r * ldo;
  for (int e = threadIdx.x; e < heads * size; e += blockDim.x) {
    const int h = e / size, i = e - h * size;
    const float* v = s + h * size;
    float res;
    if (i >= dims) {
      res = v[i];
    } else {
      int j, mate;
      bool first;
      if (interleaved) j = i >> 1, first = !(i & 1), mate = i ^ 1;
      else first = i < half, j = first ? i : i - half, mate = first ? i + half : i - half;
      const float c = cs[j], sn = cs[half + j];
      res = first ? v[i] * c - v[mate] * sn : v[i] * c + v[mate] * sn;
    }
    o[h * ohs + i] = from_f32<T>(res);
  }
}

// Queries, keys and values of a step's rows, from the 32-bit result of their one product to what the attention
// kernel and the cache read.  src [rows, (H + G) D + G V]: H query heads, G key heads, G value heads.  Of every query
// and key head the first `dims` entries are rotated as in `rotary_kernel`; then, with norm_eps >= 0, the whole head
// is divided by its root mean square over D (eps inside the root); values pass.  gridDim.y workgroups a row share
// its heads and values out (one where the rows alone fill the chip); a wavefront takes a head at a time (its sum of
// squares is the wavefront's fixed tree, so it depends on the row alone, not on how the heads were shared out).
template <typename T>
__global__ __launch_bounds__(256) void rotary_qkv_kernel(const float* __restrict__ src, int lds_, T* __restrict__ q_out,
                                                         int ldq, T* __restrict__ k_out, int ldk, T* __restrict__ v_out,
                                                         int ldv, int H, int G, int D, int VW, int dims, int interleaved,
                                                         const double* __restrict__ freqs, float mag, float norm_eps,
                                                         const int* __restrict__ row_pos) {
  extern __shared__ float cs[];  // cos[dims / 2], sin[dims / 2]
  const int r = blockIdx.x, half = dims / 2;
  const int p = row_pos[r];
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    const double a = (double)p * freqs[j];
    const double n = rint(a * 0.15915494309189533577);
    double rem = fma(-n, 6.283185307179586232, a);
    rem = fma(-n, 2.4492935982947064e-16, rem);
    float sn, c;
    sincosf((float)rem, &sn, &c);
    cs[j] = c * mag;
    cs[half + j] = sn * mag;
  }
  __syncthreads();
  const float* s = src + (long long)r * lds_;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (int h = blockIdx.y * waves + wave; h < H + G; h += waves * gridDim.y) {
    const float* v = s + h * D;
    T* o = h < H ? q_out + (long long)r * ldq + h * D : k_out + (long long)r * ldk + (h - H) * D;
    auto turned = [&](int i) -> float {
      if (i >= dims) return v[i];
      int j, mate;
      bool first;
      if (interleaved) j = i >> 1, first = !(i & 1), mate = i ^ 1;
      else first = i < half, j = first ? i : i - half, mate = first ? i + half : i - half;
      const float c = cs[j], sn = cs[half + j];
      return first ? v[i] * c - v[mate] * sn : v[i] * c + v[mate] * sn;
    };
    float inv = 1.f;
    if (norm_eps >= 0.f) {
      float ss = 0.f;
      for (int i = lane; i < D; i += 64) {
        const float t = turned(i);
        ss = fmaf(t, t, ss);
      }
      inv = 1.f / sqrtf(wave_sum(ss) / (float)D + norm_eps);
    }
    for (int i = lane; i < D; i += 64) o[i] = from_f32<T>(turned(i) * inv);
  }
  const float* vs = s + (H + G) * D;
  T* vo = v_out + (long long)r * ldv;
  for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < VW; e += blockDim.x * gridDim.y) vo[e] = from_f32<T>(vs[e]);
}

// A product a head: out[r, h ohs + n] = sum_k x[r, h K + k] w[h, n, k], bfloat16 operands on
// v_mfma_f32_16x16x16_bf16 (exact products, 32-bit sums).  A workgroup of four wavefronts takes 64 rows by 64
// columns of one head; a wavefront 16 rows by the 64 columns, its operands straight from memory (a head's weight
// is small and stays in the caches; the four wavefronts read the same columns).  K in steps of 16, ascending: a
// row's sums do not depend on what else is in the launch.
typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <typename TO>
__global__ __launch_bounds__(256) void linear_heads_kernel(const bf16_t* __restrict__ x, int ldx,
                                                           const bf16_t* __restrict__ w, TO* __restrict__ out, int ldo,
                                                           int rows, int N, int K, int ohs) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  const int h = blockIdx.z, r0 = blockIdx.x * 64 + 16 * wave, n0 = blockIdx.y * 64;
  if (r0 >= rows) return;
  const bf16_t* xa = x + (long long)min(r0 + c, rows - 1) * ldx + (long long)h * K + 4 * g;
  const bf16_t* wb[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) wb[j] = w + ((long long)h * N + min(n0 + 16 * j + c, N - 1)) * K + 4 * g;
  f32x4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  for (int ks = 0; ks < K; ks += 16) {
    const bf16x4_t a = __builtin_bit_cast(bf16x4_t, *(const uint2*)(xa + ks));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bf16x4_t bv = __builtin_bit_cast(bf16x4_t, *(const uint2*)(wb[j] + ks));
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, bv, acc[j], 0, 0, 0);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + 16 * j + c;
    if (n >= N) continue;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int r = r0 + 4 * g + e;
      if (r < rows) out[(long long)r * ldo + (long long)h * ohs + n] = from_f32<TO>(acc[j][e]);
    }
  }
}

}  // namespace

extern "C" int lq_rmsnorm_cols(const float* src, int lds_, const float* w, float eps, void* out, int out_dtype, int ldo,
                               int rows, int n, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && n > 0 && lds_ >= n && ldo >= n, "rmsnorm_cols: rows %d, columns %d, strides %d and %d", rows, n, lds_, ldo);
  LQ_REQUIRE(src && w && out, "rmsnorm_cols: null pointer");
  if (out_dtype == LQ_F32) rmsnorm_cols_kernel<float><<<rows, 256, 0, stream>>>(src, lds_, w, eps, (float*)out, ldo, n);
  else if (out_dtype == LQ_BF16) rmsnorm_cols_kernel<bf16_t><<<rows, 256, 0, stream>>>(src, lds_, w, eps, (bf16_t*)out, ldo, n);
  else LQ_REQUIRE(false, "rmsnorm_cols: unknown dtype %d", out_dtype);
  LQ_CHECK_LAUNCH("rmsnorm_cols");
  return 0;
}

extern "C" int lq_rotary(const float* src, int lds_, void* out, int out_dtype, int ldo, int rows, int heads, int size,
                         int out_head_stride, int dims, int interleaved, const double* freqs, float magnitude,
                         const int* row_pos, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && heads > 0 && size > 0, "rotary: rows %d, heads %d, size %d", rows, heads, size);
  LQ_REQUIRE(dims >= 2 && dims % 2 == 0 && dims <= size && dims <= 8192, "rotary: %d rotated entries of %d", dims, size);
  LQ_REQUIRE(out_head_stride >= size && lds_ >= heads * size && ldo >= (heads - 1) * out_head_stride + size,
             "rotary: a stride is smaller than what it steps over");
  LQ_REQUIRE(src && out && freqs && row_pos, "rotary: null pointer");
  const size_t lds_bytes = (size_t)dims * sizeof(float);
  if (out_dtype == LQ_F32)
    rotary_kernel<float><<<rows, 128, lds_bytes, stream>>>(src, lds_, (float*)out, ldo, heads, size, out_head_stride, dims,
                                                           interleaved, freqs, magnitude, row_pos);
  else if (out_dtype == LQ_BF16)
    rotary_kernel<bf16_t><<<rows, 128, lds_bytes, stream>>>(src, lds_, (bf16_t*)out, ldo, heads, size, out_head_stride, dims,
                                                            interleaved, freqs, magnitude, row_pos);
  else LQ_REQUIRE(false, "rotary: unknown dtype %d", out_dtype);
  LQ_CHECK_LAUNCH("rotary");
  return 0;
}

// src [rows, (heads + kv_heads) * key_dim + kv_heads * value_dim] float32 (stride lds_): queries, keys, values.
// dims = 0: no rotation (freqs may be null); norm_eps < 0: no norm.
extern "C" int lq_rotary_qkv(const float* src, int lds_, void* q_out, int ldq, void* k_out, int ldk, void* v_out, int ldv,
                             int out_dtype, int rows, int heads, int kv_heads, int key_dim, int value_dim, int dims,
                             int interleaved, const double* freqs, float magnitude, float norm_eps, const int* row_pos,
                             int value_width, hipStream_t stream) {
  // `value_width` > 0: so many value entries a row pass, in the place of kv_heads * value_dim (key heads that share
  // a value head)
  const int VW = value_width > 0 ? value_width : kv_heads * value_dim;
  LQ_REQUIRE(rows > 0 && heads > 0 && kv_heads > 0 && key_dim > 0 && value_dim > 0, "rotary_qkv: rows %d, heads %d and %d, sizes %d and %d",
             rows, heads, kv_heads, key_dim, value_dim);
  LQ_REQUIRE(dims >= 0 && dims % 2 == 0 && dims <= key_dim && dims <= 8192, "rotary_qkv: %d rotated entries of %d", dims, key_dim);
  LQ_REQUIRE(lds_ >= (heads + kv_heads) * key_dim + VW && ldq >= heads * key_dim && ldk >= kv_heads * key_dim &&
                 ldv >= VW, "rotary_qkv: a row stride is smaller than its row");
  LQ_REQUIRE(src && q_out && k_out && v_out && row_pos && (dims == 0 || freqs), "rotary_qkv: null pointer");
  const size_t lds_bytes = (size_t)dims * sizeof(float);
  // few rows (single tokens): a wavefront a head, so that no wavefront walks through its heads one after the other
  const int share = rows >= 512 ? 1 : (lq_ceil_div(heads + kv_heads, 4) < 64 ? lq_ceil_div(heads + kv_heads, 4) : 64);
  const dim3 grid(rows, share);
  if (out_dtype == LQ_F32)
    rotary_qkv_kernel<float><<<grid, 256, lds_bytes, stream>>>(src, lds_, (float*)q_out, ldq, (float*)k_out, ldk, (float*)v_out,
                                                               ldv, heads, kv_heads, key_dim, VW, dims, interleaved,
                                                               freqs, magnitude, norm_eps, row_pos);
  else if (out_dtype == LQ_BF16)
    rotary_qkv_kernel<bf16_t><<<grid, 256, lds_bytes, stream>>>(src, lds_, (bf16_t*)q_out, ldq, (bf16_t*)k_out, ldk,
                                                                (bf16_t*)v_out, ldv, heads, kv_heads, key_dim, VW, dims,
                                                                interleaved, freqs, magnitude, norm_eps, row_pos);
  else LQ_REQUIRE(false, "rotary_qkv: unknown dtype %d", out_dtype);
  LQ_CHECK_LAUNCH("rotary_qkv");
  return 0;
}

// Whether lq_linear_heads takes these operands (else the caller runs a product a head).
extern "C" int lq_linear_heads_accepts(const void* x, const void* w, int in_dtype, int K, int ldx) {
  return in_dtype == LQ_BF16 && K % 16 == 0 && ldx % 4 == 0 && ((uintptr_t)x % 8) == 0 && ((uintptr_t)w % 8) == 0;
}

// x [rows, heads * K] (stride ldx), w [heads, N, K] dense, out: head h's N columns from column h * out_head_stride
extern "C" int lq_linear_heads(const void* x, int ldx, const void* w, void* out, int in_dtype, int out_dtype, int ldo,
                               int rows, int heads, int N, int K, int out_head_stride, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && heads > 0 && heads <= 65535 && N > 0 && K > 0, "linear_heads: rows %d, heads %d, N %d, K %d", rows,
             heads, N, K);
  LQ_REQUIRE(ldx >= heads * K && out_head_stride >= N && ldo >= (heads - 1) * out_head_stride + N,
             "linear_heads: a stride is smaller than what it steps over");
  LQ_REQUIRE(x && w && out, "linear_heads: null pointer");
  LQ_REQUIRE(lq_linear_heads_accepts(x, w, in_dtype, K, ldx), "linear_heads: bfloat16 operands, K in 16s, rows on 8 bytes");
  LQ_REQUIRE(lq_ceil_div(N, 64) <= 65535, "linear_heads: too many columns");
  dim3 grid(lq_ceil_div(rows, 64), lq_ceil_div(N, 64), heads);
  if (out_dtype == LQ_F32)
    linear_heads_kernel<float><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, (float*)out, ldo, rows, N, K,
                                                         out_head_stride);
  else if (out_dtype == LQ_BF16)
    linear_heads_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, (bf16_t*)out, ldo, rows, N,
                                                          K, out_head_stride);
  else LQ_REQUIRE(false, "linear_heads: unknown dtype %d", out_dtype);
  LQ_CHECK_LAUNCH("linear_heads");
  return 0;
}

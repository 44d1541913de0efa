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

// Kernels of the mixers with a recurrent state (the Mamba-2 state-space layer, the gated delta rule), of the
// short causal convolution in front of them, and of the element-wise steps around them: Dynamic Tanh, the
// scaled residual add, a gated linear unit's activation, the gated RMS norm in groups, the mean of RMS-normed
// branches.  Everything is 32-bit arithmetic; only an output that feeds a matrix product is rounded to the run's
// dtype.
//
// The scans walk a sequence's tokens in order, one workgroup a (sequence, head, slice of the head's columns),
// the state in registers, and are the same kernel for a prompt and for single tokens: a token's result is made of
// the same operations in the same order however the sequence was cut into steps and whatever else is in the batch.
#include "common.h"

namespace {

__device__ inline float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ inline float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ inline float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ inline float gelu_tanh_f(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

enum { ACT_NONE = 0, ACT_SILU = 1, ACT_RELU = 2, ACT_GELU_TANH = 3 };

__device__ inline float activate(float z, int act) {
  switch (act) {
    case ACT_SILU: return silu_f(z);
    case ACT_RELU: return fmaxf(z, 0.f);
    case ACT_GELU_TANH: return gelu_tanh_f(z);
    default: return z;
  }
}

template <typename T>
__device__ inline void store_as(T* p, float v);
template <>
__device__ inline void store_as<float>(float* p, float v) { *p = v; }
template <>
__device__ inline void store_as<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// ---------------------------------------------------------------- Dynamic Tanh and the scaled add
// (x += scale * (piece 0 + piece 1 + ...);)  out = tanh(alpha x) w + b
template <typename T>
__global__ __launch_bounds__(256) void dynamic_tanh_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                                           int pieces, long long piece_stride, float scale,
                                                           const float* __restrict__ w, const float* __restrict__ b,
                                                           const float* __restrict__ alpha, T* __restrict__ out,
                                                           long long n, int width) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float v = x[i];
  if (pieces > 0) {
    float d = delta[i];
    for (int p = 1; p < pieces; ++p) d += delta[i + p * piece_stride];
    v += scale * d;
    x[i] = v;
  }
  const int c = (int)(i % width);
  store_as<T>(out + i, tanhf(alpha[0] * v) * w[c] + b[c]);
}

__global__ __launch_bounds__(256) void add_scaled_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                                         int pieces, long long piece_stride, float scale, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float d = delta[i];
  for (int p = 1; p < pieces; ++p) d += delta[i + p * piece_stride];
  x[i] += scale * d;
}

// out[r, c] = act(gu[r, c]) * gu[r, I + c]
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void glu_kernel(const TI* __restrict__ gu, int ld, TO* __restrict__ out, int ldo,
                                                  int I, int act) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= I) return;
  const float g = to_f32(gu[(long long)r * ld + c]), u = to_f32(gu[(long long)r * ld + I + c]);
  store_as<TO>(out + (long long)r * ldo + c, activate(g, act) * u);
}

// ---------------------------------------------------------------- short causal convolution
// y[t, c] = act(bias[c] + sum_j w[c, j] x[t - (taps - 1) + j, c]); inputs before this step's rows come from
// the sequence's state (its last taps - 1 inputs, zeros at the start of a sequence).
__global__ __launch_bounds__(256) void causal_conv_kernel(const float* __restrict__ x, int ldx,
                                                          const float* __restrict__ w, const float* __restrict__ bias,
                                                          const float* __restrict__ state, float* __restrict__ out,
                                                          int ldo, int C, int taps, const int* __restrict__ row_seq,
                                                          const int* __restrict__ row_pos,
                                                          const int* __restrict__ seq_slot,
                                                          const int* __restrict__ seq_start,
                                                          const int* __restrict__ cu_rows, int act) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int b = row_seq[r];
  const int since = row_pos[r] - seq_start[b];  // rows of this step before this one, in its sequence
  const long long first = cu_rows[b];
  const float* st = state + (long long)seq_slot[b] * (taps - 1) * C;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;  // how many tokens before this one
    const float v = back <= since ? x[(first + since - back) * ldx + c] : st[(long long)(taps - 1 - (back - since)) * C + c];
    acc = fmaf(w[(long long)c * taps + j], v, acc);
  }
  if (bias != nullptr) acc += bias[c];
  out[(long long)r * ldo + c] = activate(acc, act);
}

// The state after the step: the last taps - 1 inputs of each sequence (old ones move up where the step brought fewer).
__global__ __launch_bounds__(256) void conv_state_kernel(const float* __restrict__ x, int ldx, float* __restrict__ state,
                                                         int C, int taps, const int* __restrict__ seq_slot,
                                                         const int* __restrict__ cu_rows) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const long long first = cu_rows[b];
  const int n_new = (int)(cu_rows[b + 1] - first);
  float* st = state + (long long)seq_slot[b] * (taps - 1) * C;
  for (int j = 0; j < taps - 1; ++j) {  // ascending: entry j is written after entry j + n_new was read
    const int src = j + n_new;
    st[(long long)j * C + c] = src < taps - 1 ? st[(long long)src * C + c] : x[(first + src - (taps - 1)) * ldx + c];
  }
}

// ---------------------------------------------------------------- the scans
// A head's state is [columns P][state size N] in memory.  A thread owns, of one column, the entries n = i LN + l
// (i = 0 .. slab - 1): LN threads share a column, LN a power of two, slab = ceil(N / LN) <= 16.  Sums over n are
// a thread's own entries in ascending i, then an exchange over the LN lanes.
constexpr int SLAB = 16;
constexpr int SCAN_CHUNK = 8;  // tokens whose shared inputs are staged in LDS at a time

template <int LN>
__device__ inline float group_sum(float v) {
#pragma unroll
  for (int off = 1; off < LN; off <<= 1) v += __shfl_xor(v, off, LQ_WAVE);
  return v;
}

// Mamba-2: S <- exp(-exp(A_log) dt) S + dt B x^T,  y = S^T C + D x,  dt = softplus(raw + bias)
template <int LN>
__global__ void ssd_scan_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ Bm, int ldb,
                                const float* __restrict__ Cm, int ldc, const float* __restrict__ dt, int lddt,
                                const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                const float* __restrict__ d_skip, float* __restrict__ state, float* __restrict__ y,
                                int ldy, int heads, int P, int N, int groups, const int* __restrict__ seq_slot,
                                const int* __restrict__ cu_rows) {
  extern __shared__ float lds[];  // [chunk][B: N | C: N] then [chunk][decay, dt]
  const int b = blockIdx.x / heads, h = blockIdx.x % heads, g = h / (heads / groups);
  const int cols = blockDim.x / LN;
  const int l = threadIdx.x % LN, p = blockIdx.y * cols + threadIdx.x / LN;
  const bool live = p < P;
  const int slab = (N + LN - 1) / LN;
  const long long r0 = cu_rows[b], r1 = cu_rows[b + 1];
  float* sp = state + (((long long)seq_slot[b] * heads + h) * P + (live ? p : 0)) * N;
  float* scal = lds + SCAN_CHUNK * 2 * N;
  float S[SLAB];
#pragma unroll
  for (int i = 0; i < SLAB; ++i) {
    const int n = i * LN + l;
    S[i] = (live && i < slab && n < N) ? sp[n] : 0.f;
  }
  const float A = -expf(a_log[h]), bias = dt_bias[h], D = d_skip[h];
  for (long long c0 = r0; c0 < r1; c0 += SCAN_CHUNK) {
    const int nt = (int)min((long long)SCAN_CHUNK, r1 - c0);
    __syncthreads();  // the chunk before has been read
    for (int e = threadIdx.x; e < nt * N; e += blockDim.x) {
      const int t = e / N, n = e - t * N;
      lds[t * 2 * N + n] = Bm[(c0 + t) * ldb + g * N + n];
      lds[t * 2 * N + N + n] = Cm[(c0 + t) * ldc + g * N + n];
    }
    if (threadIdx.x < nt) {
      const float step = softplus_f(dt[(c0 + threadIdx.x) * lddt + h] + bias);
      scal[2 * threadIdx.x] = expf(A * step);
      scal[2 * threadIdx.x + 1] = step;
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float decay = scal[2 * t], step = scal[2 * t + 1];
      const float xv = live ? x[(c0 + t) * ldx + h * P + p] : 0.f;
      const float dx = step * xv;
      const float* Bs = lds + t * 2 * N;
      const float* Cs = Bs + N;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < SLAB; ++i) {
        const int n = i * LN + l;
        if (i < slab && n < N) {
          S[i] = fmaf(Bs[n], dx, decay * S[i]);
          acc = fmaf(S[i], Cs[n], acc);
        }
      }
      acc = group_sum<LN>(acc);
      if (live && l == 0) y[(c0 + t) * ldy + h * P + p] = fmaf(D, xv, acc);
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < SLAB; ++i) {
      const int n = i * LN + l;
      if (i < slab && n < N) sp[n] = S[i];
    }
  }
}

// Gated delta rule: S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q, with q and k made unit
// vectors (x / sqrt(sum x^2 + unit_eps)), q times q_scale, beta = sigmoid(raw), g = exp(-exp(A_log) softplus(raw + bias)).
template <int LN>
__global__ void delta_scan_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk,
                                  const float* __restrict__ v, int ldv, const float* __restrict__ beta, int ldbeta,
                                  const float* __restrict__ a, int lda, const float* __restrict__ dt_bias,
                                  const float* __restrict__ a_log, float* __restrict__ state, float* __restrict__ out,
                                  int ldo, int heads, int kv_heads, int Dk, int P, float q_scale, float unit_eps,
                                  const int* __restrict__ seq_slot, const int* __restrict__ cu_rows) {
  extern __shared__ float lds[];  // [chunk][q: Dk | k: Dk] then [chunk][decay, beta]
  const int b = blockIdx.x / heads, h = blockIdx.x % heads, j = h / (heads / kv_heads);
  const int cols = blockDim.x / LN;
  const int l = threadIdx.x % LN, p = blockIdx.y * cols + threadIdx.x / LN;
  const bool live = p < P;
  const int slab = (Dk + LN - 1) / LN;
  const long long r0 = cu_rows[b], r1 = cu_rows[b + 1];
  float* sp = state + (((long long)seq_slot[b] * heads + h) * P + (live ? p : 0)) * Dk;
  float* scal = lds + SCAN_CHUNK * 2 * Dk;
  float S[SLAB];
#pragma unroll
  for (int i = 0; i < SLAB; ++i) {
    const int n = i * LN + l;
    S[i] = (live && i < slab && n < Dk) ? sp[n] : 0.f;
  }
  const float A = -expf(a_log[h]), bias = dt_bias[h];
  for (long long c0 = r0; c0 < r1; c0 += SCAN_CHUNK) {
    const int nt = (int)min((long long)SCAN_CHUNK, r1 - c0);
    __syncthreads();
    for (int e = threadIdx.x; e < nt * Dk; e += blockDim.x) {
      const int t = e / Dk, n = e - t * Dk;
      lds[t * 2 * Dk + n] = q[(c0 + t) * ldq + j * Dk + n];
      lds[t * 2 * Dk + Dk + n] = k[(c0 + t) * ldk + j * Dk + n];
    }
    if (threadIdx.x < nt) {
      scal[2 * threadIdx.x] = expf(A * softplus_f(a[(c0 + threadIdx.x) * lda + h] + bias));
      scal[2 * threadIdx.x + 1] = sigmoid_f(beta[(c0 + threadIdx.x) * ldbeta + h]);
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float decay = scal[2 * t], bt = scal[2 * t + 1];
      const float vv = live ? v[(c0 + t) * ldv + h * P + p] : 0.f;
      const float* Qs = lds + t * 2 * Dk;
      const float* Ks = Qs + Dk;
      float kk[SLAB], qq[SLAB];
      float ssq = 0.f, ssk = 0.f;
#pragma unroll
      for (int i = 0; i < SLAB; ++i) {
        const int n = i * LN + l;
        const bool in = i < slab && n < Dk;
        kk[i] = in ? Ks[n] : 0.f;
        qq[i] = in ? Qs[n] : 0.f;
        ssk = fmaf(kk[i], kk[i], ssk);
        ssq = fmaf(qq[i], qq[i], ssq);
      }
      const float kinv = 1.f / sqrtf(group_sum<LN>(ssk) + unit_eps);
      const float qinv = q_scale / sqrtf(group_sum<LN>(ssq) + unit_eps);
      float sk = 0.f;
#pragma unroll
      for (int i = 0; i < SLAB; ++i) {
        kk[i] *= kinv;
        S[i] *= decay;
        sk = fmaf(S[i], kk[i], sk);
      }
      const float u = bt * (vv - group_sum<LN>(sk));
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < SLAB; ++i) {
        S[i] = fmaf(kk[i], u, S[i]);
        o = fmaf(S[i], qq[i], o);
      }
      o = group_sum<LN>(o) * qinv;
      if (live && l == 0) out[(c0 + t) * ldo + h * P + p] = o;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < SLAB; ++i) {
      const int n = i * LN + l;
      if (i < slab && n < Dk) sp[n] = S[i];
    }
  }
}

// ---------------------------------------------------------------- norms after the scans
// One workgroup a (row, group of `group` columns).  gate_first: v = y silu(z), out = v / rms(v) w;
// else: out = y / rms(y) w silu(z).  w has `wlen` entries and repeats (one weight for all groups, or one a column).
template <typename T>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ y, int ldy, const float* __restrict__ z, int ldz,
                                     const float* __restrict__ w, int wlen, float eps, int group, T* __restrict__ out,
                                     int ldo, int gate_first) {
  __shared__ float red[16];
  const int r = blockIdx.y, c0 = blockIdx.x * group;
  const float* yr = y + (long long)r * ldy + c0;
  const float* zr = z + (long long)r * ldz + c0;
  float ss = 0.f;
  for (int c = threadIdx.x; c < group; c += blockDim.x) {
    const float v = gate_first ? yr[c] * silu_f(zr[c]) : yr[c];
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / group + eps);
  for (int c = threadIdx.x; c < group; c += blockDim.x) {
    const float gate = silu_f(zr[c]);
    const float v = gate_first ? yr[c] * gate * inv * w[(c0 + c) % wlen] : yr[c] * inv * w[(c0 + c) % wlen] * gate;
    store_as<T>(out + (long long)r * ldo + c0 + c, v);
  }
}

struct MeanInputs {
  const float* x[4];
  const float* w[4];
};

// out = (1 / n) sum_i x_i / rms(x_i) w_i, row by row
__global__ void rmsnorm_mean_kernel(MeanInputs in, int n_in, float eps, float* __restrict__ out, int width) {
  __shared__ float red[16];
  const long long r = blockIdx.x;
  float inv[4];
  for (int i = 0; i < n_in; ++i) {
    const float* xr = in.x[i] + r * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) ss = fmaf(xr[c], xr[c], ss);
    inv[i] = 1.f / sqrtf(block_sum(ss, red) / width + eps);
  }
  const float share = 1.f / n_in;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = 0.f;
    for (int i = 0; i < n_in; ++i) acc += in.x[i][r * width + c] * inv[i] * in.w[i][c];
    out[r * width + c] = acc * share;
  }
}

int scan_lanes(int n) {  // the power of two LN with ceil(n / LN) <= SLAB
  int ln = 1;
  while ((n + ln - 1) / ln > SLAB) ln <<= 1;
  return ln;
}

// threads a workgroup: as many columns as fit, fewer where the launch would otherwise leave compute units idle
int scan_threads(int ln, int P, long long seq_heads) {
  int threads = 256;
  while (threads > 64 && (threads / ln >= 2 * P || seq_heads * lq_ceil_div(P, threads / ln) < 2ll * lq_compute_units()))
    threads >>= 1;
  return threads < ln ? ln : threads;
}

}  // namespace

extern "C" int lq_dynamic_tanh(float* x, const float* delta, int pieces, long long piece_stride, float scale,
                               const float* w, const float* b, const float* alpha, void* out, int out_dtype, int rows,
                               int width, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && width > 0, "dynamic_tanh: rows %d and width %d must be positive", rows, width);
  LQ_REQUIRE(x && w && b && alpha && out, "dynamic_tanh: null pointer");
  LQ_REQUIRE(pieces >= 0 && (pieces == 0 || delta != nullptr), "dynamic_tanh: %d pieces of a delta", pieces);
  const long long n = (long long)rows * width;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (out_dtype == LQ_F32)
    dynamic_tanh_kernel<float><<<blocks, 256, 0, stream>>>(x, delta, pieces, piece_stride, scale, w, b, alpha, (float*)out, n, width);
  else if (out_dtype == LQ_BF16)
    dynamic_tanh_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, delta, pieces, piece_stride, scale, w, b, alpha, (bf16_t*)out, n, width);
  else
    LQ_REQUIRE(false, "dynamic_tanh: unknown dtype %d", out_dtype);
  LQ_CHECK_LAUNCH("dynamic_tanh");
  return 0;
}

extern "C" int lq_add_scaled(float* x, const float* delta, int pieces, long long piece_stride, float scale, long long n,
                             hipStream_t stream) {
  LQ_REQUIRE(x && delta && pieces > 0 && n > 0, "add_scaled: bad arguments");
  add_scaled_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, delta, pieces, piece_stride, scale, n);
  LQ_CHECK_LAUNCH("add_scaled");
  return 0;
}

extern "C" int lq_glu(const void* gu, int in_dtype, int ld, void* out, int out_dtype, int ldo, int rows, int I, int act,
                      hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && I > 0 && ld >= 2 * I && ldo >= I, "glu: rows %d, inner %d, strides %d and %d", rows, I, ld, ldo);
  LQ_REQUIRE(act >= ACT_SILU && act <= ACT_GELU_TANH, "glu: unknown activation %d", act);
  LQ_REQUIRE(rows <= 65535 * 64, "glu: too many rows");
  LQ_REQUIRE(gu && out, "glu: null pointer");
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    dim3 grid(lq_ceil_div(I, 256), nr);
#define LQ_GLU(TI, TO)                                                                                              \
  glu_kernel<TI, TO><<<grid, 256, 0, stream>>>((const TI*)gu + (long long)r0 * ld, ld, (TO*)out + (long long)r0 * ldo, \
                                               ldo, I, act)
    if (in_dtype == LQ_F32 && out_dtype == LQ_F32) LQ_GLU(float, float);
    else if (in_dtype == LQ_F32 && out_dtype == LQ_BF16) LQ_GLU(float, bf16_t);
    else if (in_dtype == LQ_BF16 && out_dtype == LQ_BF16) LQ_GLU(bf16_t, bf16_t);
    else if (in_dtype == LQ_BF16 && out_dtype == LQ_F32) LQ_GLU(bf16_t, float);
    else LQ_REQUIRE(false, "glu: unknown dtypes %d, %d", in_dtype, out_dtype);
#undef LQ_GLU
  }
  LQ_CHECK_LAUNCH("glu");
  return 0;
}

// x [rows, C] (stride ldx), w [C, taps], bias [C] or null, state [slots, taps - 1, C]; out [rows, C] (stride ldo).
// The state is read for the step's outputs and then moved on by a second launch.
extern "C" int lq_causal_conv(const float* x, int ldx, const float* w, const float* bias, float* state, float* out,
                              int ldo, int rows, int C, int taps, const int* row_seq, const int* row_pos,
                              const int* seq_slot, const int* seq_start, const int* cu_rows, int batch, int act,
                              hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && C > 0 && taps >= 1 && batch > 0, "causal_conv: rows %d, channels %d, taps %d, sequences %d", rows, C,
             taps, batch);
  LQ_REQUIRE(ldx >= C && ldo >= C, "causal_conv: a row stride is smaller than its row");
  LQ_REQUIRE(x && w && out && row_seq && row_pos && seq_slot && seq_start && cu_rows && (taps == 1 || state),
             "causal_conv: null pointer");
  LQ_REQUIRE(act >= ACT_NONE && act <= ACT_GELU_TANH, "causal_conv: unknown activation %d", act);
  LQ_REQUIRE(batch <= 65535, "causal_conv: too many sequences");
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    causal_conv_kernel<<<dim3(lq_ceil_div(C, 256), nr), 256, 0, stream>>>(
        x, ldx, w, bias, state, out + (long long)r0 * ldo, ldo, C, taps, row_seq + r0, row_pos + r0, seq_slot, seq_start,
        cu_rows, act);
  }
  LQ_CHECK_LAUNCH("causal_conv");
  if (taps > 1) {
    conv_state_kernel<<<dim3(lq_ceil_div(C, 256), batch), 256, 0, stream>>>(x, ldx, state, C, taps, seq_slot, cu_rows);
    LQ_CHECK_LAUNCH("causal_conv(state)");
  }
  return 0;
}

#define LQ_SCAN_LANES(LAUNCH)          \
  switch (ln) {                        \
    case 1: LAUNCH(1); break;          \
    case 2: LAUNCH(2); break;          \
    case 4: LAUNCH(4); break;          \
    case 8: LAUNCH(8); break;          \
    case 16: LAUNCH(16); break;        \
    case 32: LAUNCH(32); break;        \
    default: LAUNCH(64); break;        \
  }

// x [rows, heads * P], B and C [rows, groups * N], dt [rows, heads] (before its softplus), state
// [slots, heads, P, N], y [rows, heads * P]; rows lie sequence by sequence (cu_rows).
extern "C" int lq_ssd_scan(const float* x, int ldx, const float* Bm, int ldb, const float* Cm, int ldc, const float* dt,
                           int lddt, const float* dt_bias, const float* a_log, const float* d_skip, float* state, float* y,
                           int ldy, int heads, int P, int N, int groups, const int* seq_slot, const int* cu_rows, int batch,
                           hipStream_t stream) {
  LQ_REQUIRE(heads > 0 && P > 0 && N > 0 && groups > 0 && heads % groups == 0 && batch > 0, "ssd_scan: bad sizes");
  LQ_REQUIRE(N <= SLAB * 64, "ssd_scan: state size %d exceeds %d", N, SLAB * 64);
  LQ_REQUIRE(ldx >= heads * P && ldy >= heads * P && ldb >= groups * N && ldc >= groups * N && lddt >= heads,
             "ssd_scan: a row stride is smaller than its row");
  LQ_REQUIRE(x && Bm && Cm && dt && dt_bias && a_log && d_skip && state && y && seq_slot && cu_rows, "ssd_scan: null pointer");
  const int ln = scan_lanes(N);
  const int threads = scan_threads(ln, P, (long long)batch * heads);
  dim3 grid((unsigned)(batch * heads), lq_ceil_div(P, threads / ln));
  const size_t lds = (size_t)SCAN_CHUNK * (2 * N + 2) * sizeof(float);
  LQ_REQUIRE(lds <= 64 * 1024, "ssd_scan: state size %d needs too much LDS", N);
#define LQ_SSD(LN)                                                                                                      \
  ssd_scan_kernel<LN><<<grid, threads, lds, stream>>>(x, ldx, Bm, ldb, Cm, ldc, dt, lddt, dt_bias, a_log, d_skip, state, \
                                                      y, ldy, heads, P, N, groups, seq_slot, cu_rows)
  LQ_SCAN_LANES(LQ_SSD)
#undef LQ_SSD
  LQ_CHECK_LAUNCH("ssd_scan");
  return 0;
}

// q and k [rows, kv_heads * Dk], v [rows, heads * P], beta and a [rows, heads] (raw), state [slots, heads, P, Dk],
// out [rows, heads * P]
extern "C" int lq_delta_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* beta,
                             int ldbeta, const float* a, int lda, const float* dt_bias, const float* a_log, float* state,
                             float* out, int ldo, int heads, int kv_heads, int Dk, int P, float q_scale, float unit_eps,
                             const int* seq_slot, const int* cu_rows, int batch, hipStream_t stream) {
  LQ_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && Dk > 0 && P > 0 && batch > 0, "delta_scan: bad sizes");
  LQ_REQUIRE(Dk <= SLAB * 64, "delta_scan: key size %d exceeds %d", Dk, SLAB * 64);
  LQ_REQUIRE(ldq >= kv_heads * Dk && ldk >= kv_heads * Dk && ldv >= heads * P && ldo >= heads * P && ldbeta >= heads &&
                 lda >= heads, "delta_scan: a row stride is smaller than its row");
  LQ_REQUIRE(q && k && v && beta && a && dt_bias && a_log && state && out && seq_slot && cu_rows, "delta_scan: null pointer");
  const int ln = scan_lanes(Dk);
  const int threads = scan_threads(ln, P, (long long)batch * heads);
  dim3 grid((unsigned)(batch * heads), lq_ceil_div(P, threads / ln));
  const size_t lds = (size_t)SCAN_CHUNK * (2 * Dk + 2) * sizeof(float);
  LQ_REQUIRE(lds <= 64 * 1024, "delta_scan: key size %d needs too much LDS", Dk);
#define LQ_DELTA(LN)                                                                                                 \
  delta_scan_kernel<LN><<<grid, threads, lds, stream>>>(q, ldq, k, ldk, v, ldv, beta, ldbeta, a, lda, dt_bias, a_log,  \
                                                        state, out, ldo, heads, kv_heads, Dk, P, q_scale, unit_eps,    \
                                                        seq_slot, cu_rows)
  LQ_SCAN_LANES(LQ_DELTA)
#undef LQ_DELTA
  LQ_CHECK_LAUNCH("delta_scan");
  return 0;
}

extern "C" int lq_gated_rmsnorm(const float* y, int ldy, const float* z, int ldz, const float* w, int wlen, float eps,
                                int group, void* out, int out_dtype, int ldo, int rows, int n, int gate_first,
                                hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && n > 0 && group > 0 && n % group == 0, "gated_rmsnorm: %d columns in groups of %d", n, group);
  LQ_REQUIRE(wlen > 0 && (wlen == n || group % wlen == 0), "gated_rmsnorm: a weight of %d entries for groups of %d", wlen, group);
  LQ_REQUIRE(ldy >= n && ldz >= n && ldo >= n, "gated_rmsnorm: a row stride is smaller than its row");
  LQ_REQUIRE(y && z && w && out, "gated_rmsnorm: null pointer");
  const int threads = group >= 1024 ? 256 : group > 64 ? 128 : 64;
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    dim3 grid(n / group, nr);
    if (out_dtype == LQ_F32)
      gated_rmsnorm_kernel<float><<<grid, threads, 0, stream>>>(y + (long long)r0 * ldy, ldy, z + (long long)r0 * ldz, ldz, w,
                                                               wlen, eps, group, (float*)out + (long long)r0 * ldo, ldo, gate_first);
    else if (out_dtype == LQ_BF16)
      gated_rmsnorm_kernel<bf16_t><<<grid, threads, 0, stream>>>(y + (long long)r0 * ldy, ldy, z + (long long)r0 * ldz, ldz, w,
                                                                wlen, eps, group, (bf16_t*)out + (long long)r0 * ldo, ldo, gate_first);
    else
      LQ_REQUIRE(false, "gated_rmsnorm: unknown dtype %d", out_dtype);
  }
  LQ_CHECK_LAUNCH("gated_rmsnorm");
  return 0;
}

// stack [n_in, rows, width] dense float32; w0..w3 the branches' weights [width]
extern "C" int lq_rmsnorm_mean(const float* stack, int n_in, const float* w0, const float* w1, const float* w2,
                               const float* w3, float eps, float* out, int rows, int width, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && width > 0 && n_in >= 1 && n_in <= 4, "rmsnorm_mean: %d branches of %d x %d", n_in, rows, width);
  const float* ws[4] = {w0, w1, w2, w3};
  MeanInputs in;
  for (int i = 0; i < 4; ++i) {
    in.x[i] = i < n_in ? stack + (long long)i * rows * width : nullptr;
    in.w[i] = ws[i];
    LQ_REQUIRE(i >= n_in || ws[i] != nullptr, "rmsnorm_mean: branch %d has no weight", i);
  }
  LQ_REQUIRE(stack && out, "rmsnorm_mean: null pointer");
  rmsnorm_mean_kernel<<<rows, width >= 1024 ? 256 : 64, 0, stream>>>(in, n_in, eps, out, width);
  LQ_CHECK_LAUNCH("rmsnorm_mean");
  return 0;
}

// Kernels of a mixture of experts whose experts' matrices lie side by side: the router's choice and the experts'
// activation.  Router scores and weights are 32-bit.
#include "common.h"

namespace {

// One thread a row: s = sigmoid(z), the `top` largest win (the lower index on a tie); route[r, e] = the expert's
// weight (its score, or its share of the chosen scores), -1 for an expert that was not chosen.
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ z, int ldz, float* __restrict__ route,
                                                       int rows, int E, int top, int renorm) {
  const int r = blockIdx.x * 64 + threadIdx.x;
  if (r >= rows) return;
  const float* zr = z + (long long)r * ldz;
  float* out = route + (long long)r * E;
  for (int e = 0; e < E; ++e) out[e] = -1.f;
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bz = 0.f;
    for (int e = 0; e < E; ++e) {
      if (out[e] >= 0.f) continue;  // chosen already
      const float v = 1.f / (1.f + expf(-zr[e]));  // scores are compared, not logits: equal scores are a tie
      if (best < 0 || v > bz) best = e, bz = v;
    }
    if (best < 0) break;
    out[best] = bz == bz ? bz : 0.f;
    total += out[best];
  }
  if (renorm && total > 0.f)
    for (int e = 0; e < E; ++e)
      if (out[e] >= 0.f) out[e] /= total;
}

// gu [rows, E, 2, ff] (gate then up of every expert), route [rows, E]; out [rows, E, ff]:
// g = min(w gate, limit), u = clamp(w up, -limit, limit), y = g sigmoid(1.702 g) (u + 1) for a chosen expert (its
// weight w on what it read: `on_input`; otherwise w multiplies y), 0 for the others.
template <typename T>
__global__ __launch_bounds__(256) void moe_glu_kernel(const float* __restrict__ gu, long long ldg,
                                                      const float* __restrict__ route, T* __restrict__ out,
                                                      long long ldo, int E, int ff, float limit, int on_input) {
  const int r = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= E * ff) return;
  const int e = i / ff, c = i - e * ff;
  const float w = route[(long long)r * E + e];
  float y = 0.f;
  if (w >= 0.f) {
    const float* p = gu + r * ldg + (long long)e * 2 * ff;
    const float s = on_input ? w : 1.f;
    const float g = fminf(p[c] * s, limit);
    const float u = fminf(fmaxf(p[ff + c] * s, -limit), limit);
    y = g / (1.f + expf(-1.702f * g)) * (u + 1.f);
    if (!on_input) y *= w;
  }
  out[r * ldo + i] = from_f32<T>(y);
}

}  // namespace

extern "C" int lq_moe_route(const float* z, int ldz, float* route, int rows, int experts, int top, int renormalize,
                            hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && experts > 0 && top >= 1 && top <= experts && ldz >= experts, "moe_route: rows %d, %d of %d experts",
             rows, top, experts);
  LQ_REQUIRE(z && route, "moe_route: null pointer");
  moe_route_kernel<<<lq_ceil_div(rows, 64), 64, 0, stream>>>(z, ldz, route, rows, experts, top, renormalize);
  LQ_CHECK_LAUNCH("moe_route");
  return 0;
}

extern "C" int lq_moe_glu(const float* gu, long long ldg, const float* route, void* out, int out_dtype, long long ldo,
                          int rows, int experts, int ff, float limit, int on_input, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && experts > 0 && ff > 0 && (long long)experts * ff <= 0x7fffffff, "moe_glu: rows %d, experts %d, inner %d",
             rows, experts, ff);
  LQ_REQUIRE(ldg >= 2ll * experts * ff && ldo >= (long long)experts * ff, "moe_glu: a row stride is smaller than its row");
  LQ_REQUIRE(gu && route && out, "moe_glu: null pointer");
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    dim3 grid(lq_ceil_div(experts * ff, 256), nr);
    if (out_dtype == LQ_F32)
      moe_glu_kernel<float><<<grid, 256, 0, stream>>>(gu + r0 * ldg, ldg, route + (long long)r0 * experts,
                                                      (float*)out + r0 * ldo, ldo, experts, ff, limit, on_input);
    else if (out_dtype == LQ_BF16)
      moe_glu_kernel<bf16_t><<<grid, 256, 0, stream>>>(gu + r0 * ldg, ldg, route + (long long)r0 * experts,
                                                       (bf16_t*)out + r0 * ldo, ldo, experts, ff, limit, on_input);
    else LQ_REQUIRE(false, "moe_glu: unknown dtype %d", out_dtype);
  }
  LQ_CHECK_LAUNCH("moe_glu");
  return 0;
}

// Kernels of a mixture of experts whose experts' matrices lie side by side: the router's choice and the experts'
// activation.  Router scores and weights are 32-bit.
#include "common.h"

namespace {

// One thread a row: s = sigmoid(z), the `top` largest win (the lower index on a tie); route[r, e] = the expert's
// weight (its score, or its share of the chosen scores), -1 for an expert that was not chosen.
// With `correction` the experts are chosen by s + correction[e]; the weights stay the scores s.  With `groups` > 1
// the experts form that many equal groups of neighbours; a group's mark is the sum of its two largest choice scores
// (of its one, in groups of one), and only experts of the `keep` groups with the largest marks (the lower index on a
// tie) can be chosen.  `softmax`: s = softmax(z) over all E outputs in the sigmoid's place.  `mark_max`: a group's mark
// is its largest choice score alone.  `renorm_eps` is added to the chosen scores' sum before the division.  The last
// `n_ident` of the E outputs are experts without tensors: their weights go to `ident` [rows, n_ident] (-1: not
// chosen) and `route` has the E - n_ident others.
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ z, int ldz, float* __restrict__ route,
                                                       int rows, int E, int top, int renorm,
                                                       const float* __restrict__ correction, int groups, int keep,
                                                       int softmax, int mark_max, float renorm_eps,
                                                       float* __restrict__ ident, int n_ident) {
  const int r = blockIdx.x * 64 + threadIdx.x;
  if (r >= rows) return;
  const float* zr = z + (long long)r * ldz;
  const int R = E - n_ident;  // experts with tensors
  float* out_real = route + (long long)r * R;
  float* out_ident = n_ident > 0 ? ident + (long long)r * n_ident : nullptr;
  auto out = [&](int e) -> float& { return e < R ? out_real[e] : out_ident[e - R]; };
  for (int e = 0; e < E; ++e) out(e) = -1.f;
  float zmax = -INFINITY, inv_sum = 1.f;
  if (softmax) {
    for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, zr[e]);
    float sum = 0.f;
    for (int e = 0; e < E; ++e) sum += expf(zr[e] - zmax);
    inv_sum = 1.f / sum;
  }
  auto score = [&](int e) { return softmax ? expf(zr[e] - zmax) * inv_sum : 1.f / (1.f + expf(-zr[e])); };
  auto choice = [&](int e) { return correction != nullptr ? score(e) + correction[e] : score(e); };
  unsigned long long kept = ~0ull;  // bit g: group g may be chosen from
  const int per = groups > 1 ? E / groups : E;
  if (groups > 1 && keep < groups) {
    kept = 0ull;
    for (int n = 0; n < keep; ++n) {
      int best = -1;
      float bm = 0.f;
      for (int g = 0; g < groups; ++g) {
        if ((kept >> g) & 1ull) continue;
        float a = -INFINITY, b = -INFINITY;  // the group's two largest choice scores
        for (int e = g * per; e < (g + 1) * per; ++e) {
          const float v = choice(e);
          if (v > a) b = a, a = v;
          else if (v > b) b = v;
        }
        const float mark = per > 1 && !mark_max ? a + b : a;
        if (best < 0 || mark > bm) best = g, bm = mark;
      }
      if (best < 0) break;
      kept |= 1ull << best;
    }
  }
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bz = 0.f;
    for (int e = 0; e < E; ++e) {
      if (out(e) >= 0.f) continue;  // chosen already
      if (groups > 1 && !((kept >> (e / per)) & 1ull)) continue;
      const float v = choice(e);  // scores are compared, not logits: equal scores are a tie
      if (best < 0 || v > bz) best = e, bz = v;
    }
    if (best < 0) break;
    const float w = score(best);
    out(best) = w == w ? w : 0.f;
    total += out(best);
  }
  total += renorm_eps;
  if (renorm && total > 0.f)
    for (int e = 0; e < E; ++e)
      if (out(e) >= 0.f) out(e) /= total;
}

// out[r, :] += h[r, :] * (the sum of the row's chosen identity experts' weights); weights [rows, n] (-1: not chosen)
template <typename T>
__global__ __launch_bounds__(256) void moe_identity_kernel(const T* __restrict__ h, int ldh,
                                                           const float* __restrict__ weights, int n,
                                                           float* __restrict__ out, int ldo, int width) {
  const int r = blockIdx.x;
  float w = 0.f;
  for (int i = 0; i < n; ++i) {
    const float v = weights[(long long)r * n + i];
    if (v >= 0.f) w += v;
  }
  if (w == 0.f) return;
  for (int c = threadIdx.x; c < width; c += 256) out[(long long)r * ldo + c] += w * to_f32(h[(long long)r * ldh + c]);
}

// gu [rows, E, 2, ff] (gate then up of every expert), route [rows, E]; out [rows, E, ff]:
// g = min(w gate, limit), u = clamp(w up, -limit, limit), y = g sigmoid(1.702 g) (u + 1) for a chosen expert (its
// weight w on what it read: `on_input`; otherwise w multiplies y), 0 for the others.  `plain_silu`: the expert is
// y = silu(gate) up without clamps.
template <typename T>
__global__ __launch_bounds__(256) void moe_glu_kernel(const float* __restrict__ gu, long long ldg,
                                                      const float* __restrict__ route, T* __restrict__ out,
                                                      long long ldo, int E, int ff, float limit, int on_input,
                                                      int plain_silu) {
  const int r = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= E * ff) return;
  const int e = i / ff, c = i - e * ff;
  const float w = route[(long long)r * E + e];
  float y = 0.f;
  if (w >= 0.f) {
    const float* p = gu + r * ldg + (long long)e * 2 * ff;
    const float s = on_input ? w : 1.f;
    if (plain_silu) {
      const float g = p[c] * s;
      y = g / (1.f + expf(-g)) * (p[ff + c] * s);
    } else {
      const float g = fminf(p[c] * s, limit);
      const float u = fminf(fmaxf(p[ff + c] * s, -limit), limit);
      y = g / (1.f + expf(-1.702f * g)) * (u + 1.f);
    }
    if (!on_input) y *= w;
  }
  out[r * ldo + i] = from_f32<T>(y);
}

// ---- a step's rows sorted by expert ----------------------------------------------------------------------------------
// counts[e] = rows that chose expert e; one workgroup an expert.
__global__ __launch_bounds__(256) void moe_count_kernel(const float* __restrict__ route, int rows, int E,
                                                        int* __restrict__ counts) {
  __shared__ float red[16];
  const int e = blockIdx.x;
  float n = 0.f;  // (counts of up to 2^24 rows are whole numbers in 32-bit floats)
  for (int r = threadIdx.x; r < rows; r += 256) n += route[(long long)r * E + e] >= 0.f ? 1.f : 0.f;
  n = block_sum(n, red);
  if (threadIdx.x == 0) counts[e] = (int)n;
}

// Expert e's rows, in ascending order, take the places offset(e) .. offset(e) + counts[e] - 1 of the sorted list
// (offset: the counts of the experts before it): order[place] = row, weight[place] = the row's weight for the expert,
// place_of[row, e] = place (-1 for an expert the row did not choose).  One workgroup an expert walks the rows in
// chunks of 256 with a running count, so the order does not depend on timing.
__global__ __launch_bounds__(256) void moe_place_kernel(const float* __restrict__ route, int rows, int E,
                                                        const int* __restrict__ counts, int* __restrict__ order,
                                                        float* __restrict__ weight, int* __restrict__ place_of) {
  __shared__ int wave_n[4];
  __shared__ int base;
  const int e = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) {
    int off = 0;
    for (int i = 0; i < e; ++i) off += counts[i];
    base = off;
  }
  __syncthreads();
  for (int r0 = 0; r0 < rows; r0 += 256) {
    const int r = r0 + threadIdx.x;
    const float w = r < rows ? route[(long long)r * E + e] : -1.f;
    const bool chosen = w >= 0.f;
    const unsigned long long mask = __ballot(chosen);
    const int before = __popcll(mask & ((1ull << lane) - 1ull));
    if (lane == 0) wave_n[wave] = __popcll(mask);
    __syncthreads();
    int at = base + before;
    for (int i = 0; i < wave; ++i) at += wave_n[i];
    if (chosen) order[at] = r, weight[at] = w;
    if (r < rows) place_of[(long long)r * E + e] = chosen ? at : -1;
    __syncthreads();
    if (threadIdx.x == 0) base += wave_n[0] + wave_n[1] + wave_n[2] + wave_n[3];
    __syncthreads();
  }
}

// dst[i, :] = src[order[i], :] (16-bit or 32-bit rows)
template <typename T>
__global__ __launch_bounds__(256) void moe_gather_kernel(const T* __restrict__ src, int lds_, const int* __restrict__ order,
                                                         T* __restrict__ dst, int width) {
  const T* s = src + (long long)order[blockIdx.x] * lds_;
  T* d = dst + (long long)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += 256) d[i] = s[i];
}

// out[r, :] = the sum, over the experts that row r chose in ascending order, of ys[place_of[r, e], :]
__global__ __launch_bounds__(256) void moe_scatter_kernel(const float* __restrict__ ys, const int* __restrict__ place_of, int E,
                                                          float* __restrict__ out, int ldo, int width) {
  const int r = blockIdx.x;
  const int* places = place_of + (long long)r * E;
  for (int i = threadIdx.x; i < width; i += 256) {
    float acc = 0.f;
    for (int e = 0; e < E; ++e) {
      const int at = places[e];
      if (at >= 0) acc += ys[(long long)at * width + i];
    }
    out[(long long)r * ldo + i] = acc;
  }
}

}  // namespace

// `experts` counts every output of the router, the `n_ident` identity experts at its end included: route is
// [rows, experts - n_ident], ident [rows, n_ident] (null without identity experts).
extern "C" int lq_moe_route(const float* z, int ldz, float* route, int rows, int experts, int top, int renormalize,
                            const float* correction, int groups, int keep, int softmax, int mark_max, float renorm_eps,
                            float* ident, int n_ident, hipStream_t stream) {
  LQ_REQUIRE(groups >= 0 && (groups <= 1 || (groups <= 64 && experts % groups == 0 && keep >= 1 && keep <= groups)),
             "moe_route: %d experts in %d groups of which %d are kept", experts, groups, keep);
  LQ_REQUIRE(rows > 0 && experts > 0 && top >= 1 && top <= experts && ldz >= experts, "moe_route: rows %d, %d of %d experts",
             rows, top, experts);
  LQ_REQUIRE(n_ident >= 0 && n_ident < experts && (n_ident == 0 || ident != nullptr) && renorm_eps >= 0.f,
             "moe_route: %d identity experts of %d", n_ident, experts);
  LQ_REQUIRE(z && route, "moe_route: null pointer");
  moe_route_kernel<<<lq_ceil_div(rows, 64), 64, 0, stream>>>(z, ldz, route, rows, experts, top, renormalize, correction,
                                                             groups, keep, softmax, mark_max, renorm_eps, ident, n_ident);
  LQ_CHECK_LAUNCH("moe_route");
  return 0;
}

extern "C" int lq_moe_identity(const void* h, int dtype, int ldh, const float* weights, int n, float* out, int ldo, int rows,
                               int width, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && width > 0 && n > 0 && ldh >= width && ldo >= width, "moe_identity: rows %d, width %d, %d experts", rows,
             width, n);
  LQ_REQUIRE(h && weights && out, "moe_identity: null pointer");
  if (dtype == LQ_F32)
    moe_identity_kernel<float><<<rows, 256, 0, stream>>>((const float*)h, ldh, weights, n, out, ldo, width);
  else if (dtype == LQ_BF16)
    moe_identity_kernel<bf16_t><<<rows, 256, 0, stream>>>((const bf16_t*)h, ldh, weights, n, out, ldo, width);
  else LQ_REQUIRE(false, "moe_identity: unknown dtype %d", dtype);
  LQ_CHECK_LAUNCH("moe_identity");
  return 0;
}

extern "C" int lq_moe_glu(const float* gu, long long ldg, const float* route, void* out, int out_dtype, long long ldo,
                          int rows, int experts, int ff, float limit, int on_input, int plain_silu, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && experts > 0 && ff > 0 && (long long)experts * ff <= 0x7fffffff, "moe_glu: rows %d, experts %d, inner %d",
             rows, experts, ff);
  LQ_REQUIRE(ldg >= 2ll * experts * ff && ldo >= (long long)experts * ff, "moe_glu: a row stride is smaller than its row");
  LQ_REQUIRE(gu && route && out, "moe_glu: null pointer");
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    dim3 grid(lq_ceil_div(experts * ff, 256), nr);
    if (out_dtype == LQ_F32)
      moe_glu_kernel<float><<<grid, 256, 0, stream>>>(gu + r0 * ldg, ldg, route + (long long)r0 * experts,
                                                      (float*)out + r0 * ldo, ldo, experts, ff, limit, on_input, plain_silu);
    else if (out_dtype == LQ_BF16)
      moe_glu_kernel<bf16_t><<<grid, 256, 0, stream>>>(gu + r0 * ldg, ldg, route + (long long)r0 * experts,
                                                       (bf16_t*)out + r0 * ldo, ldo, experts, ff, limit, on_input, plain_silu);
    else LQ_REQUIRE(false, "moe_glu: unknown dtype %d", out_dtype);
  }
  LQ_CHECK_LAUNCH("moe_glu");
  return 0;
}

// route [rows, experts] (a weight, or -1): counts [experts], order and weight [pairs] (pairs: the chosen
// (row, expert) couples, expert by expert, rows ascending), place_of [rows, experts]
extern "C" int lq_moe_sort(const float* route, int rows, int experts, int* counts, int* order, float* weight, int* place_of,
                           hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && rows < (1 << 24) && experts > 0 && experts <= 65535, "moe_sort: rows %d, experts %d", rows, experts);
  LQ_REQUIRE(route && counts && order && weight && place_of, "moe_sort: null pointer");
  moe_count_kernel<<<experts, 256, 0, stream>>>(route, rows, experts, counts);
  LQ_CHECK_LAUNCH("moe_sort(count)");
  moe_place_kernel<<<experts, 256, 0, stream>>>(route, rows, experts, counts, order, weight, place_of);
  LQ_CHECK_LAUNCH("moe_sort(place)");
  return 0;
}

extern "C" int lq_moe_gather(const void* src, int dtype, int ld, const int* order, void* dst, int n, int width,
                             hipStream_t stream) {
  LQ_REQUIRE(n > 0 && width > 0 && ld >= width, "moe_gather: %d rows of %d (stride %d)", n, width, ld);
  LQ_REQUIRE(src && order && dst, "moe_gather: null pointer");
  if (dtype == LQ_F32) moe_gather_kernel<float><<<n, 256, 0, stream>>>((const float*)src, ld, order, (float*)dst, width);
  else if (dtype == LQ_BF16) moe_gather_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)src, ld, order, (bf16_t*)dst, width);
  else LQ_REQUIRE(false, "moe_gather: unknown dtype %d", dtype);
  LQ_CHECK_LAUNCH("moe_gather");
  return 0;
}

extern "C" int lq_moe_scatter(const float* ys, const int* place_of, int experts, float* out, int ldo, int rows, int width,
                              hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && width > 0 && experts > 0 && ldo >= width, "moe_scatter: rows %d, width %d, experts %d", rows, width, experts);
  LQ_REQUIRE(ys && place_of && out, "moe_scatter: null pointer");
  moe_scatter_kernel<<<rows, 256, 0, stream>>>(ys, place_of, experts, out, ldo, width);
  LQ_CHECK_LAUNCH("moe_scatter");
  return 0;
}

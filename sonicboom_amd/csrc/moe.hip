// Routed experts: the choice, and the experts' products over the rows that chose them.
//
//   sb_moe_route    from router scores z f32 [rows, stride]: the `top` largest of the first
//                   n_experts (ties to the lower number), in falling order, and their weights, the
//                   softmax over the chosen scores alone; with has_gate also sigmoid(z[n_experts]),
//                   the multiplier of an expert that every row takes.
//                   ids int32 [rows, top]; weights f32 [rows, top + 1] (the last: the gate, or 0).
//   sb_moe_product  Y[p,:] = X[p / x_div,:] W_e^T for every pair p = (row, choice), e = ids[p]
//                   (ids NULL: expert 0 for all); gated: W_e = [W_gate; W_up] and
//                   Y = g' sigmoid(alpha g') (u' + 1), g' = min(g, limit), u' = u cut to +-limit.
//                   The plain form: a thread an output, sums in ascending k, so a pair's bits depend
//                   on its row and expert alone.  Any sizes; f32 or bf16 operands.
#include "common.h"

namespace {

constexpr int kMaxTop = 16;

__global__ void __launch_bounds__(64)
moe_route_kernel(int32_t *__restrict__ ids, float *__restrict__ weights, const float *__restrict__ z, int n_rows,
                 int stride, int n_experts, int top, int has_gate) {
  const int r = blockIdx.x * 64 + threadIdx.x;
  if (r >= n_rows) return;
  const float *zr = z + size_t(r) * stride;
  int chosen[kMaxTop];
  float score[kMaxTop];
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bz = 0.0f;
    for (int e = 0; e < n_experts; ++e) {
      const float v = zr[e];
      // candidates: below the last choice, or equal to it with a higher number (the order is
      // falling scores, rising numbers among equals); NaN scores are never chosen
      if (k > 0 && !(v < score[k - 1] || (v == score[k - 1] && e > chosen[k - 1]))) continue;
      if (best < 0 || v > bz) { best = e; bz = v; }
    }
    if (best < 0) { best = 0; bz = -__builtin_inff(); }
    chosen[k] = best;
    score[k] = bz;
  }
  float sum = 0.0f, w[kMaxTop];
  for (int k = 0; k < top; ++k) { w[k] = expf(score[k] - score[0]); sum += w[k]; }
  for (int k = 0; k < top; ++k) {
    ids[size_t(r) * top + k] = chosen[k];
    weights[size_t(r) * (top + 1) + k] = w[k] / sum;
  }
  weights[size_t(r) * (top + 1) + top] = has_gate ? 1.0f / (1.0f + expf(-zr[n_experts])) : 0.0f;
}

template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(256)
moe_product_plain_kernel(TY *__restrict__ y, const TX *__restrict__ x, const TW *__restrict__ w,
                         const int32_t *__restrict__ ids, int x_div, int n_out, int n_in, int n_experts, int gated,
                         float limit, float alpha) {
  extern __shared__ float xs[];
  const int p = blockIdx.x;
  const int e = ids ? ids[p] : 0;
  const TX *xr = x + size_t(p / x_div) * n_in;
  for (int k = threadIdx.x; k < n_in; k += 256) xs[k] = ld_f(xr, k);
  __syncthreads();
  if (e < 0 || e >= n_experts) return;
  const int o = blockIdx.y * 256 + threadIdx.x;
  if (o >= n_out) return;
  const size_t w_rows = size_t(gated ? 2 : 1) * n_out;
  const TW *wg = w + (size_t(e) * w_rows + o) * n_in;
  float g = 0.0f;
  for (int k = 0; k < n_in; ++k) g = fmaf(xs[k], ld_f(wg, k), g);
  if (gated) {
    const TW *wu = wg + size_t(n_out) * n_in;
    float u = 0.0f;
    for (int k = 0; k < n_in; ++k) u = fmaf(xs[k], ld_f(wu, k), u);
    g = swish_clamp_mul(g, u, limit, alpha);
  }
  st_f(y, size_t(p) * n_out + o, g);
}

}  // namespace

extern "C" int sb_moe_max_top(void) { return kMaxTop; }

extern "C" int sb_moe_route(int32_t *ids, float *weights, const float *z, int n_rows, int stride, int n_experts,
                            int top, int has_gate, void *stream) {
  SB_REQUIRE(ids && weights && z, "sb_moe_route: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_experts > 0 && top > 0 && top <= n_experts && stride >= n_experts + (has_gate ? 1 : 0),
             "sb_moe_route: bad sizes rows=%d experts=%d top=%d stride=%d", n_rows, n_experts, top, stride);
  SB_SUPPORT(top <= kMaxTop, "sb_moe_route: %d choices a row are more than %d", top, kMaxTop);
  if (n_rows == 0) return SB_OK;
  moe_route_kernel<<<(n_rows + 63) / 64, 64, 0, (hipStream_t)stream>>>(ids, weights, z, n_rows, stride, n_experts, top, has_gate);
  return sb::check_launch("sb_moe_route");
}

extern "C" int sb_moe_product(void *y, int y_dtype, const void *x, int x_dtype, const void *w, int w_dtype,
                              const int32_t *ids, int n_pairs, int x_div, int n_out, int n_in, int n_experts,
                              int gated, float limit, float alpha, void *stream) {
  SB_REQUIRE(y && x && w, "sb_moe_product: null pointer");
  SB_REQUIRE(n_pairs >= 0 && x_div > 0 && n_out > 0 && n_in > 0 && n_experts > 0,
             "sb_moe_product: bad sizes pairs=%d out=%d in=%d experts=%d", n_pairs, n_out, n_in, n_experts);
  SB_REQUIRE(sb::valid_dtype(y_dtype) && sb::valid_dtype(x_dtype) && sb::valid_dtype(w_dtype), "sb_moe_product: unknown dtype");
  SB_SUPPORT(n_in <= 16384, "sb_moe_product: rows of %d are longer than 16384", n_in);
  if (n_pairs == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(n_pairs, (n_out + 255) / 256);
  const size_t lds = size_t(n_in) * sizeof(float);
#define SB_GO(TX, TW, TY)                                                                                   \
  moe_product_plain_kernel<TX, TW, TY><<<grid, 256, lds, s>>>((TY *)y, (const TX *)x, (const TW *)w, ids, x_div, \
                                                                n_out, n_in, n_experts, gated, limit, alpha)
  const int which = (x_dtype == SB_BF16 ? 4 : 0) + (w_dtype == SB_BF16 ? 2 : 0) + (y_dtype == SB_BF16 ? 1 : 0);
  switch (which) {
    case 0: SB_GO(float, float, float); break;
    case 1: SB_GO(float, float, bf16_t); break;
    case 2: SB_GO(float, bf16_t, float); break;
    case 3: SB_GO(float, bf16_t, bf16_t); break;
    case 4: SB_GO(bf16_t, float, float); break;
    case 5: SB_GO(bf16_t, float, bf16_t); break;
    case 6: SB_GO(bf16_t, bf16_t, float); break;
    default: SB_GO(bf16_t, bf16_t, bf16_t); break;
  }
#undef SB_GO
  return sb::check_launch("sb_moe_product");
}

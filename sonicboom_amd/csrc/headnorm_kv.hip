// Queries and keys normed per head, values mixed with an earlier layer's, keys and values stored.
//
// From the float32 rows of a stacked product [q: heads_q x dk | k: heads_kv x dk | v: heads_kv x dv]
// (whole, or in K slices that are added here in ascending order):
//   every head of q and k is divided by its root mean square (eps inside the root) and multiplied by
//   a weight of the head's size that the heads share (NULL: the head passes as it is);
//   v <- (1 - lam) v + lam v_first when v_first is given (lam one number in memory), and the v of
//   before the mixing is written to v_out when that is given (the first mixing layer's);
//   q goes out in the activation type, k and v into the page of the row's position.
// One block a row; a wave a head at a time.
#include "common.h"

namespace {

constexpr int kMaxHead = 256;

struct Args {
  void *q_out;
  const float *qkv; int row_stride, n_slices; size_t slice_stride;
  const void *q_w, *k_w; int w_dtype; float eps;
  const float *v_first; const void *lam; int lam_dtype; float *v_out;
  const int32_t *row_pos, *row_seq, *page_table; int max_pages, n_pages;
  void *k_cache, *v_cache;
  int heads_q, heads_kv, dk, dv, store;
};

constexpr int kMaxSlices = 8;      // slices whose loads the unrolled loops ask for together (more: the plain loop)

// the sum over the slices of one number of a row: all loads asked for before any is added
__device__ __forceinline__ float sum_slices(const float *p, int n_slices, size_t slice_stride) {
  if (n_slices == 1) return p[0];
  if (n_slices <= kMaxSlices) {
    float in[kMaxSlices];
#pragma unroll
    for (int s = 0; s < kMaxSlices; ++s) in[s] = p[size_t(min(s, n_slices - 1)) * slice_stride];
    float v = 0.0f;
#pragma unroll
    for (int s = 0; s < kMaxSlices; ++s)
      if (s < n_slices) v += in[s];
    return v;
  }
  float v = 0.0f;
  for (int s = 0; s < n_slices; ++s) v += p[s * slice_stride];
  return v;
}

template <typename TQ, typename TC, int THREADS>
__global__ void __launch_bounds__(THREADS) headnorm_kv_store_kernel(Args a) {
  const int row = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float *src = a.qkv + size_t(row) * a.row_stride;
  int page = -1, slot = 0;
  if (a.store) {
    const int pos = a.row_pos[row], c = pos / SB_PAGE;
    slot = pos % SB_PAGE;
    if (c < a.max_pages) page = a.page_table[size_t(a.row_seq[row]) * a.max_pages + c];
    if (page >= a.n_pages) page = -1;
  }
  const int units = a.heads_q + (a.store ? a.heads_kv : 0);
  for (int u = wave; u < units; u += THREADS / 64) {
    const int col = u * a.dk;
    float v[kMaxHead / 64];
    double sq = 0.0;
#pragma unroll
    for (int i = 0; i < kMaxHead / 64; ++i) {
      const int d = lane + 64 * i;
      v[i] = 0.0f;
      if (d < a.dk) {
        v[i] = sum_slices(src + col + d, a.n_slices, a.slice_stride);
        sq += double(v[i] * v[i]);
      }
    }
    const bool is_q = u < a.heads_q;
    const void *w = is_q ? a.q_w : a.k_w;
    float inv = 1.0f;
    if (w) inv = 1.0f / sqrtf(float(wave_sum(sq) / double(a.dk)) + a.eps);
#pragma unroll
    for (int i = 0; i < kMaxHead / 64; ++i) {
      const int d = lane + 64 * i;
      if (d >= a.dk) continue;
      const float o = w ? (v[i] * inv) * ld_dyn(w, a.w_dtype, d) : v[i];
      if (is_q) st_f((TQ *)a.q_out, size_t(row) * a.heads_q * a.dk + col + d, o);
      else if (page >= 0)
        st_f((TC *)a.k_cache, (size_t(page) * a.heads_kv + (u - a.heads_q)) * SB_PAGE * a.dk + sb_key_index(slot, d, a.dk), o);
    }
  }
  if (!a.store) return;
  const int v0 = (a.heads_q + a.heads_kv) * a.dk, nv = a.heads_kv * a.dv;
  const float lam = a.v_first ? ld_dyn(a.lam, a.lam_dtype, 0) : 0.0f;
  for (int e = threadIdx.x; e < nv; e += THREADS) {
    float v = sum_slices(src + v0 + e, a.n_slices, a.slice_stride);
    if (a.v_out) a.v_out[size_t(row) * nv + e] = v;
    if (a.v_first) v = (1.0f - lam) * v + lam * a.v_first[size_t(row) * nv + e];
    if (page >= 0)
      st_f((TC *)a.v_cache, (size_t(page) * a.heads_kv + e / a.dv) * a.dv * SB_PAGE + sb_value_index(e % a.dv, slot), v);
  }
}

// The same for long steps of bfloat16 queries and cache, one slice, head sizes in eights: eight lanes
// a head (more for heads above 64 numbers), eight numbers a lane in two 16-byte loads and one 16-byte store;
// sums of squares in double by a butterfly over the head's lanes.  The arithmetic of every number is
// that of the form above.
template <int LANES>      // lanes a head: 8, 16 or 32 (heads of up to 64, 128, 256 numbers)
__global__ void __launch_bounds__(256) headnorm_kv_store_wide_kernel(Args a) {
  constexpr int HEADS_PER_BLOCK = 256 / LANES;
  const int row = blockIdx.x, tid = threadIdx.x, sub = tid % LANES, slot_in_block = tid / LANES;
  const float *src = a.qkv + size_t(row) * a.row_stride;
  int page = -1, slot = 0;
  if (a.store) {
    const int pos = a.row_pos[row], c = pos / SB_PAGE;
    slot = pos % SB_PAGE;
    if (c < a.max_pages) page = a.page_table[size_t(a.row_seq[row]) * a.max_pages + c];
    if (page >= a.n_pages) page = -1;
  }
  const int units = a.heads_q + (a.store ? a.heads_kv : 0);
  for (int u0 = 0; u0 < units; u0 += HEADS_PER_BLOCK) {       // every lane walks the loop: the butterflies need them all
    const int u = u0 + slot_in_block, d = 8 * sub;
    const bool live = u < units && d < a.dk;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (live) {
      const float4 lo = *reinterpret_cast<const float4 *>(src + u * a.dk + d), hi = *reinterpret_cast<const float4 *>(src + u * a.dk + d + 4);
      v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    }
    double sq = 0.0;
#pragma unroll
    for (int i = 0; i < 8; ++i) sq += double(v[i] * v[i]);
#pragma unroll
    for (int off = LANES / 2; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
    if (!live) continue;
    const bool is_q = u < a.heads_q;
    const void *w = is_q ? a.q_w : a.k_w;
    const float inv = w ? 1.0f / sqrtf(float(sq / double(a.dk)) + a.eps) : 1.0f;
    uint32_t packed[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float o0 = w ? (v[2 * i] * inv) * ld_dyn(w, a.w_dtype, d + 2 * i) : v[2 * i];
      const float o1 = w ? (v[2 * i + 1] * inv) * ld_dyn(w, a.w_dtype, d + 2 * i + 1) : v[2 * i + 1];
      packed[i] = uint32_t(f32_to_bf16(o0)) | uint32_t(f32_to_bf16(o1)) << 16;
    }
    const uint4 out = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    if (is_q) *reinterpret_cast<uint4 *>((bf16_t *)a.q_out + size_t(row) * a.heads_q * a.dk + u * a.dk + d) = out;
    else if (page >= 0)       // eight neighbouring numbers of a key stay neighbours in the cache's order
      *reinterpret_cast<uint4 *>((bf16_t *)a.k_cache + (size_t(page) * a.heads_kv + (u - a.heads_q)) * SB_PAGE * a.dk +
                                 sb_key_index(slot, d, a.dk)) = out;
  }
  if (!a.store) return;
  const int v0 = (a.heads_q + a.heads_kv) * a.dk, nv = a.heads_kv * a.dv;
  const float lam = a.v_first ? ld_dyn(a.lam, a.lam_dtype, 0) : 0.0f;
  for (int e = tid; e < nv; e += 256) {
    float v = src[v0 + e];
    if (a.v_out) a.v_out[size_t(row) * nv + e] = v;
    if (a.v_first) v = (1.0f - lam) * v + lam * a.v_first[size_t(row) * nv + e];
    if (page >= 0)
      st_f((bf16_t *)a.v_cache, (size_t(page) * a.heads_kv + e / a.dv) * a.dv * SB_PAGE + sb_value_index(e % a.dv, slot), v);
  }
}

}  // namespace

extern "C" int sb_headnorm_kv_store(void *q_out, int q_dtype, const float *qkv, int row_stride, int n_slices,
                                    const void *q_w, const void *k_w, int w_dtype, float eps, const float *v_first,
                                    const void *lam, int lam_dtype, float *v_out, const int32_t *row_pos,
                                    const int32_t *row_seq, void *k_cache, void *v_cache, int cache_dtype,
                                    const int32_t *page_table, int max_pages, int n_pages, int n_rows, int heads_q,
                                    int heads_kv, int dk, int dv, int store, void *stream) {
  SB_REQUIRE(q_out && qkv, "sb_headnorm_kv_store: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads_q > 0 && heads_kv >= 0 && dk > 0 && dv > 0 && n_slices > 0,
             "sb_headnorm_kv_store: bad sizes rows=%d heads=%d/%d dk=%d dv=%d", n_rows, heads_q, heads_kv, dk, dv);
  SB_REQUIRE(!store || (row_pos && row_seq && k_cache && v_cache && page_table && max_pages > 0 && n_pages > 0 && heads_kv > 0),
             "sb_headnorm_kv_store: storing needs positions, page table and cache");
  SB_REQUIRE(row_stride >= heads_q * dk + (store ? heads_kv * (dk + dv) : 0), "sb_headnorm_kv_store: rows of %d are too short", row_stride);
  SB_REQUIRE(!v_first || lam, "sb_headnorm_kv_store: mixing needs its number");
  SB_REQUIRE(sb::valid_dtype(q_dtype) && (!store || sb::valid_dtype(cache_dtype)) && ((!q_w && !k_w) || sb::valid_dtype(w_dtype)) &&
                 (!lam || sb::valid_dtype(lam_dtype)), "sb_headnorm_kv_store: unknown dtype");
  SB_SUPPORT(dk <= kMaxHead, "sb_headnorm_kv_store: head size %d is above the limit of %d", dk, kMaxHead);
  if (n_rows == 0) return SB_OK;
  const Args a{q_out, qkv, row_stride, n_slices, size_t(n_rows) * row_stride, q_w, k_w, w_dtype, eps, v_first, lam, lam_dtype, v_out,
               row_pos, row_seq, page_table, max_pages, n_pages, k_cache, v_cache, heads_q, heads_kv, dk, dv, store ? 1 : 0};
  hipStream_t s = (hipStream_t)stream;
  const bool qf = q_dtype == SB_F32, cf = !store || cache_dtype == SB_F32;
  // (a wave a head: the sums do not depend on the block's size, so few rows may take more waves a row)
  if (qf && cf) headnorm_kv_store_kernel<float, float, 256><<<n_rows, 256, 0, s>>>(a);
  else if (qf) headnorm_kv_store_kernel<float, bf16_t, 256><<<n_rows, 256, 0, s>>>(a);
  else if (cf && store) headnorm_kv_store_kernel<bf16_t, float, 256><<<n_rows, 256, 0, s>>>(a);
  else if (n_rows <= 64) headnorm_kv_store_kernel<bf16_t, bf16_t, 1024><<<n_rows, 1024, 0, s>>>(a);
  else if (n_rows >= 512 && n_slices == 1 && dk % 8 == 0 && row_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(qkv) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(q_out) & 15) == 0 && (!store || (reinterpret_cast<uintptr_t>(k_cache) & 15) == 0)) {
    if (dk <= 64) headnorm_kv_store_wide_kernel<8><<<n_rows, 256, 0, s>>>(a);
    else if (dk <= 128) headnorm_kv_store_wide_kernel<16><<<n_rows, 256, 0, s>>>(a);
    else headnorm_kv_store_wide_kernel<32><<<n_rows, 256, 0, s>>>(a);
  }
  else headnorm_kv_store_kernel<bf16_t, bf16_t, 256><<<n_rows, 256, 0, s>>>(a);
  return sb::check_launch("sb_headnorm_kv_store");
}

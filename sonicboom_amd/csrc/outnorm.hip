// Norms for blocks that norm what leaves a sublayer, and for weights kept as multiplier minus offset:
//   un(v, w) = v / sqrt(mean(v^2) + eps) * (offset + w)      (offset 1: "one plus the weight")
//
//   sb_offset_norm      y[r,:] = un(x[rows[r],:])                               (final norm, any norm)
//   sb_norm_add         x[t,:] += un(sum_s a_s(t) part_s[t,:] (+ b(t) extra[t,:]))   and a copy of
//                       the new x in the activation type: the pass that ends a sublayer
//                       (do_norm 0: the sum is added as it is)
//   sb_embed_pos_norm   x[r,:] = un(table[id[r],:] * scale + pos[p[r],:])       (the start of a step)
//
// Sums of squares in double, per thread in ascending order, a fixed butterfly over the wave, the
// four waves in ascending order: a row's bits depend on the row alone.
#include "common.h"

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ double block_sum4(double part) {
  __shared__ double wave_part[kThreads / 64];
  part = wave_sum(part);
  __syncthreads();      // the slots may still be read by a sum before this one
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = part;
  __syncthreads();
  return ((wave_part[0] + wave_part[1]) + wave_part[2]) + wave_part[3];
}

__device__ __forceinline__ float inv_rms(double total, int width, float eps) {
  return 1.0f / sqrtf(float(total / double(width)) + eps);
}

template <typename TO>
__global__ void __launch_bounds__(kThreads)
offset_norm_kernel(TO *__restrict__ y, const float *__restrict__ x, const void *__restrict__ w, int w_dtype,
                   const int32_t *__restrict__ rows, int width, float eps, float offset) {
  const int r = blockIdx.x;
  const float *xr = x + size_t(rows ? rows[r] : r) * width;
  double part = 0.0;
  for (int i = threadIdx.x; i < width; i += kThreads) { const float v = xr[i]; part += double(v * v); }
  const float inv = inv_rms(block_sum4(part), width, eps);
  for (int i = threadIdx.x; i < width; i += kThreads) {
    const float m = w ? offset + ld_dyn(w, w_dtype, i) : 1.0f;
    st_f(y, size_t(r) * width + i, (xr[i] * inv) * m);
  }
}

struct AddArgs {
  float *x; void *copy;
  const float *part; int n_slices; size_t slice_stride, row_stride;
  const float *part_w; int part_w_stride;            // NULL: every slice counts once
  const float *extra; const float *extra_w; int extra_w_stride;
  const void *w; int w_dtype; int width; float eps, offset; int do_norm;
};

template <typename TC>
__global__ void __launch_bounds__(kThreads) norm_add_kernel(AddArgs a) {
  extern __shared__ float row[];
  const int t = blockIdx.x;
  const float *p = a.part + size_t(t) * a.row_stride;
  const float *pw = a.part_w ? a.part_w + size_t(t) * a.part_w_stride : nullptr;
  const float ew = a.extra ? (a.extra_w ? a.extra_w[size_t(t) * a.extra_w_stride] : 1.0f) : 0.0f;
  double sq = 0.0;
  for (int i = threadIdx.x; i < a.width; i += kThreads) {
    float v = 0.0f;
    if (pw) for (int s = 0; s < a.n_slices; ++s) v = fmaf(pw[s], p[s * a.slice_stride + i], v);
    else for (int s = 0; s < a.n_slices; ++s) v += p[s * a.slice_stride + i];
    if (a.extra) v = fmaf(ew, a.extra[size_t(t) * a.width + i], v);
    row[i] = v;
    sq += double(v * v);
  }
  const float inv = a.do_norm ? inv_rms(block_sum4(sq), a.width, a.eps) : 1.0f;
  float *xr = a.x + size_t(t) * a.width;
  TC *cr = a.copy ? (TC *)a.copy + size_t(t) * a.width : nullptr;
  for (int i = threadIdx.x; i < a.width; i += kThreads) {
    const float m = a.do_norm && a.w ? a.offset + ld_dyn(a.w, a.w_dtype, i) : 1.0f;
    const float v = xr[i] + (row[i] * inv) * m;
    xr[i] = v;
    if (cr) st_f(cr, i, v);
  }
}

// The same pass for rows in fours that fit a block's registers: a thread keeps KEEP groups of four, asks
// for every slice of all of them before it adds any (slices past the last read the last again with a
// multiplier of zero: no branch stands between the loads), and the row never goes through LDS.  Few rows:
// 1024 threads a row, so that a row's loads are one round trip; many rows: 256.
constexpr int kMaxFastSlices = 8;

template <int THREADS>
__device__ __forceinline__ double block_sum_n(double part) {
  __shared__ double wave_part[THREADS / 64];
  part = wave_sum(part);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = part;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int k = 0; k < THREADS / 64; ++k) total += wave_part[k];
  return total;
}

template <typename TC, int THREADS, int KEEP, int SL>      // SL: slices the unrolled loops ask for (>= the row's)
__global__ void __launch_bounds__(THREADS) norm_add_fast_kernel(AddArgs a) {
  const int t = blockIdx.x, tid = threadIdx.x;
  const int n_groups = a.width / 4;
  const float4 *p = reinterpret_cast<const float4 *>(a.part + size_t(t) * a.row_stride);
  const size_t slice4 = a.slice_stride / 4;
  float sw[SL];
#pragma unroll
  for (int s = 0; s < SL; ++s)
    sw[s] = s < a.n_slices ? (a.part_w ? a.part_w[size_t(t) * a.part_w_stride + s] : 1.0f) : 0.0f;
  const float ew = a.extra ? (a.extra_w ? a.extra_w[size_t(t) * a.extra_w_stride] : 1.0f) : 0.0f;
  float4 v[KEEP], xv[KEEP], ev[KEEP], in[KEEP][SL];
  const float4 *x4 = reinterpret_cast<const float4 *>(a.x + size_t(t) * a.width);
  const float4 *e4 = a.extra ? reinterpret_cast<const float4 *>(a.extra + size_t(t) * a.width) : x4;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int g = min(tid + i * THREADS, n_groups - 1);
#pragma unroll
    for (int s = 0; s < SL; ++s) in[i][s] = p[size_t(min(s, a.n_slices - 1)) * slice4 + g];
    xv[i] = x4[g];
    ev[i] = e4[g];
  }
  double sq = 0.0;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (a.part_w) {
#pragma unroll
      for (int s = 0; s < SL; ++s) {
        acc.x = fmaf(sw[s], in[i][s].x, acc.x); acc.y = fmaf(sw[s], in[i][s].y, acc.y);
        acc.z = fmaf(sw[s], in[i][s].z, acc.z); acc.w = fmaf(sw[s], in[i][s].w, acc.w);
      }
    } else {
#pragma unroll
      for (int s = 0; s < SL; ++s)
        if (s < a.n_slices) { acc.x += in[i][s].x; acc.y += in[i][s].y; acc.z += in[i][s].z; acc.w += in[i][s].w; }
    }
    if (a.extra) {
      acc.x = fmaf(ew, ev[i].x, acc.x); acc.y = fmaf(ew, ev[i].y, acc.y);
      acc.z = fmaf(ew, ev[i].z, acc.z); acc.w = fmaf(ew, ev[i].w, acc.w);
    }
    v[i] = acc;
    if (tid + i * THREADS < n_groups)
      sq += double(acc.x * acc.x) + double(acc.y * acc.y) + double(acc.z * acc.z) + double(acc.w * acc.w);
  }
  const float inv = a.do_norm ? inv_rms(block_sum_n<THREADS>(sq), a.width, a.eps) : 1.0f;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int g = tid + i * THREADS;
    if (g >= n_groups) continue;
    float m[4] = {1.f, 1.f, 1.f, 1.f};
    if (a.do_norm && a.w) {
#pragma unroll
      for (int e = 0; e < 4; ++e) m[e] = a.offset + ld_dyn(a.w, a.w_dtype, 4 * g + e);
    }
    float4 o;
    o.x = xv[i].x + (v[i].x * inv) * m[0]; o.y = xv[i].y + (v[i].y * inv) * m[1];
    o.z = xv[i].z + (v[i].z * inv) * m[2]; o.w = xv[i].w + (v[i].w * inv) * m[3];
    reinterpret_cast<float4 *>(a.x + size_t(t) * a.width)[g] = o;
    if (a.copy) {
      TC *cr = (TC *)a.copy + size_t(t) * a.width + 4 * g;
      if constexpr (sizeof(TC) == 2) {
        uint2 w2;
        w2.x = uint32_t(f32_to_bf16(o.x)) | uint32_t(f32_to_bf16(o.y)) << 16;
        w2.y = uint32_t(f32_to_bf16(o.z)) | uint32_t(f32_to_bf16(o.w)) << 16;
        *reinterpret_cast<uint2 *>(cr) = w2;
      } else {
        *reinterpret_cast<float4 *>(cr) = o;
      }
    }
  }
}

template <typename TC, int THREADS, int SL>
bool launch_fast_sl(const AddArgs &a, int n_rows, hipStream_t s) {
  const int need = (a.width / 4 + THREADS - 1) / THREADS;
  if (need <= 1) norm_add_fast_kernel<TC, THREADS, 1, SL><<<n_rows, THREADS, 0, s>>>(a);
  else if (need <= 2) norm_add_fast_kernel<TC, THREADS, 2, SL><<<n_rows, THREADS, 0, s>>>(a);
  else if (need <= 4 && THREADS == 256 && SL <= 4) norm_add_fast_kernel<TC, THREADS, 4, SL><<<n_rows, THREADS, 0, s>>>(a);
  else return false;
  return true;
}

template <typename TC, int THREADS>
bool launch_fast(const AddArgs &a, int n_rows, hipStream_t s) {
  if (a.n_slices <= 1) return launch_fast_sl<TC, THREADS, 1>(a, n_rows, s);
  if (a.n_slices <= 2) return launch_fast_sl<TC, THREADS, 2>(a, n_rows, s);
  if (a.n_slices <= 4) return launch_fast_sl<TC, THREADS, 4>(a, n_rows, s);
  return launch_fast_sl<TC, THREADS, 8>(a, n_rows, s);
}

template <typename TC>
__global__ void __launch_bounds__(kThreads)
embed_pos_norm_kernel(float *__restrict__ x, TC *__restrict__ copy, const void *__restrict__ table, int table_dtype,
                      const void *__restrict__ pos_table, int pos_dtype, const int32_t *__restrict__ ids,
                      const int32_t *__restrict__ row_pos, int vocab, int n_positions, float scale,
                      const void *__restrict__ w, int w_dtype, int width, float eps, float offset, int do_norm) {
  extern __shared__ float row[];
  const int r = blockIdx.x;
  const int id = ids[r], p = pos_table ? row_pos[r] : 0;
  float *xr = x + size_t(r) * width;
  if (id < 0 || id >= vocab || p < 0 || (pos_table && p >= n_positions)) {      // not a row of the tables
    for (int i = threadIdx.x; i < width; i += kThreads) {
      xr[i] = __uint_as_float(0x7fc00000u);
      if (copy) st_f(copy, size_t(r) * width + i, xr[i]);
    }
    return;
  }
  double sq = 0.0;
  for (int i = threadIdx.x; i < width; i += kThreads) {
    float v = ld_dyn(table, table_dtype, size_t(id) * width + i) * scale;
    if (pos_table) v += ld_dyn(pos_table, pos_dtype, size_t(p) * width + i);
    row[i] = v;
    sq += double(v * v);
  }
  float inv = 1.0f;
  if (do_norm) inv = inv_rms(block_sum4(sq), width, eps);
  for (int i = threadIdx.x; i < width; i += kThreads) {
    float v = row[i];
    if (do_norm) v = (v * inv) * (w ? offset + ld_dyn(w, w_dtype, i) : 1.0f);
    xr[i] = v;
    if (copy) st_f(copy, size_t(r) * width + i, v);
  }
}

constexpr int kMaxWidth = 16384;      // a row of floats in LDS

}  // namespace

extern "C" int sb_offset_norm(void *y, int out_dtype, const float *x, const void *w, int w_dtype, const int32_t *rows,
                              int n_rows, int width, float eps, float offset, void *stream) {
  SB_REQUIRE(y && x, "sb_offset_norm: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0, "sb_offset_norm: bad sizes rows=%d width=%d", n_rows, width);
  SB_REQUIRE(sb::valid_dtype(out_dtype) && (!w || sb::valid_dtype(w_dtype)), "sb_offset_norm: unknown dtype");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == SB_F32) offset_norm_kernel<float><<<n_rows, kThreads, 0, s>>>((float *)y, x, w, w_dtype, rows, width, eps, offset);
  else offset_norm_kernel<bf16_t><<<n_rows, kThreads, 0, s>>>((bf16_t *)y, x, w, w_dtype, rows, width, eps, offset);
  return sb::check_launch("sb_offset_norm");
}

extern "C" int sb_norm_add(float *x, void *copy, int copy_dtype, const float *part, int n_slices, size_t slice_stride,
                           size_t row_stride, const float *part_w, int part_w_stride, const float *extra,
                           const float *extra_w, int extra_w_stride, const void *w, int w_dtype, int n_rows, int width,
                           float eps, float offset, int do_norm, void *stream) {
  SB_REQUIRE(x && part, "sb_norm_add: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && n_slices > 0, "sb_norm_add: bad sizes rows=%d width=%d slices=%d", n_rows, width, n_slices);
  SB_REQUIRE((!copy || sb::valid_dtype(copy_dtype)) && (!w || sb::valid_dtype(w_dtype)), "sb_norm_add: unknown dtype");
  SB_SUPPORT(width <= kMaxWidth, "sb_norm_add: rows of %d are wider than %d", width, kMaxWidth);
  if (n_rows == 0) return SB_OK;
  const AddArgs a{x, copy, part, n_slices, slice_stride, row_stride, part_w, part_w_stride, extra, extra_w, extra_w_stride,
                  w, w_dtype, width, eps, offset, do_norm};
  hipStream_t s = (hipStream_t)stream;
  const bool bf = copy && copy_dtype == SB_BF16;
  const auto aligned = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  if (width % 4 == 0 && n_slices <= kMaxFastSlices && slice_stride % 4 == 0 && row_stride % 4 == 0 && aligned(x) &&
      aligned(part) && aligned(extra) && aligned(copy)) {
    // (float32 throughout keeps one block shape whatever the number of rows: the order of a row's sum
    // of squares, and so its bits, must not depend on what else the step holds)
    bool done;
    if (bf && n_rows <= 64) done = launch_fast<bf16_t, 1024>(a, n_rows, s);
    else done = bf ? launch_fast<bf16_t, 256>(a, n_rows, s) : launch_fast<float, 256>(a, n_rows, s);
    if (done) return sb::check_launch("sb_norm_add");
  }
  const size_t lds = size_t(width) * sizeof(float);
  if (bf) norm_add_kernel<bf16_t><<<n_rows, kThreads, lds, s>>>(a);
  else norm_add_kernel<float><<<n_rows, kThreads, lds, s>>>(a);
  return sb::check_launch("sb_norm_add");
}

extern "C" int sb_embed_pos_norm(float *x, void *copy, int copy_dtype, const void *table, int table_dtype,
                                 const void *pos_table, int pos_dtype, const int32_t *ids, const int32_t *row_pos,
                                 int n_rows, int vocab, int n_positions, float scale, const void *w, int w_dtype,
                                 int width, float eps, float offset, int do_norm, void *stream) {
  SB_REQUIRE(x && table && ids && (!pos_table || row_pos), "sb_embed_pos_norm: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && vocab > 0, "sb_embed_pos_norm: bad sizes rows=%d width=%d", n_rows, width);
  SB_REQUIRE(sb::valid_dtype(table_dtype) && (!pos_table || sb::valid_dtype(pos_dtype)) && (!w || sb::valid_dtype(w_dtype)) &&
                 (!copy || sb::valid_dtype(copy_dtype)), "sb_embed_pos_norm: unknown dtype");
  SB_SUPPORT(width <= kMaxWidth, "sb_embed_pos_norm: rows of %d are wider than %d", width, kMaxWidth);
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = size_t(width) * sizeof(float);
  if (copy && copy_dtype == SB_BF16)
    embed_pos_norm_kernel<bf16_t><<<n_rows, kThreads, lds, s>>>(x, (bf16_t *)copy, table, table_dtype, pos_table, pos_dtype, ids,
                                                                row_pos, vocab, n_positions, scale, w, w_dtype, width, eps, offset, do_norm);
  else
    embed_pos_norm_kernel<float><<<n_rows, kThreads, lds, s>>>(x, (float *)copy, table, table_dtype, pos_table, pos_dtype, ids,
                                                               row_pos, vocab, n_positions, scale, w, w_dtype, width, eps, offset, do_norm);
  return sb::check_launch("sb_embed_pos_norm");
}

// Latent attention on the matrix cores (bfloat16): the per-head products that carry queries into
// the latent space and results out of it, and attention over the cached latent rows.
//
// sb_head_product_bf16: out[t, a, :] = W[a] in[t, a, :], W[a] [n_out, n_in] (output-major).  A wave
// takes 16 rows of one head and 64 outputs; both operands go from global memory straight into
// MFMA 16x16x32 fragments (a lane's eight k are 16 consecutive bytes on either side), the result
// lands as four consecutive outputs of one row per lane.
//
// sb_latent_attention_bf16: all query heads read the same cached rows [c | r], so a block stages
// a page of 64 rows once in LDS, twice over: as it lies (a key's numbers consecutive: the A
// operand of S^T = K Q^T) and with the latent part turned (a number's 64 keys consecutive: the A
// operand of O^T = C^T P^T), and its four waves each run a tile of 16 query columns against it.
// In a prompt step a wave's 16 columns are 16 consecutive rows of one head; in a decode step they
// are 16 heads of the one row.  The next page's rows are asked of memory before the current
// page's products start and wait in registers.  Softmax runs in the result layout of S^T (a lane
// holds 16 keys of one column a page; column maximum and sum over the four lane groups), P goes
// back in as the B operand of the second product without leaving registers: the keys of a
// 32-key step are taken in the order the first product left them, by V's fragment reads.
#include "mfma.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kPadK = 8;     // bf16 a key row is padded by in LDS
constexpr int kVtStride = SB_PAGE + 8;

template <bool GATED>
__global__ void __launch_bounds__(kThreads)
head_product_mfma_kernel(bf16_t *__restrict__ out, int out_stride, int out_hstride, const bf16_t *__restrict__ in,
                         int in_stride, int in_hstride, const bf16_t *__restrict__ w, const float *__restrict__ gate,
                         int gate_stride, int n_rows, int n_in, int n_out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int a = blockIdx.y;
  const int t = blockIdx.x * 64 + wave * 16 + (lane & 15);      // this lane's row (B operand's column)
  const int o0 = blockIdx.z * 64;
  const int g = lane >> 4;
  const bf16_t *xin = in + size_t(min(t, n_rows - 1)) * in_stride + size_t(a) * in_hstride;
  const bf16_t *wa = w + size_t(a) * n_out * n_in;
  floatx4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < n_in; k0 += 32) {
    const int k = k0 + 8 * g;
    const bool kin = k < n_in;                                   // n_in is a multiple of 8
    const uint4 b = ld16(xin + (kin ? k : 0), kin && t < n_rows);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int o = o0 + 16 * j + (lane & 15);
      const uint4 av = ld16(wa + size_t(min(o, n_out - 1)) * n_in + (kin ? k : 0), kin && o < n_out);
      acc[j] = mfma16(as_bf16x8(av), as_bf16x8(b), acc[j]);
    }
  }
  if (t >= n_rows) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int o = o0 + 16 * j + 4 * g + i;
      if (o >= n_out) continue;
      float v = acc[j][i];
      if (GATED) {
        const float gv = gate[size_t(t) * gate_stride + size_t(a) * n_out + o];
        v = v * (1.0f / (1.0f + expf(-gv)));
      }
      out[size_t(t) * out_stride + size_t(a) * out_hstride + o] = f32_to_bf16(v);
    }
  }
}

// KQ: steps of 32 over a latent row that the unrolled loops cover; NV: tiles of 16 over the latent part.
template <int KQ, int NV>
__global__ void __launch_bounds__(kThreads)
latent_attention_mfma_kernel(bf16_t *__restrict__ out, const bf16_t *__restrict__ q, const bf16_t *__restrict__ cache,
                             const int32_t *__restrict__ page_table, int max_pages, int n_pages_total,
                             const int32_t *__restrict__ row_pos, const int32_t *__restrict__ tiles, int heads, int rank,
                             int rot_dim, float scale, int window, int tile_rows) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int latent = rank + rot_dim;
  const int kq = (latent + 31) / 32, nv = (rank + 15) / 16;
  const int lk = kq * 32 + kPadK;                    // bf16 per staged key row
  bf16_t *ks = reinterpret_cast<bf16_t *>(lds);      // [SB_PAGE][lk]
  bf16_t *vt = ks + SB_PAGE * lk;                    // [nv * 16][kVtStride]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, g = lane >> 4;
  const int r0 = tiles[4 * blockIdx.x], n_tile = tiles[4 * blockIdx.x + 1], seq = tiles[4 * blockIdx.x + 2];
  const int heads_per_wave = 16 / tile_rows;
  const int head = (blockIdx.y * kWaves + wave) * heads_per_wave + col / tile_rows;
  const int r = col % tile_rows;
  const bool wave_works = (blockIdx.y * kWaves + wave) * heads_per_wave < heads;
  const bool valid = r < n_tile && head < heads;
  const int row = r0 + min(r, n_tile - 1);
  const int pos0 = row_pos[r0];
  const int pos = pos0 + min(r, n_tile - 1);         // a tile's rows are consecutive positions of one sequence
  const int lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  const int lo_blk = (window > 0 && pos0 >= window) ? pos0 - window + 1 : 0;
  const int hi_blk = pos0 + n_tile - 1;

  // the pads that staging never writes must not hold what multiplies to NaN
  for (int i = tid; i < SB_PAGE * (lk - latent); i += kThreads) {
    const int key = i / (lk - latent), e = i - key * (lk - latent);
    ks[key * lk + latent + e] = 0;
  }
  for (int i = tid; i < (nv * 16 - rank) * kVtStride; i += kThreads) vt[rank * kVtStride + i] = 0;
  for (int i = tid; i < rank * (kVtStride - SB_PAGE); i += kThreads) {
    const int d = i / (kVtStride - SB_PAGE), e = i - d * (kVtStride - SB_PAGE);
    vt[d * kVtStride + SB_PAGE + e] = 0;
  }

  // this lane's query fragments: column (row, head), k = 32 kk + 8 g .. + 7
  uint4 qf[KQ];
  const bf16_t *qrow = q + (size_t(row) * heads + min(head, heads - 1)) * latent;
#pragma unroll
  for (int kk = 0; kk < KQ; ++kk) {
    const int k = 32 * kk + 8 * g;
    qf[kk] = ld16(qrow + (k < latent ? k : 0), valid && k < latent);      // latent is a multiple of 8
  }

  const float neg_inf = -__builtin_inff();
  float m_run = neg_inf, l_run = 0.0f;
  floatx4_t o[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) o[v] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  // staging: a page is 64 rows of latent / 8 chunks of 16 bytes; thread (key = idx % 64, chunk = idx / 64)
  const int chunks = latent / 8;
  constexpr int kMaxStage = (KQ * 32 / 8 * SB_PAGE + kThreads - 1) / kThreads;
  uint4 staged[kMaxStage];
  const int c_first = lo_blk / SB_PAGE, c_last = hi_blk / SB_PAGE;
  auto page_of = [&](int c) -> int {
    const int p = c < max_pages ? page_table[size_t(seq) * max_pages + c] : -1;
    return (p >= 0 && p < n_pages_total) ? p : -1;
  };
  auto load_page = [&](int page) {
#pragma unroll
    for (int it = 0; it < kMaxStage; ++it) {
      const int idx = tid + it * kThreads;
      const int key = idx & 63, chunk = idx >> 6;
      staged[it] = ld16(cache + (size_t(max(page, 0)) * SB_PAGE + key) * latent + 8 * min(chunk, chunks - 1),
                        page >= 0 && chunk < chunks);
    }
  };
  auto store_page = [&]() {
#pragma unroll
    for (int it = 0; it < kMaxStage; ++it) {
      const int idx = tid + it * kThreads;
      const int key = idx & 63, chunk = idx >> 6;
      if (chunk >= chunks) continue;
      *reinterpret_cast<uint4 *>(ks + key * lk + 8 * chunk) = staged[it];
      if (8 * chunk < rank) {
        const uint32_t wds[4] = {staged[it].x, staged[it].y, staged[it].z, staged[it].w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int d = 8 * chunk + e;
          if (d < rank) vt[d * kVtStride + key] = bf16_t((wds[e >> 1] >> (16 * (e & 1))) & 0xffffu);
        }
      }
    }
  };

  int c = c_first;
  while (c <= c_last && page_of(c) < 0) ++c;          // pages that are not there hold no visible key
  if (c <= c_last) load_page(page_of(c));
  while (c <= c_last) {
    __syncthreads();                                  // the page before has been read by every wave
    store_page();
    __syncthreads();
    int c_next = c + 1;
    while (c_next <= c_last && page_of(c_next) < 0) ++c_next;
    if (c_next <= c_last) load_page(page_of(c_next)); // in flight while this page is worked on

    if (wave_works) {
      floatx4_t s[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        s[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
        const bf16_t *kr = ks + (16 * t + col) * lk + 8 * g;
#pragma unroll
        for (int kk = 0; kk < KQ; ++kk)
          if (kk < kq) s[t] = mfma16(as_bf16x8(*reinterpret_cast<const uint4 *>(kr + 32 * kk)), as_bf16x8(qf[kk]), s[t]);
      }
      // s[t][i] = score of key 64 c + 16 t + 4 g + i for this lane's column
      float mx = neg_inf;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = c * SB_PAGE + 16 * t + 4 * g + i;
          const bool vis = valid && j >= lo && j <= pos;
          s[t][i] = vis ? s[t][i] * scale : neg_inf;
          mx = fmaxf(mx, s[t][i]);
        }
      mx = max_over_lane_groups(mx);
      const float m_new = fmaxf(m_run, mx);
      const float m_safe = m_new == neg_inf ? 0.0f : m_new;
      const float alpha = expf(m_run - m_safe);        // 0 while nothing has been seen
      float sum = 0.0f;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[t][i] = expf(s[t][i] - m_safe);
          sum += s[t][i];
        }
      l_run = l_run * alpha + sum;
      m_run = m_new;
      uint4 pf[2];
#pragma unroll
      for (int u = 0; u < 2; ++u)
        pf[u] = make_uint4(pack_bf16(s[2 * u][0], s[2 * u][1]), pack_bf16(s[2 * u][2], s[2 * u][3]),
                           pack_bf16(s[2 * u + 1][0], s[2 * u + 1][1]), pack_bf16(s[2 * u + 1][2], s[2 * u + 1][3]));
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        if (v >= nv) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[v][i] *= alpha;
        const bf16_t *vr = vt + (16 * v + col) * kVtStride + 4 * g;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const uint2 lo8 = *reinterpret_cast<const uint2 *>(vr + 32 * u);
          const uint2 hi8 = *reinterpret_cast<const uint2 *>(vr + 32 * u + 16);
          o[v] = mfma16(as_bf16x8(make_uint4(lo8.x, lo8.y, hi8.x, hi8.y)), as_bf16x8(pf[u]), o[v]);
        }
      }
    }
    c = c_next;
  }

  if (!wave_works) return;
  float l_tot = l_run + __shfl_xor(l_run, 16, 64);
  l_tot += __shfl_xor(l_tot, 32, 64);
  if (!valid) return;
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  bf16_t *orow = out + (size_t(row) * heads + head) * rank;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    if (v >= nv) continue;
    const int d = 16 * v + 4 * g;
    if (d + 3 < rank) {
      *reinterpret_cast<uint2 *>(orow + d) = make_uint2(pack_bf16(o[v][0] * inv, o[v][1] * inv),
                                                        pack_bf16(o[v][2] * inv, o[v][3] * inv));
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (d + i < rank) orow[d + i] = f32_to_bf16(o[v][i] * inv);
    }
  }
}

template <int KQ, int NV>
int launch_attention(bf16_t *out, const bf16_t *q, const bf16_t *cache, const int32_t *page_table, int max_pages,
                     int n_pages_total, const int32_t *row_pos, const int32_t *tiles, int n_tiles, int heads, int rank,
                     int rot_dim, float scale, int window, int tile_rows, hipStream_t s) {
  const int latent = rank + rot_dim;
  const int kq = (latent + 31) / 32, nv = (rank + 15) / 16;
  const size_t lds = (size_t(SB_PAGE) * (kq * 32 + kPadK) + size_t(nv) * 16 * kVtStride) * sizeof(bf16_t);
  static bool raised = false;              // once per kernel of this shape: more dynamic LDS than the default allows
  if (!raised) {
    if (hipFuncSetAttribute((const void *)latent_attention_mfma_kernel<KQ, NV>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      (void)hipGetLastError();
    raised = true;
  }
  const int heads_per_block = kWaves * (16 / tile_rows);
  dim3 grid(n_tiles, (heads + heads_per_block - 1) / heads_per_block);
  latent_attention_mfma_kernel<KQ, NV><<<grid, kThreads, lds, s>>>(out, q, cache, page_table, max_pages, n_pages_total,
                                                                   row_pos, tiles, heads, rank, rot_dim, scale, window,
                                                                   tile_rows);
  return sb::check_launch("sb_latent_attention_bf16");
}

}  // namespace

// 1 when sb_head_product_bf16 takes these sizes and strides (all in elements).
extern "C" int sb_head_product_bf16_ok(int out_stride, int out_hstride, int in_stride, int in_hstride, int n_in) {
  (void)out_stride; (void)out_hstride;
  return n_in % 8 == 0 && in_stride % 8 == 0 && in_hstride % 8 == 0;
}

// out[t, a, o] = sum_i W[a][o][i] in[t, a, i] on the matrix cores; everything bfloat16, gate f32 or NULL
// (times sigmoid(gate[t * gate_stride + a * n_out + o])); in and W 16-byte aligned.
extern "C" int sb_head_product_bf16(void *out, int out_stride, int out_hstride, const void *in, int in_stride,
                                    int in_hstride, const void *w, const float *gate, int gate_stride, int n_rows,
                                    int heads, int n_in, int n_out, void *stream) {
  SB_REQUIRE(out && in && w, "sb_head_product_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads > 0 && n_in > 0 && n_out > 0, "sb_head_product_bf16: bad sizes");
  SB_SUPPORT(sb_head_product_bf16_ok(out_stride, out_hstride, in_stride, in_hstride, n_in),
             "sb_head_product_bf16: inner size and strides must be multiples of 8");
  SB_SUPPORT((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_head_product_bf16: operands must be 16-byte aligned");
  SB_SUPPORT(heads <= 65535 && (n_out + 63) / 64 <= 65535, "sb_head_product_bf16: too many heads or outputs");
  if (n_rows == 0) return SB_OK;
  dim3 grid((n_rows + 63) / 64, heads, (n_out + 63) / 64);
  hipStream_t s = (hipStream_t)stream;
  if (gate)
    head_product_mfma_kernel<true><<<grid, kThreads, 0, s>>>((bf16_t *)out, out_stride, out_hstride, (const bf16_t *)in,
                                                             in_stride, in_hstride, (const bf16_t *)w, gate, gate_stride,
                                                             n_rows, n_in, n_out);
  else
    head_product_mfma_kernel<false><<<grid, kThreads, 0, s>>>((bf16_t *)out, out_stride, out_hstride, (const bf16_t *)in,
                                                              in_stride, in_hstride, (const bf16_t *)w, gate, gate_stride,
                                                              n_rows, n_in, n_out);
  return sb::check_launch("sb_head_product_bf16");
}

// The height of the runs of rows (`tiles`) that a prompt step's launch takes.
extern "C" int sb_latent_attention_tile_rows(void) { return 16; }

// 1 when sb_latent_attention_bf16 takes these sizes.
extern "C" int sb_latent_attention_bf16_ok(int rank, int rot_dim) {
  return rank > 0 && rot_dim >= 0 && rank % 8 == 0 && rot_dim % 8 == 0 && rank + rot_dim <= 576 && rank <= 512;
}

// Attention over cached latent rows on the matrix cores, everything bfloat16 (see the head of the
// file).  tiles int32 [n_tiles, 4] = (first row, rows, sequence, 0): runs of up to tile_rows
// consecutive rows of one sequence; tile_rows 16 for a prompt step, 1 for a step of single rows
// (a wave then takes 16 heads of a row).  out [n_rows, heads, rank], q [n_rows, heads, rank + rot_dim].
extern "C" int sb_latent_attention_bf16(void *out, const void *q, const void *cache, const int32_t *page_table,
                                        int max_pages, int n_pages_total, const int32_t *row_pos, const int32_t *tiles,
                                        int n_tiles, int heads, int rank, int rot_dim, float scale, int window,
                                        int tile_rows, void *stream) {
  SB_REQUIRE(out && q && cache && page_table && row_pos && tiles, "sb_latent_attention_bf16: null pointer");
  SB_REQUIRE(n_tiles >= 0 && heads > 0 && max_pages > 0 && n_pages_total > 0 && window >= 0,
             "sb_latent_attention_bf16: bad sizes");
  SB_REQUIRE(tile_rows == 16 || tile_rows == 1, "sb_latent_attention_bf16: tiles of 16 rows or of one");
  SB_SUPPORT(sb_latent_attention_bf16_ok(rank, rot_dim), "sb_latent_attention_bf16: a latent row of %d + %d is not taken",
             rank, rot_dim);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(cache) | reinterpret_cast<uintptr_t>(out)) % 16 == 0,
             "sb_latent_attention_bf16: operands must be 16-byte aligned");
  if (n_tiles == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const int kq = (rank + rot_dim + 31) / 32, nv = (rank + 15) / 16;
#define SB_GO(KQ, NV)                                                                                              \
  return launch_attention<KQ, NV>((bf16_t *)out, (const bf16_t *)q, (const bf16_t *)cache, page_table, max_pages,    \
                                  n_pages_total, row_pos, tiles, n_tiles, heads, rank, rot_dim, scale, window, tile_rows, s)
  if (kq <= 6 && nv <= 8) SB_GO(6, 8);
  if (kq <= 10 && nv <= 16) SB_GO(10, 16);
  SB_GO(18, 32);
#undef SB_GO
}

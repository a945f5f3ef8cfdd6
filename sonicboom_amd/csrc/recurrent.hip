// Gated recurrences whose gates read the current token only: the state of a sequence is one
// float32 vector that every token updates element by element.
//
// minGRU:  z = sigmoid(a), cand = u + 1/2 for u >= 0 and sigmoid(u) for u < 0,
//          S_t = (1 - z_t) S_(t-1) + z_t cand_t,  out_t = S_t * silu(g_t),
// with (a, u, g) the three thirds of a row of the mixer's input product [rows, 3 * width], all
// float32.  The state of sequence s lies in state[slots[s]] and goes from step to step.
//
// The update is linear in S, S_t = A_t S_(t-1) + B_t with A = 1 - z and B = z cand.  Two kernels:
// the serial one walks a sequence's rows in order, a thread a channel (every step's rows: one
// row in decoding; its sums are those of token-by-token decoding to the bit, so the 32-bit path
// always takes it); the chunked one, for long prompts in bfloat16, cuts a sequence's rows into
// chunks of kChunk, folds every chunk into its (product of A, B of the whole chunk from a zero
// state) in parallel, carries the state over the chunk ends serially and then walks every chunk in
// parallel from the state at its start.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kChunk = 64;

__device__ __forceinline__ float sigmoid_f(float a) { return 1.0f / (1.0f + expf(-a)); }

struct Gate {
  float a, b, silu_g;
};

__device__ __forceinline__ Gate mingru_gate(const float *__restrict__ row, int width, int ch) {
  const float zp = row[ch], up = row[width + ch], gp = row[2 * size_t(width) + ch];
  const float z = sigmoid_f(zp);
  const float cand = up >= 0.0f ? up + 0.5f : sigmoid_f(up);
  Gate g;
  g.a = 1.0f - z;
  g.b = z * cand;
  g.silu_g = gp * sigmoid_f(gp);
  return g;
}

template <typename TO>
__global__ void __launch_bounds__(kThreads)
mingru_serial_kernel(TO *__restrict__ out, const float *__restrict__ p, float *__restrict__ state,
                     const int32_t *__restrict__ cu_rows, const int32_t *__restrict__ slots, int width) {
  const int seq = blockIdx.y;
  const int ch = blockIdx.x * kThreads + threadIdx.x;
  if (ch >= width) return;
  const int r0 = cu_rows[seq], r1 = cu_rows[seq + 1];
  float *sp = state + size_t(slots[seq]) * width + ch;
  float s = *sp;
  for (int r = r0; r < r1; ++r) {
    const Gate g = mingru_gate(p + size_t(r) * 3 * width, width, ch);
    s = g.a * s + g.b;
    st_f(out, size_t(r) * width + ch, s * g.silu_g);
  }
  if (r1 > r0) *sp = s;
}

// chunk c of the launch: rows [first, first + n) of sequence seq, as int32 [n_chunks, 4] =
// (first row, rows, sequence, 0).
__global__ void __launch_bounds__(kThreads)
mingru_fold_kernel(float2 *__restrict__ folded, const float *__restrict__ p, const int32_t *__restrict__ chunks,
                   int width) {
  const int c = blockIdx.y;
  const int ch = blockIdx.x * kThreads + threadIdx.x;
  if (ch >= width) return;
  const int r0 = chunks[4 * c], n = chunks[4 * c + 1];
  float a = 1.0f, b = 0.0f;
  for (int r = r0; r < r0 + n; ++r) {
    const Gate g = mingru_gate(p + size_t(r) * 3 * width, width, ch);
    a = g.a * a;
    b = g.a * b + g.b;
  }
  folded[size_t(c) * width + ch] = make_float2(a, b);
}

// The state at the start of every chunk, in place of its folded pair's first number; the state
// after a sequence's last chunk goes back to state[].
__global__ void __launch_bounds__(kThreads)
mingru_carry_kernel(float2 *__restrict__ folded, float *__restrict__ state, const int32_t *__restrict__ chunks,
                    int n_chunks, const int32_t *__restrict__ slots, int width) {
  const int seq = blockIdx.y;
  const int ch = blockIdx.x * kThreads + threadIdx.x;
  if (ch >= width) return;
  // the chunks lie in the order of the rows, so a sequence's are together: find the first
  int lo = 0, hi = n_chunks;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (chunks[4 * mid + 2] < seq) lo = mid + 1;
    else hi = mid;
  }
  float *sp = state + size_t(slots[seq]) * width + ch;
  float s = *sp;
  int c = lo;
  for (; c < n_chunks && chunks[4 * c + 2] == seq; ++c) {
    const float2 f = folded[size_t(c) * width + ch];
    folded[size_t(c) * width + ch].x = s;
    s = f.x * s + f.y;
  }
  if (c > lo) *sp = s;
}

template <typename TO>
__global__ void __launch_bounds__(kThreads)
mingru_walk_kernel(TO *__restrict__ out, const float *__restrict__ p, const float2 *__restrict__ folded,
                   const int32_t *__restrict__ chunks, int width) {
  const int c = blockIdx.y;
  const int ch = blockIdx.x * kThreads + threadIdx.x;
  if (ch >= width) return;
  const int r0 = chunks[4 * c], n = chunks[4 * c + 1];
  float s = folded[size_t(c) * width + ch].x;
  for (int r = r0; r < r0 + n; ++r) {
    const Gate g = mingru_gate(p + size_t(r) * 3 * width, width, ch);
    s = g.a * s + g.b;
    st_f(out, size_t(r) * width + ch, s * g.silu_g);
  }
}

}  // namespace

extern "C" int sb_mingru_chunk_rows(void) { return kChunk; }

// out[r, :] = S_r * silu(g_r) for the rows of a step, sequence by sequence, and state[] moved on.
//   p        f32 [n_rows, 3 * width]: the pre-activations (a | u | g) of every row
//   state    f32 [*, width]; sequence s uses row slots[s]
//   cu_rows  int32 [n_seqs + 1]: first row of every sequence
//   chunks, folded: NULL for the serial kernel; else the step's rows in chunks of at most
//            sb_mingru_chunk_rows() rows of one sequence, int32 [n_chunks, 4] (first row, rows,
//            sequence, 0) in the order of the rows, and scratch of 2 * n_chunks * width floats
//            (8-byte aligned).
extern "C" int sb_mingru_scan(void *out, int out_dtype, const float *p, float *state, const int32_t *cu_rows,
                              const int32_t *slots, int n_seqs, int n_rows, int width, const int32_t *chunks,
                              int n_chunks, float *folded, void *stream) {
  SB_REQUIRE(out && p && state && cu_rows && slots, "sb_mingru_scan: null pointer");
  SB_REQUIRE(n_seqs >= 0 && n_rows >= 0 && width > 0, "sb_mingru_scan: bad sizes");
  SB_REQUIRE(sb::valid_dtype(out_dtype), "sb_mingru_scan: unknown dtype");
  SB_SUPPORT(n_seqs <= 65535 && n_chunks <= 65535, "sb_mingru_scan: more than 65535 sequences or chunks");
  if (n_seqs == 0 || n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const unsigned bx = unsigned((width + kThreads - 1) / kThreads);
  if (!chunks) {
    dim3 grid(bx, n_seqs);
    if (out_dtype == SB_F32) mingru_serial_kernel<float><<<grid, kThreads, 0, s>>>((float *)out, p, state, cu_rows, slots, width);
    else mingru_serial_kernel<bf16_t><<<grid, kThreads, 0, s>>>((bf16_t *)out, p, state, cu_rows, slots, width);
    return sb::check_launch("sb_mingru_scan");
  }
  SB_REQUIRE(folded && n_chunks > 0, "sb_mingru_scan: the chunked form needs its tables and scratch");
  SB_REQUIRE(reinterpret_cast<uintptr_t>(folded) % 8 == 0, "sb_mingru_scan: scratch must be 8-byte aligned");
  dim3 cgrid(bx, n_chunks), sgrid(bx, n_seqs);
  mingru_fold_kernel<<<cgrid, kThreads, 0, s>>>((float2 *)folded, p, chunks, width);
  mingru_carry_kernel<<<sgrid, kThreads, 0, s>>>((float2 *)folded, state, chunks, n_chunks, slots, width);
  if (out_dtype == SB_F32) mingru_walk_kernel<float><<<cgrid, kThreads, 0, s>>>((float *)out, p, (const float2 *)folded, chunks, width);
  else mingru_walk_kernel<bf16_t><<<cgrid, kThreads, 0, s>>>((bf16_t *)out, p, (const float2 *)folded, chunks, width);
  return sb::check_launch("sb_mingru_scan");
}

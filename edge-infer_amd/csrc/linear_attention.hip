// Linear attention with a fixed decay per head.  A row of the projection is
// [q: H * DK | k: H * DK | v: H * DV | g: H * DV]; with q, k, v passed through silu, per head
//
//   S_t = decay_h S_(t-1) + k_t v_t^T        S is [DK, DV], float32, zero before the sequence
//   o_t = S_t^T q_t
//
// and then out = rmsnorm(o over all heads) * w * sigmoid(g) in the rows' type.  The state is a
// float32 table with two versions of every sequence's row ([H][DK][DV]): a step reads the row
// `seq_in` names and writes the whole row `seq_out` names.  The walk over a sequence's tokens
// is a true recurrence: tokens are taken in order, one after the other, whatever the step
// holds (a whole prompt, a portion, one token), so a position's result does not depend on how
// its sequence was cut.
#include "common.h"

namespace {

constexpr int kTile = 16;      // tokens whose operands lie in LDS at a time
constexpr int kThreads = 256;

template <typename TI>
__device__ __forceinline__ float sliced(const TI* p, int nsplit, size_t split_stride) {
  float v = 0.f;
  for (int s = 0; s < nsplit; ++s) v += ei::to_f32<TI>(p[s * split_stride]);
  return v;
}

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

// A block a (sequence, head, COLS columns of S).  Thread (c, g): column c, rows g R .. g R + R - 1
// (R a multiple of 4; the 256 / COLS groups g hold G R >= DK rows; rows beyond DK hold zeros).
// A tile of 16 tokens' q, k and v lies in LDS while its tokens are walked; with AHEAD the next
// tile's values are asked of global memory before the walk and wait in registers (launches of
// few blocks, which live on how soon a tile is there; launches that fill the chip lose more by
// the registers than they gain).  ACT: the rows hold raw projections and silu is taken here;
// else they hold q, k and v as `la_activate` left them (a prompt's many tokens: every block of
// a head would take the same silu of q and k again).
template <typename TI, int R, int COLS, bool AHEAD, bool ACT>
__global__ void __launch_bounds__(kThreads)
la_scan_kernel(const TI* __restrict__ proj, int nsplit, size_t split_stride, size_t row_stride,
               const float* __restrict__ decay, const float* state_in_table, float* state_out_table,
               const int32_t* __restrict__ seq_in, const int32_t* __restrict__ seq_out,
               const int32_t* __restrict__ seq_count, const int32_t* __restrict__ seq_row0,
               float* __restrict__ o_raw, int H, int DK, int DV) {
  constexpr int G = kThreads / COLS;
  constexpr int DKP = G * R;
  constexpr int QK_PER = kTile * DKP / kThreads;      // q (and k) values a thread fetches a tile
  constexpr int V_PER = (kTile * COLS + kThreads - 1) / kThreads;
  __shared__ __attribute__((aligned(16))) float qs[kTile][DKP];
  __shared__ __attribute__((aligned(16))) float ks[kTile][DKP];
  __shared__ float vs[kTile][COLS];
  __shared__ float part[kTile][G][COLS];
  const int seq = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * COLS;
  const int count = seq_count[seq];
  if (count <= 0) return;                       // a padding sequence
  const int t = threadIdx.x, c = t % COLS, g = t / COLS;
  const int col = col0 + c;
  const bool col_live = col < DV;
  const size_t state_floats = static_cast<size_t>(H) * DK * DV;
  const float* s_in = state_in_table + static_cast<size_t>(seq_in[seq]) * state_floats +
                      static_cast<size_t>(head) * DK * DV;
  float* s_out = state_out_table + static_cast<size_t>(seq_out[seq]) * state_floats +
                 static_cast<size_t>(head) * DK * DV;
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = g * R + i;
    S[i] = (col_live && row < DK) ? s_in[static_cast<size_t>(row) * DV + col] : 0.f;
  }
  const float d = decay[head];
  const int row0 = seq_row0[seq];
  const size_t q_at = static_cast<size_t>(head) * DK;
  const size_t k_at = static_cast<size_t>(H) * DK + q_at;
  const size_t v_at = 2 * static_cast<size_t>(H) * DK + static_cast<size_t>(head) * DV + col0;
  const size_t out_width = static_cast<size_t>(H) * DV;

  float q_next[QK_PER], k_next[QK_PER], v_next[V_PER];
  // the raw projections of the tile that starts at `tile0`, into registers
  auto fetch = [&](int tile0) {
    const int nt = min(kTile, count - tile0);
#pragma unroll
    for (int u = 0; u < QK_PER; ++u) {
      const int idx = t + u * kThreads, tt = idx / DKP, row = idx % DKP;
      q_next[u] = k_next[u] = 0.f;
      if (tt < nt && row < DK) {
        const TI* src = proj + static_cast<size_t>(row0 + tile0 + tt) * row_stride;
        q_next[u] = sliced(src + q_at + row, nsplit, split_stride);
        k_next[u] = sliced(src + k_at + row, nsplit, split_stride);
      }
    }
#pragma unroll
    for (int u = 0; u < V_PER; ++u) {
      const int idx = t + u * kThreads, tt = idx / COLS, cc = idx % COLS;
      v_next[u] = 0.f;
      if (idx < kTile * COLS && tt < nt && col0 + cc < DV)
        v_next[u] = sliced(proj + static_cast<size_t>(row0 + tile0 + tt) * row_stride + v_at + cc,
                           nsplit, split_stride);
    }
  };
  if constexpr (AHEAD) fetch(0);
  for (int tile0 = 0; tile0 < count; tile0 += kTile) {
    const int nt = min(kTile, count - tile0);
    if constexpr (!AHEAD) fetch(tile0);
#pragma unroll
    for (int u = 0; u < QK_PER; ++u) {
      const int idx = t + u * kThreads;
      qs[idx / DKP][idx % DKP] = ACT ? silu_f32(q_next[u]) : q_next[u];
      ks[idx / DKP][idx % DKP] = ACT ? silu_f32(k_next[u]) : k_next[u];
    }
#pragma unroll
    for (int u = 0; u < V_PER; ++u) {
      const int idx = t + u * kThreads;
      if (idx < kTile * COLS) vs[idx / COLS][idx % COLS] = ACT ? silu_f32(v_next[u]) : v_next[u];
    }
    __syncthreads();
    if constexpr (AHEAD) {
      if (tile0 + kTile < count) fetch(tile0 + kTile);
    }
    for (int tt = 0; tt < nt; ++tt) {
      const float vv = vs[tt][c];
      const float4* kq = reinterpret_cast<const float4*>(&ks[tt][g * R]);
      const float4* qq = reinterpret_cast<const float4*>(&qs[tt][g * R]);
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < R / 4; ++i4) {
        const float4 k4 = kq[i4], q4 = qq[i4];
        S[4 * i4 + 0] = d * S[4 * i4 + 0] + k4.x * vv;
        S[4 * i4 + 1] = d * S[4 * i4 + 1] + k4.y * vv;
        S[4 * i4 + 2] = d * S[4 * i4 + 2] + k4.z * vv;
        S[4 * i4 + 3] = d * S[4 * i4 + 3] + k4.w * vv;
        a0 += S[4 * i4 + 0] * q4.x;
        a1 += S[4 * i4 + 1] * q4.y;
        a2 += S[4 * i4 + 2] * q4.z;
        a3 += S[4 * i4 + 3] * q4.w;
      }
      part[tt][g][c] = (a0 + a1) + (a2 + a3);
    }
    __syncthreads();
    for (int idx = t; idx < nt * COLS; idx += kThreads) {
      const int tt = idx / COLS, cc = idx % COLS;
      if (col0 + cc < DV) {
        float o = part[tt][0][cc];
#pragma unroll
        for (int gg = 1; gg < G; ++gg) o += part[tt][gg][cc];
        o_raw[static_cast<size_t>(row0 + tile0 + tt) * out_width + static_cast<size_t>(head) * DV +
              col0 + cc] = o;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = g * R + i;
    if (col_live && row < DK) s_out[static_cast<size_t>(row) * DV + col] = S[i];
  }
}

// act [N, width] float32 = silu(sum of the slices of the first `width` columns of proj's rows).
template <typename TI>
__global__ void la_activate_kernel(const TI* __restrict__ proj, int nsplit, size_t split_stride,
                                   size_t row_stride, float* __restrict__ act, size_t total,
                                   int width) {
  const size_t index = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const size_t row = index / width, col = index % width;
  act[index] = silu_f32(sliced(proj + row * row_stride + col, nsplit, split_stride));
}

// A block a row: out = o / sqrt(mean(o^2) + eps) * w * sigmoid(g), g the columns of the
// projection from `gate_at` on (the sum of its float32 slices).
template <typename TI, typename TO>
__global__ void la_out_kernel(const float* __restrict__ o_raw, const TI* __restrict__ proj, int nsplit,
                              size_t split_stride, size_t row_stride, size_t gate_at,
                              const float* __restrict__ norm_w, float eps,
                              const int32_t* __restrict__ row_seq, TO* __restrict__ out, int HV) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  if (row_seq && row_seq[row] < 0) return;      // a padding row
  const float* o = o_raw + static_cast<size_t>(row) * HV;
  float squares = 0.f;
  for (int i = threadIdx.x; i < HV; i += blockDim.x) squares += o[i] * o[i];
  const float inv = 1.0f / sqrtf(ei::block_sum(squares, scratch) / static_cast<float>(HV) + eps);
  const TI* gate = proj + static_cast<size_t>(row) * row_stride + gate_at;
  for (int i = threadIdx.x; i < HV; i += blockDim.x) {
    const float gv = sliced(gate + i, nsplit, split_stride);
    const float y = (o[i] * inv) * norm_w[i] / (1.0f + expf(-gv));
    out[static_cast<size_t>(row) * HV + i] = ei::from_f32<TO>(y);
  }
}

}  // namespace

// Floats of one sequence's state.
extern "C" long long ei_la_state_floats(int H, int DK, int DV) {
  return static_cast<long long>(H) * DK * DV;
}

// proj: [nsplit][N, row_stride] of proj_dtype, rows as above; state: float32 rows of
// H * DK * DV; o_raw: float32 [N, H * DV].
extern "C" int ei_la_scan(const void* proj, int proj_dtype, int nsplit, long long split_stride,
                          long long row_stride, const float* decay, float* state,
                          const int32_t* seq_in, const int32_t* seq_out, const int32_t* seq_count,
                          const int32_t* seq_row0, float* o_raw, int n_seqs, int H, int DK, int DV,
                          int activated, hipStream_t stream) {
  EI_REQUIRE(proj && decay && state && seq_in && seq_out && seq_count && seq_row0 && o_raw,
             "la_scan: null pointer");
  EI_REQUIRE(n_seqs > 0 && H > 0 && DK >= 1 && DK <= 256 && DV >= 1 && nsplit >= 1,
             "la_scan: key heads of 1 to 256 elements");
  EI_REQUIRE(row_stride >= 2LL * H * DK + 1LL * H * DV, "la_scan: rows narrower than q, k and v");
  EI_REQUIRE(H <= 65535 && (DV + 15) / 16 <= 65535, "la_scan: too many heads");
  // 64 columns a block where that fills the chip; 16 (and a quarter of the rows a thread)
  // where the sequences and heads are few, so that more blocks walk shorter chains
  const long long wide_blocks = 1LL * n_seqs * H * ((DV + 63) / 64);
  const bool narrow = wide_blocks < ei_compute_units();
  const int cols = narrow ? 16 : 64;
  const dim3 grid(n_seqs, H, (DV + cols - 1) / cols);
  const size_t ss = static_cast<size_t>(split_stride), rs = static_cast<size_t>(row_stride);
#define EI_LA(TI, R, COLS, AHEAD)                                                              \
  do {                                                                                         \
    if (activated)                                                                             \
      la_scan_kernel<TI, R, COLS, AHEAD, false><<<grid, kThreads, 0, stream>>>(                \
          static_cast<const TI*>(proj), nsplit, ss, rs, decay, state, state, seq_in, seq_out,  \
          seq_count, seq_row0, o_raw, H, DK, DV);                                              \
    else                                                                                       \
      la_scan_kernel<TI, R, COLS, AHEAD, true><<<grid, kThreads, 0, stream>>>(                 \
          static_cast<const TI*>(proj), nsplit, ss, rs, decay, state, state, seq_in, seq_out,  \
          seq_count, seq_row0, o_raw, H, DK, DV);                                              \
  } while (0)
#define EI_LA_T(TI)                                       \
  do {                                                    \
    if (narrow) {                                         \
      if (DK <= 64) EI_LA(TI, 4, 16, true);               \
      else if (DK <= 128) EI_LA(TI, 8, 16, true);         \
      else EI_LA(TI, 16, 16, true);                       \
    } else if (DK <= 32) EI_LA(TI, 8, 64, false);         \
    else if (DK <= 64) EI_LA(TI, 16, 64, false);          \
    else if (DK <= 128) EI_LA(TI, 32, 64, false);         \
    else EI_LA(TI, 64, 64, false);                        \
  } while (0)
  if (proj_dtype == EI_F32) EI_LA_T(float);
  else if (proj_dtype == EI_BF16) EI_LA_T(bf16_t);
  else EI_REQUIRE(false, "la_scan: unknown dtype");
#undef EI_LA_T
#undef EI_LA
  EI_LAUNCH_CHECK();
}

// act: float32 [N, width] = silu of the first `width` columns of proj's rows (q, k and v).
extern "C" int ei_la_activate(const void* proj, int proj_dtype, int nsplit, long long split_stride,
                              long long row_stride, float* act, int N, int width,
                              hipStream_t stream) {
  EI_REQUIRE(proj && act && N > 0 && width > 0 && nsplit >= 1 && row_stride >= width,
             "la_activate: bad arguments");
  const size_t total = static_cast<size_t>(N) * width;
  const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
  const size_t ss = static_cast<size_t>(split_stride), rs = static_cast<size_t>(row_stride);
  if (proj_dtype == EI_F32)
    la_activate_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(proj), nsplit, ss,
                                                          rs, act, total, width);
  else if (proj_dtype == EI_BF16)
    la_activate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(proj), nsplit,
                                                           ss, rs, act, total, width);
  else
    EI_REQUIRE(false, "la_activate: unknown dtype");
  EI_LAUNCH_CHECK();
}

extern "C" int ei_la_out(const float* o_raw, const void* proj, int proj_dtype, int nsplit,
                         long long split_stride, long long row_stride, long long gate_at,
                         const float* norm_w, float eps, const int32_t* row_seq, void* out,
                         int out_dtype, int N, int HV, hipStream_t stream) {
  EI_REQUIRE(o_raw && proj && norm_w && out && N > 0 && HV > 0 && nsplit >= 1, "la_out: bad arguments");
  EI_REQUIRE(row_stride >= gate_at + HV, "la_out: rows narrower than the gate's columns");
  const int threads = HV >= 2048 ? 512 : (HV >= 512 ? 256 : 128);
  const size_t ss = static_cast<size_t>(split_stride), rs = static_cast<size_t>(row_stride);
  const size_t ga = static_cast<size_t>(gate_at);
#define EI_LO(TI, TO)                                                                          \
  la_out_kernel<TI, TO><<<N, threads, 0, stream>>>(o_raw, static_cast<const TI*>(proj), nsplit, ss, \
                                                   rs, ga, norm_w, eps, row_seq,               \
                                                   static_cast<TO*>(out), HV)
  if (proj_dtype == EI_F32 && out_dtype == EI_F32) EI_LO(float, float);
  else if (proj_dtype == EI_F32 && out_dtype == EI_BF16) EI_LO(float, bf16_t);
  else if (proj_dtype == EI_BF16 && out_dtype == EI_BF16) EI_LO(bf16_t, bf16_t);
  else EI_REQUIRE(false, "la_out: unsupported dtype combination");
#undef EI_LO
  EI_LAUNCH_CHECK();
}

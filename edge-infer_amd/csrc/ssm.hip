// Selective state-space mixer with a scalar decay per head (Mamba-2): convolution, scan, read-out.
//
// A row of the input projection is [z: inner | xBC: inner + 2 G N | dt: heads] with
// inner = heads * P.  The xBC part passes a short causal convolution per channel (with a bias)
// and silu; then, per head h (group g = h / (heads / G)) and token t, all in float32:
//
//   dt_t = softplus(dt_t + dt_bias_h)         a_t = exp(-exp(A_log_h) dt_t)
//   S_t  = a_t S_{t-1} + dt_t B_t x_t^T       S is [N, P]
//   y_t  = S_t^T C_t + D_h x_t
//
// and y * silu(z), RMS-normed in `parts` equal parts of the row, times a weight.
//
// Per sequence the state row holds S of every head as [head][p][n] and then the last taps - 1
// inputs of every convolved channel, oldest first.  A step reads the row `seq_in` names and
// writes the whole row `seq_out` names, so a prompt may come whole, in portions or token by
// token, and a step that fails changes nothing.
#include "common.h"

namespace {

template <typename TI>
__device__ __forceinline__ float sliced(const TI* p, int nsplit, size_t split_stride) {
  float v = 0.f;
  for (int s = 0; s < nsplit; ++s) v += ei::to_f32<TI>(p[s * split_stride]);
  return v;
}

template <typename TI>
__device__ __forceinline__ void ssm_tail_element(const TI* proj, int nsplit, size_t split_stride,
                                                 size_t row_stride, int col0, float* state,
                                                 size_t state_stride, size_t tail_offset,
                                                 const int32_t* seq_in, const int32_t* seq_out,
                                                 const int32_t* seq_count, const int32_t* seq_row0,
                                                 int n_seqs, int C, int J, size_t idx);

// conv [N, C] float32 = silu(bias + sum_j w[c, j] * input(t - (J - 1) + j)); inputs before the
// step's first row come from the sequence's tail in the state.  A thread a (row, channel);
// the threads beyond those renew the tails (a thread a (sequence, tap, channel)): the new tail
// is written to another row of the state than the old one is read from.
template <typename TI>
__global__ void ssm_conv_kernel(const TI* __restrict__ proj, int nsplit, size_t split_stride,
                                size_t row_stride, int col0, const float* __restrict__ w,
                                const float* __restrict__ bias, const float* state,
                                size_t state_stride, size_t tail_offset,
                                const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_seq,
                                const int32_t* __restrict__ seq_in, const int32_t* __restrict__ seq_start,
                                float* __restrict__ conv, int N, int C, int J,
                                float* state_out, const int32_t* __restrict__ seq_out,
                                const int32_t* __restrict__ seq_count,
                                const int32_t* __restrict__ seq_row0, int n_seqs, unsigned conv_blocks) {
  if (blockIdx.x >= conv_blocks) {
    ssm_tail_element(proj, nsplit, split_stride, row_stride, col0, state_out, state_stride,
                     tail_offset, seq_in, seq_out, seq_count, seq_row0, n_seqs, C, J,
                     static_cast<size_t>(blockIdx.x - conv_blocks) * blockDim.x + threadIdx.x);
    return;
  }
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= static_cast<size_t>(N) * C) return;
  const int row = static_cast<int>(idx / C), c = static_cast<int>(idx % C);
  const int seq = row_seq[row];
  if (seq < 0) return;
  const int local = row_pos[row] - seq_start[seq];     // this row's index among the step's rows
  const float* tail = state + static_cast<size_t>(seq_in[seq]) * state_stride + tail_offset;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < J; ++j) {
    const int at = local - (J - 1) + j;
    float x;
    if (at >= 0)
      x = sliced(proj + static_cast<size_t>(row - local + at) * row_stride + col0 + c, nsplit, split_stride);
    else
      x = tail[static_cast<size_t>(J - 1 + at) * C + c];
    acc += w[static_cast<size_t>(c) * J + j] * x;
  }
  conv[idx] = acc / (1.0f + expf(-acc));
}

// The new tail of every sequence: its last J - 1 inputs, from the step's rows or, where the
// step brought fewer, from the old tail.  A thread a (sequence, tap, channel).
template <typename TI>
__device__ __forceinline__ void ssm_tail_element(const TI* proj, int nsplit, size_t split_stride,
                                                 size_t row_stride, int col0, float* state,
                                                 size_t state_stride, size_t tail_offset,
                                                 const int32_t* seq_in, const int32_t* seq_out,
                                                 const int32_t* seq_count, const int32_t* seq_row0,
                                                 int n_seqs, int C, int J, size_t idx) {
  const size_t per_seq = static_cast<size_t>(J - 1) * C;
  if (idx >= static_cast<size_t>(n_seqs) * per_seq) return;
  const int seq = static_cast<int>(idx / per_seq);
  const int j = static_cast<int>((idx % per_seq) / C), c = static_cast<int>(idx % C);
  const int count = seq_count[seq];
  if (count <= 0) return;
  const float* old_tail = state + static_cast<size_t>(seq_in[seq]) * state_stride + tail_offset;
  float* new_tail = state + static_cast<size_t>(seq_out[seq]) * state_stride + tail_offset;
  const int at = count - (J - 1) + j;
  float x;
  if (at >= 0)
    x = sliced(proj + static_cast<size_t>(seq_row0[seq] + at) * row_stride + col0 + c, nsplit, split_stride);
  else
    x = old_tail[static_cast<size_t>(j + count) * C + c];
  new_tail[static_cast<size_t>(j) * C + c] = x;
}

// Sum over the L neighbouring lanes (L a power of two, the group's first lane a multiple of L)
// that share a column, every lane getting it: DPP adds inside a row of 16 lanes, row swaps
// beyond; no step goes through LDS.
__device__ __forceinline__ float group_sum(float v, int L) {
  if (L >= 2) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xb1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  if (L >= 4) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4e, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  if (L >= 8) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // row_half_mirror
  if (L >= 16) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false)); // row_mirror
  if (L >= 32) {
    const ei::ei_u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r.x) + __uint_as_float(r.y);
  }
  if (L >= 64) {
    const ei::ei_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r.x) + __uint_as_float(r.y);
  }
  return v;
}

constexpr int kScanRows = 16;     // rows of S a thread owns
constexpr int kScanTile = 16;     // tokens staged through LDS at a time
constexpr int kScanThreads = 256;

// A block a (sequence, head, block of columns of S).  A thread owns kScanRows rows of one
// column; the L = Npad / kScanRows lanes of a column add their partial read-outs with DPP adds,
// and a token's operands are read from LDS while the token before it multiplies.
// AHEAD: the next tile's rows are asked for from global memory before this tile is walked
// (for launches of few blocks, where nothing else hides those reads; it costs registers, and
// with them waves a SIMD where the chip is full).
template <typename TI, bool AHEAD>
__global__ void __launch_bounds__(kScanThreads)
ssm_scan_kernel(const float* __restrict__ conv, const TI* __restrict__ proj, int nsplit,
                size_t split_stride, size_t row_stride, int dt_col0,
                const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                const float* __restrict__ d_skip, float* __restrict__ state, size_t state_stride,
                const int32_t* __restrict__ seq_in, const int32_t* __restrict__ seq_out,
                const int32_t* __restrict__ seq_count, const int32_t* __restrict__ seq_row0,
                float* __restrict__ y_raw, int heads, int groups, int P, int Nst, int L) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x, head = blockIdx.y;
  const int count = seq_count[seq];
  if (count <= 0) return;                       // padding: the whole block leaves together
  const int cols = kScanThreads / L;            // columns of S this block walks
  const int npad = L * kScanRows;
  const int tid = threadIdx.x;
  const int sub = tid % L, col_local = tid / L;
  const int col = blockIdx.z * cols + col_local;
  const bool live = col < P;
  const int n0 = sub * kScanRows;
  const int group = head / (heads / groups);
  const int inner = heads * P, C = inner + 2 * groups * Nst;
  float* xs = lds;                              // [tile][cols]
  float* bs = xs + kScanTile * cols;            // [tile][npad]
  float* cs = bs + kScanTile * npad;            // [tile][npad]
  float* dts = cs + kScanTile * npad;           // [tile]
  float* decays = dts + kScanTile;              // [tile]

  float S[kScanRows];
  const float* s_in = state + static_cast<size_t>(seq_in[seq]) * state_stride +
                      (static_cast<size_t>(head) * P + (live ? col : 0)) * Nst;
  float* s_out = state + static_cast<size_t>(seq_out[seq]) * state_stride +
                 (static_cast<size_t>(head) * P + (live ? col : 0)) * Nst;
  // (rows in 16-byte pieces where the state's rows and the head's columns begin on such)
  const bool pieces = Nst % 4 == 0 && state_stride % 4 == 0;
  if (pieces) {
#pragma unroll
    for (int r = 0; r < kScanRows; r += 4) {
      const float4 v = (live && n0 + r < Nst) ? *reinterpret_cast<const float4*>(s_in + n0 + r)
                                              : make_float4(0.f, 0.f, 0.f, 0.f);
      S[r] = v.x; S[r + 1] = v.y; S[r + 2] = v.z; S[r + 3] = v.w;
    }
  } else {
#pragma unroll
    for (int r = 0; r < kScanRows; ++r) S[r] = (live && n0 + r < Nst) ? s_in[n0 + r] : 0.f;
  }
  const float rate = expf(a_log[head]), bias = dt_bias[head], skip = d_skip[head];
  const int row0 = seq_row0[seq];

  // Where the sizes allow 16-byte pieces and a thread's share of a tile is at most four of them
  // an array, the next tile's rows are asked for from global memory before this tile is walked
  // and go to LDS after it: the walk, not the reads, is then what a tile takes.
  const int quads = npad / 4;                   // 16-byte pieces of a token's B (or C) in LDS
  constexpr bool ahead = AHEAD;      // (the host has checked the sizes)
  float4 pb[4], pc[4];
  float px[4], pz = 0.f;
  auto ask = [&](int t0n) {
    const int ntn = min(kScanTile, count - t0n);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = tid + u * kScanThreads;
      pb[u] = pc[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < ntn * quads) {
        const int t = i / quads, n = (i % quads) * 4;
        const float* src = conv + static_cast<size_t>(row0 + t0n + t) * C + inner + group * Nst;
        if (n < Nst) {
          pb[u] = *reinterpret_cast<const float4*>(src + n);
          pc[u] = *reinterpret_cast<const float4*>(src + groups * Nst + n);
        }
      }
      px[u] = 0.f;
      if (i < ntn * cols) {
        const int t = i / cols, c = blockIdx.z * cols + i % cols;
        if (c < P) px[u] = conv[static_cast<size_t>(row0 + t0n + t) * C + head * P + c];
      }
    }
    if (tid < ntn)
      pz = sliced(proj + static_cast<size_t>(row0 + t0n + tid) * row_stride + dt_col0 + head, nsplit,
                  split_stride);
  };
  auto put = [&](int ntc) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = tid + u * kScanThreads;
      if (i < ntc * quads) {
        *reinterpret_cast<float4*>(bs + 4 * i) = pb[u];
        *reinterpret_cast<float4*>(cs + 4 * i) = pc[u];
      }
      if (i < ntc * cols) xs[i] = px[u];
    }
    if (tid < ntc) {
      const float z = pz + bias;
      const float dt = z > 20.f ? z : log1pf(expf(z));
      dts[tid] = dt;
      decays[tid] = expf(-rate * dt);
    }
  };
  if constexpr (ahead) ask(0);

  for (int t0 = 0; t0 < count; t0 += kScanTile) {
    const int nt = min(kScanTile, count - t0);
    __syncthreads();
    if constexpr (ahead) {
      put(nt);
      if (t0 + kScanTile < count) ask(t0 + kScanTile);
    } else {
      for (int i = tid; i < nt * cols; i += kScanThreads) {
        const int t = i / cols, cl = i % cols, c = blockIdx.z * cols + cl;
        xs[i] = c < P ? conv[static_cast<size_t>(row0 + t0 + t) * C + head * P + c] : 0.f;
      }
      for (int i = tid; i < nt * npad; i += kScanThreads) {
        const int t = i / npad, n = i % npad;
        const float* src = conv + static_cast<size_t>(row0 + t0 + t) * C + inner + group * Nst;
        bs[i] = n < Nst ? src[n] : 0.f;
        cs[i] = n < Nst ? src[groups * Nst + n] : 0.f;
      }
      if (tid < nt) {
        const float z = sliced(proj + static_cast<size_t>(row0 + t0 + tid) * row_stride + dt_col0 + head,
                               nsplit, split_stride) + bias;
        const float dt = z > 20.f ? z : log1pf(expf(z));
        dts[tid] = dt;
        decays[tid] = expf(-rate * dt);
      }
    }
    __syncthreads();
    // Two sets of a token's operands take turns: the LDS reads of the next token are asked
    // for before this one multiplies, so a token waits for no read of its own.
    float4 b0[4], c0[4], b1[4], c1[4];
    float decay0, xdt0, x0, decay1, xdt1, x1;
    auto fetch = [&](int t, float4 (&b4)[4], float4 (&c4)[4], float& decay, float& xdt, float& xv) {
      const int tt = min(t, nt - 1);               // (a token beyond the tile: read, never used)
      const float* bp = bs + tt * npad + n0;
      const float* cp = cs + tt * npad + n0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        b4[i] = *reinterpret_cast<const float4*>(bp + 4 * i);
        c4[i] = *reinterpret_cast<const float4*>(cp + 4 * i);
      }
      decay = decays[tt];
      xv = xs[tt * cols + col_local];
      xdt = xv * dts[tt];
    };
    auto step = [&](int t, const float4 (&b4)[4], const float4 (&c4)[4], float decay, float xdt, float xv) {
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;   // four sums: no single chain of additions
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        S[4 * i] = decay * S[4 * i] + b4[i].x * xdt;
        S[4 * i + 1] = decay * S[4 * i + 1] + b4[i].y * xdt;
        S[4 * i + 2] = decay * S[4 * i + 2] + b4[i].z * xdt;
        S[4 * i + 3] = decay * S[4 * i + 3] + b4[i].w * xdt;
        a0 += S[4 * i] * c4[i].x;
        a1 += S[4 * i + 1] * c4[i].y;
        a2 += S[4 * i + 2] * c4[i].z;
        a3 += S[4 * i + 3] * c4[i].w;
      }
      const float total = group_sum((a0 + a1) + (a2 + a3), L);
      if (live && sub == 0)
        y_raw[static_cast<size_t>(row0 + t0 + t) * inner + head * P + col] = total + skip * xv;
    };
    static_assert(kScanRows == 16, "the walk takes a thread's rows as four 16-byte pieces");
    fetch(0, b0, c0, decay0, xdt0, x0);
#pragma unroll 1
    for (int t = 0; t < nt; t += 2) {
      fetch(t + 1, b1, c1, decay1, xdt1, x1);
      step(t, b0, c0, decay0, xdt0, x0);
      fetch(t + 2, b0, c0, decay0, xdt0, x0);
      if (t + 1 < nt) step(t + 1, b1, c1, decay1, xdt1, x1);
    }
  }
  if (live) {
    if (pieces) {
#pragma unroll
      for (int r = 0; r < kScanRows; r += 4)
        if (n0 + r < Nst)
          *reinterpret_cast<float4*>(s_out + n0 + r) = make_float4(S[r], S[r + 1], S[r + 2], S[r + 3]);
    } else {
#pragma unroll
      for (int r = 0; r < kScanRows; ++r)
        if (n0 + r < Nst) s_out[n0 + r] = S[r];
    }
  }
}

// out = rmsnorm_per_part(y * silu(z)) * weight.  A wave a (row, part).
template <typename TI, typename TO>
__global__ void ssm_out_kernel(const float* __restrict__ y_raw, const TI* __restrict__ proj, int nsplit,
                               size_t split_stride, size_t row_stride, const float* __restrict__ weight,
                               float eps, const int32_t* __restrict__ row_seq, TO* __restrict__ out,
                               int N, int inner, int parts) {
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= N * parts) return;
  const int row = wave / parts, part = wave % parts;
  if (row_seq[row] < 0) return;
  const int width = inner / parts, first = part * width;
  const float* y = y_raw + static_cast<size_t>(row) * inner + first;
  const TI* z = proj + static_cast<size_t>(row) * row_stride + first;
  float sum = 0.f;
  for (int e = lane; e < width; e += EI_WAVE) {
    const float g = sliced(z + e, nsplit, split_stride);
    const float v = y[e] * (g / (1.0f + expf(-g)));
    sum += v * v;
  }
  const float inv = 1.0f / sqrtf(ei::wave_sum(sum) / static_cast<float>(width) + eps);
  TO* dst = out + static_cast<size_t>(row) * inner + first;
  for (int e = lane; e < width; e += EI_WAVE) {
    const float g = sliced(z + e, nsplit, split_stride);
    const float v = y[e] * (g / (1.0f + expf(-g)));
    dst[e] = ei::from_f32<TO>((v * inv) * weight[first + e]);
  }
}

inline int scan_lanes(int Nst) {
  int L = 1;
  while (L * kScanRows < Nst) L *= 2;
  return L;
}

}  // namespace

// Floats of a sequence's state row: S of every head, then the convolution's tail.
extern "C" int ei_ssm_state_floats(int heads, int groups, int P, int Nst, int taps) {
  return heads * P * Nst + (taps - 1) * (heads * P + 2 * groups * Nst);
}

#define EI_SSM_SHAPE(what)                                                                        \
  EI_REQUIRE(heads > 0 && groups > 0 && heads % groups == 0 && P > 0 && Nst > 0 && taps >= 1 &&   \
                 taps <= 64 && Nst <= 64 * kScanRows,                                             \
             what ": sizes outside what the kernels take");                                      \
  const int inner = heads * P, C = inner + 2 * groups * Nst;                                      \
  const size_t tail_offset = static_cast<size_t>(inner) * Nst;                                    \
  EI_REQUIRE(row_stride >= 2LL * inner + 2LL * groups * Nst + heads, what ": rows narrower than the projection"); \
  (void)C; (void)tail_offset

extern "C" int ei_ssm_conv(const void* proj, int in_dtype, int nsplit, long long split_stride,
                           long long row_stride, const float* w, const float* bias, float* state,
                           long long state_stride, const int32_t* row_pos, const int32_t* row_seq,
                           const int32_t* seq_in, const int32_t* seq_out, const int32_t* seq_start,
                           const int32_t* seq_count, const int32_t* seq_row0, float* conv, int N,
                           int n_seqs, int heads, int groups, int P, int Nst, int taps,
                           hipStream_t stream) {
  EI_SSM_SHAPE("ssm_conv");
  EI_REQUIRE(proj && w && state && row_pos && row_seq && seq_in && seq_out && seq_start && seq_count &&
                 seq_row0 && conv && N > 0 && n_seqs > 0 && nsplit >= 1,
             "ssm_conv: bad arguments");
  const int threads = 256;
  const size_t total = static_cast<size_t>(N) * C;
  const unsigned blocks = static_cast<unsigned>((total + threads - 1) / threads);
  const size_t tails = static_cast<size_t>(n_seqs) * (taps - 1) * C;
  const unsigned tail_blocks = static_cast<unsigned>((tails + threads - 1) / threads);
  const size_t ss = static_cast<size_t>(split_stride), rs = static_cast<size_t>(row_stride);
  const size_t st = static_cast<size_t>(state_stride);
#define EI_SSM_CONV(TI)                                                                          \
  ssm_conv_kernel<TI><<<blocks + (taps > 1 ? tail_blocks : 0), threads, 0, stream>>>(            \
      static_cast<const TI*>(proj), nsplit, ss, rs, inner, w, bias, state, st, tail_offset,      \
      row_pos, row_seq, seq_in, seq_start, conv, N, C, taps, state, seq_out, seq_count,          \
      seq_row0, n_seqs, blocks)
  if (in_dtype == EI_F32) EI_SSM_CONV(float);
  else if (in_dtype == EI_BF16) EI_SSM_CONV(bf16_t);
  else EI_REQUIRE(false, "ssm_conv: unknown dtype");
#undef EI_SSM_CONV
  EI_LAUNCH_CHECK();
}

extern "C" int ei_ssm_scan(const float* conv, const void* proj, int in_dtype, int nsplit,
                           long long split_stride, long long row_stride, const float* a_log,
                           const float* dt_bias, const float* d_skip, float* state,
                           long long state_stride, const int32_t* seq_in, const int32_t* seq_out,
                           const int32_t* seq_count, const int32_t* seq_row0, float* y_raw,
                           int n_seqs, int heads, int groups, int P, int Nst, int taps,
                           hipStream_t stream) {
  EI_SSM_SHAPE("ssm_scan");
  EI_REQUIRE(conv && proj && a_log && dt_bias && d_skip && state && seq_in && seq_out && seq_count &&
                 seq_row0 && y_raw && n_seqs > 0 && nsplit >= 1,
             "ssm_scan: bad arguments");
  EI_REQUIRE(heads <= 65535, "ssm_scan: too many heads for one launch");
  const int L = scan_lanes(Nst);
  const int cols = kScanThreads / L;
  const int npad = L * kScanRows;
  const size_t lds = sizeof(float) * (static_cast<size_t>(kScanTile) * (cols + 2 * npad) + 2 * kScanTile);
  const dim3 grid(n_seqs, heads, (P + cols - 1) / cols);
  const size_t ss = static_cast<size_t>(split_stride), rs = static_cast<size_t>(row_stride);
  const int dt_col0 = inner + C;
  // rows asked for a tile ahead: 16-byte pieces, at most four of them an array and thread, and a
  // launch of so few blocks that a compute unit holds at most one (measured at 64, 512 and
  // 4,096 blocks: 1,076 -> 790, 306 -> 334 and 1,760 -> 2,640 us)
  const bool ahead = L >= 4 && L <= 16 && Nst % 4 == 0 && inner % 4 == 0 && (groups * Nst) % 4 == 0 &&
                     static_cast<long long>(grid.x) * grid.y * grid.z <= 1LL * ei_compute_units();
#define EI_SSM_SCAN(TI)                                                                           \
  do {                                                                                            \
    if (ahead) EI_SSM_SCAN_AS(TI, true);                                                          \
    else EI_SSM_SCAN_AS(TI, false);                                                               \
  } while (0)
#define EI_SSM_SCAN_AS(TI, AHEAD)                                                                 \
  do {                                                                                            \
    if (lds > 48 * 1024)                                                                          \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&ssm_scan_kernel<TI, AHEAD>),       \
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
    ssm_scan_kernel<TI, AHEAD><<<grid, kScanThreads, lds, stream>>>(                              \
        conv, static_cast<const TI*>(proj), nsplit, ss, rs, dt_col0, a_log, dt_bias, d_skip,      \
        state, static_cast<size_t>(state_stride), seq_in, seq_out, seq_count, seq_row0, y_raw,    \
        heads, groups, P, Nst, L);                                                                \
  } while (0)
  if (in_dtype == EI_F32) EI_SSM_SCAN(float);
  else if (in_dtype == EI_BF16) EI_SSM_SCAN(bf16_t);
  else EI_REQUIRE(false, "ssm_scan: unknown dtype");
#undef EI_SSM_SCAN
#undef EI_SSM_SCAN_AS
  EI_LAUNCH_CHECK();
}

extern "C" int ei_ssm_out(const float* y_raw, const void* proj, int in_dtype, int nsplit,
                          long long split_stride, long long row_stride, const float* weight,
                          float eps, const int32_t* row_seq, void* out, int out_dtype, int N,
                          int inner, int parts, hipStream_t stream) {
  EI_REQUIRE(y_raw && proj && weight && row_seq && out && N > 0 && inner > 0 && parts > 0 &&
                 inner % parts == 0 && nsplit >= 1 && row_stride >= inner,
             "ssm_out: bad arguments");
  const int threads = 256;
  const size_t waves = static_cast<size_t>(N) * parts;
  const unsigned blocks = static_cast<unsigned>((waves * EI_WAVE + threads - 1) / threads);
  const size_t ss = static_cast<size_t>(split_stride), rs = static_cast<size_t>(row_stride);
#define EI_SSM_OUT(TI, TO)                                                                    \
  ssm_out_kernel<TI, TO><<<blocks, threads, 0, stream>>>(                                     \
      y_raw, static_cast<const TI*>(proj), nsplit, ss, rs, weight, eps, row_seq,              \
      static_cast<TO*>(out), N, inner, parts)
  if (in_dtype == EI_F32 && out_dtype == EI_F32) EI_SSM_OUT(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16) EI_SSM_OUT(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16) EI_SSM_OUT(bf16_t, bf16_t);
  else EI_REQUIRE(false, "ssm_out: unsupported dtype combination");
#undef EI_SSM_OUT
  EI_LAUNCH_CHECK();
}

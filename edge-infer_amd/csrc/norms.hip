// Norms with a mean and a bias, in the three places a block arrangement puts a norm, and the
// join of mixers that run side by side.  Everything is float32: sums, means, variances, the
// stream; a result is rounded once to the output type.
//
// norm(x) = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b   (`centred`, b may be null)
//         =  x / sqrt(mean(x^2) + eps) * w                         (not centred)
#include "common.h"

namespace {

// mean and 1 / sqrt(variance + eps) of the H values a block holds in `values` (LDS).
__device__ __forceinline__ void row_moments(const float* values, int H, int centred, float eps,
                                            float* scratch, float& mean, float& inv) {
  mean = 0.f;
  if (centred) {
    float sum = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) sum += values[i];
    mean = ei::block_sum(sum, scratch) / static_cast<float>(H);
  }
  float squares = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float d = values[i] - mean;
    squares += d * d;
  }
  inv = 1.0f / sqrtf(ei::block_sum(squares, scratch) / static_cast<float>(H) + eps);
}

// One block per output row; src = rows ? rows[row] : row (negative: a padding row, whose output
// is zero).  With d = sum over slices of delta[src] (+ delta_bias):
//   w_after:  d <- norm(d; w_after, b_after)         (the norm on a sublayer's output)
//   y = residual[src] + d (stored back if `write_residual`); without delta, y = residual[src]
//   out:      out[row] = norm(y; w_next, b_next)      (the next sublayer's input norm)
template <typename TD, typename TO>
__global__ void stream_norm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                   int nsplit, size_t split_stride,
                                   const float* __restrict__ delta_bias,
                                   const int32_t* __restrict__ rows,
                                   const float* __restrict__ w_after,
                                   const float* __restrict__ b_after,
                                   const float* __restrict__ w_next,
                                   const float* __restrict__ b_next, float eps, int centred,
                                   TO* __restrict__ out, int H, int write_residual) {
  extern __shared__ float values[];
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  if (src < 0) {
    if (out)
      for (int i = threadIdx.x; i < H; i += blockDim.x)
        out[static_cast<size_t>(row) * H + i] = ei::from_f32<TO>(0.f);
    return;
  }
  float* res = residual + static_cast<size_t>(src) * H;
  if (delta) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const TD* d = delta + static_cast<size_t>(src) * H + i;
      float x = 0.f;
      for (int s = 0; s < nsplit; ++s) x += ei::to_f32<TD>(d[s * split_stride]);
      if (delta_bias) x += delta_bias[i];
      values[i] = x;
    }
    if (w_after) {
      __syncthreads();
      float mean, inv;
      row_moments(values, H, centred, eps, scratch, mean, inv);
      for (int i = threadIdx.x; i < H; i += blockDim.x)
        values[i] = ((values[i] - mean) * inv) * w_after[i] + (b_after ? b_after[i] : 0.f);
    }
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float y = res[i] + values[i];
      values[i] = y;
      if (write_residual) res[i] = y;
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) values[i] = res[i];
  }
  if (!out) return;
  __syncthreads();
  float mean, inv;
  row_moments(values, H, centred, eps, scratch, mean, inv);
  TO* dst = out + static_cast<size_t>(row) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    dst[i] = ei::from_f32<TO>(((values[i] - mean) * inv) * w_next[i] + (b_next ? b_next[i] : 0.f));
}

using ei::Vec4;

// The short causal convolution of a step in which every sequence brings one token (a decode
// step: row r is sequence r), taken in by the norm kernel that makes the convolution's input:
// with h the normed row as it is stored, out = h + sum_j w[j] x_j, x_j the last taps - 1 inputs
// of the sequence (its state, part `part` of row seq_in[r] of a table with two versions) and,
// for the last tap, h itself; the state row seq_out[r] receives the inputs moved on by one.
// w null: no convolution.  The sums are taken in the order of the kernel that convolves a
// step's rows on its own, so a token gives the same values either way.
struct ConvTail {
  const float* w;          // [taps, H]
  const float* state;      // rows of parts * (taps - 1) * H floats
  float* state_out;        // (the same table)
  const int32_t* seq_in;
  const int32_t* seq_out;
  int taps, part, parts;
};

// Four neighbouring elements of a row as the sum of its slices, in slice order; eight loads are
// issued before the first sum, so that a row costs one trip to memory per eight slices.
template <typename TD>
__device__ __forceinline__ void sliced4(const TD* p, int nsplit, size_t split_stride, float (&x)[4]) {
  x[0] = x[1] = x[2] = x[3] = 0.f;
  for (int s0 = 0; s0 < nsplit; s0 += 8) {
    float v[8][4];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + u < nsplit) Vec4<TD>::load(p + (s0 + u) * split_stride, v[u]);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + u < nsplit) {
#pragma unroll
        for (int i = 0; i < 4; ++i) x[i] += v[u][i];
      }
  }
}

// mean and 1 / sqrt(variance + eps) of a row that the block's threads hold in registers
// (CHUNKS quads a thread; quads beyond the row hold zeros and are told by `live`).
template <int CHUNKS>
__device__ __forceinline__ void held_moments(const float (&x)[CHUNKS][4], const bool (&live)[CHUNKS],
                                             int H, int centred, float eps, float* scratch,
                                             float& mean, float& inv) {
  mean = 0.f;
  if (centred) {
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k)
      if (live[k]) sum += (x[k][0] + x[k][1]) + (x[k][2] + x[k][3]);
    mean = ei::block_sum(sum, scratch) / static_cast<float>(H);
  }
  float squares = 0.f;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k)
    if (live[k]) {
#pragma unroll
      for (int i = 0; i < 4; ++i) squares += (x[k][i] - mean) * (x[k][i] - mean);
    }
  inv = 1.0f / sqrtf(ei::block_sum(squares, scratch) / static_cast<float>(H) + eps);
}

// stream_norm_kernel for widths that are a multiple of 4: 16-byte accesses, the row kept in
// registers, up to 1024 threads a row so that few rows still have many loads in flight.
template <typename TD, typename TO, int CHUNKS>
__global__ void stream_norm_vec_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                       int nsplit, size_t split_stride,
                                       const float* __restrict__ delta_bias,
                                       const int32_t* __restrict__ rows,
                                       const float* __restrict__ w_after,
                                       const float* __restrict__ b_after,
                                       const float* __restrict__ w_next,
                                       const float* __restrict__ b_next, float eps, int centred,
                                       TO* __restrict__ out, int H, int write_residual,
                                       ConvTail conv) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  const int quads = H / 4;
  if (src < 0) {
    if (out) {
      const float zero[4] = {0.f, 0.f, 0.f, 0.f};
      for (int qd = threadIdx.x; qd < quads; qd += blockDim.x)
        Vec4<TO>::store(out + static_cast<size_t>(row) * H + qd * 4, zero);
    }
    return;
  }
  float* res = residual + static_cast<size_t>(src) * H;
  bool live[CHUNKS];
  float y[CHUNKS][4];
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    live[k] = qd < quads;
    y[k][0] = y[k][1] = y[k][2] = y[k][3] = 0.f;
    if (live[k]) Vec4<float>::load(res + qd * 4, y[k]);
  }
  if (delta) {
    float x[CHUNKS][4];
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
      const int qd = threadIdx.x + k * blockDim.x;
      x[k][0] = x[k][1] = x[k][2] = x[k][3] = 0.f;
      if (live[k]) {
        sliced4(delta + static_cast<size_t>(src) * H + qd * 4, nsplit, split_stride, x[k]);
        if (delta_bias) {
          float b[4];
          Vec4<float>::load(delta_bias + qd * 4, b);
#pragma unroll
          for (int i = 0; i < 4; ++i) x[k][i] += b[i];
        }
      }
    }
    if (w_after) {
      float mean, inv;
      held_moments<CHUNKS>(x, live, H, centred, eps, scratch, mean, inv);
#pragma unroll
      for (int k = 0; k < CHUNKS; ++k) {
        const int qd = threadIdx.x + k * blockDim.x;
        if (live[k]) {
          float w[4], b[4] = {0.f, 0.f, 0.f, 0.f};
          Vec4<float>::load(w_after + qd * 4, w);
          if (b_after) Vec4<float>::load(b_after + qd * 4, b);
#pragma unroll
          for (int i = 0; i < 4; ++i) x[k][i] = ((x[k][i] - mean) * inv) * w[i] + b[i];
        }
      }
    }
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
      const int qd = threadIdx.x + k * blockDim.x;
      if (live[k]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) y[k][i] += x[k][i];
        if (write_residual) Vec4<float>::store(res + qd * 4, y[k]);
      }
    }
  }
  if (!out) return;
  float mean, inv;
  held_moments<CHUNKS>(y, live, H, centred, eps, scratch, mean, inv);
  TO* dst = out + static_cast<size_t>(row) * H;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (live[k]) {
      float w[4], b[4] = {0.f, 0.f, 0.f, 0.f}, z[4];
      Vec4<float>::load(w_next + qd * 4, w);
      if (b_next) Vec4<float>::load(b_next + qd * 4, b);
#pragma unroll
      for (int i = 0; i < 4; ++i) z[i] = ((y[k][i] - mean) * inv) * w[i] + b[i];
      if (conv.w) {
        // the row as the next kernel would have read it, then its taps
        float h[4], acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = h[i] = ei::to_f32<TO>(ei::from_f32<TO>(z[i]));
        const int tail = conv.taps - 1;
        const size_t row_floats = static_cast<size_t>(conv.parts) * tail * H;
        const size_t at = static_cast<size_t>(conv.part) * tail * H + qd * 4;
        const float* old = nullptr;
        float* renewed = nullptr;
        if (tail > 0) {
          old = conv.state + static_cast<size_t>(conv.seq_in[row]) * row_floats + at;
          renewed = conv.state_out + static_cast<size_t>(conv.seq_out[row]) * row_floats + at;
        }
        for (int j = 0; j < tail; ++j) {
          float x[4], wj[4];
          Vec4<float>::load(old + static_cast<size_t>(j) * H, x);
          Vec4<float>::load(conv.w + static_cast<size_t>(j) * H + qd * 4, wj);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] += wj[i] * x[i];
          if (j > 0) Vec4<float>::store(renewed + static_cast<size_t>(j - 1) * H, x);
        }
        float wl[4];
        Vec4<float>::load(conv.w + static_cast<size_t>(tail) * H + qd * 4, wl);
#pragma unroll
        for (int i = 0; i < 4; ++i) z[i] = acc[i] + wl[i] * h[i];
        if (tail > 0) Vec4<float>::store(renewed + static_cast<size_t>(tail - 1) * H, h);
      }
      Vec4<TO>::store(dst + qd * 4, z);
    }
  }
}

constexpr int kMaxBranches = 4;

struct Branches {
  const void* rows[kMaxBranches];
  const float* weight[kMaxBranches];
  int nsplit[kMaxBranches];
  long long split_stride[kMaxBranches];
  int dtype[kMaxBranches];
};

// out[row] = (1 / n) sum over branches b of rmsnorm(sum of the slices of x_b[row]) * w_b.
__global__ void norm_mean_kernel(Branches branches, int n, float eps, float* __restrict__ out,
                                 int H) {
  extern __shared__ float values[];      // [2][H]: the branch at hand, the running sum
  __shared__ float scratch[16];
  float* current = values;
  float* total = values + H;
  const size_t base = static_cast<size_t>(blockIdx.x) * H;
  for (int b = 0; b < n; ++b) {
    const bool narrow = branches.dtype[b] == EI_BF16;
    const float* x32 = static_cast<const float*>(branches.rows[b]) + base;
    const bf16_t* x16 = static_cast<const bf16_t*>(branches.rows[b]) + base;
    float squares = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      float v = 0.f;
      for (int s = 0; s < branches.nsplit[b]; ++s) {
        const size_t at = static_cast<size_t>(s) * branches.split_stride[b] + i;
        v += narrow ? ei::bf16_to_f32(x16[at]) : x32[at];
      }
      current[i] = v;
      squares += v * v;
    }
    const float inv = 1.0f / sqrtf(ei::block_sum(squares, scratch) / static_cast<float>(H) + eps);
    const float* w = branches.weight[b];
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float y = (current[i] * inv) * w[i];
      total[i] = b == 0 ? y : total[i] + y;
    }
  }
  const float share = 1.0f / static_cast<float>(n);
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[base + i] = total[i] * share;
}

// norm_mean_kernel for widths that are a multiple of 4 (and slices that lie a multiple of 4
// apart): 16-byte accesses, rows and running sums kept in registers.
template <int CHUNKS>
__global__ void norm_mean_vec_kernel(Branches branches, int n, float eps, float* __restrict__ out,
                                     int H) {
  __shared__ float scratch[16];
  const size_t base = static_cast<size_t>(blockIdx.x) * H;
  const int quads = H / 4;
  float total[CHUNKS][4];
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) total[k][0] = total[k][1] = total[k][2] = total[k][3] = 0.f;
  for (int b = 0; b < n; ++b) {
    const bool narrow = branches.dtype[b] == EI_BF16;
    const size_t stride = static_cast<size_t>(branches.split_stride[b]);
    float x[CHUNKS][4];
    float squares = 0.f;
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
      const int qd = threadIdx.x + k * blockDim.x;
      x[k][0] = x[k][1] = x[k][2] = x[k][3] = 0.f;
      if (qd < quads) {
        if (narrow)
          sliced4(static_cast<const bf16_t*>(branches.rows[b]) + base + qd * 4, branches.nsplit[b],
                  stride, x[k]);
        else
          sliced4(static_cast<const float*>(branches.rows[b]) + base + qd * 4, branches.nsplit[b],
                  stride, x[k]);
#pragma unroll
        for (int i = 0; i < 4; ++i) squares += x[k][i] * x[k][i];
      }
    }
    const float inv = 1.0f / sqrtf(ei::block_sum(squares, scratch) / static_cast<float>(H) + eps);
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
      const int qd = threadIdx.x + k * blockDim.x;
      if (qd < quads) {
        float w[4];
        Vec4<float>::load(branches.weight[b] + qd * 4, w);
#pragma unroll
        for (int i = 0; i < 4; ++i) total[k][i] += (x[k][i] * inv) * w[i];
      }
    }
  }
  const float share = 1.0f / static_cast<float>(n);
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) {
#pragma unroll
      for (int i = 0; i < 4; ++i) total[k][i] *= share;
      Vec4<float>::store(out + base + qd * 4, total[k]);
    }
  }
}

// Threads a row of the register-held forms: up to 1024 for few rows, so that many loads are in
// flight; 256 for many rows, so that several rows share a compute unit.
int vec_threads(int N, int quads) {
  const int most = N >= 512 && quads <= 4 * 256 ? 256 : 1024;
  int threads = (quads + EI_WAVE - 1) / EI_WAVE * EI_WAVE;
  return threads > most ? most : threads;
}

int row_threads(int H) { return H >= 4096 ? 512 : (H >= 1024 ? 256 : (H >= 256 ? 128 : 64)); }

}  // namespace

// residual [*, H] float32; delta [nsplit][*, H] of delta_dtype or null; rows null or int32 [N];
// w_after / b_after null: the delta is added as it is; out null: nothing is normed for a
// reader.  centred 1: norms with a mean (and the biases, where given); 0: RMS norms.
extern "C" int ei_stream_norm(float* residual, const void* delta, int delta_dtype, int nsplit,
                              long long split_stride, const float* delta_bias,
                              const int32_t* rows, const float* w_after, const float* b_after,
                              const float* w_next, const float* b_next, float eps, int centred,
                              void* out, int out_dtype, int N, int H, int write_residual,
                              const float* conv_w, float* conv_state, const int32_t* seq_in,
                              const int32_t* seq_out, int taps, int part, int parts,
                              hipStream_t stream) {
  EI_REQUIRE(N > 0 && H > 0, "stream_norm: sizes must be positive");
  const ConvTail conv{conv_w, conv_state, conv_state, seq_in, seq_out, taps, part, parts};
  EI_REQUIRE(!conv_w || (out && !rows && taps >= 1 && taps <= 64 && parts >= 1 && part >= 0 &&
                         part < parts && (taps == 1 || (conv_state && seq_in && seq_out)) &&
                         H % 4 == 0 && (!delta || split_stride % 4 == 0) && H <= 16384),
             "stream_norm: the convolution of a decode step needs rows that are sequences, its "
             "state and a width that is a multiple of 4");
  EI_REQUIRE(residual, "stream_norm: null pointer");
  EI_REQUIRE(!delta || nsplit >= 1, "stream_norm: nsplit must be at least 1");
  EI_REQUIRE(delta || !w_after, "stream_norm: a norm on a sublayer's output needs that output");
  EI_REQUIRE((out != nullptr) == (w_next != nullptr), "stream_norm: an output needs its norm's weight");
  EI_REQUIRE(eps > 0.f, "stream_norm: eps must be positive");
  EI_REQUIRE(static_cast<size_t>(H) * sizeof(float) <= 64 * 1024, "stream_norm: row too wide");
  const int threads = row_threads(H);
  const size_t lds = static_cast<size_t>(H) * sizeof(float);
  const size_t ss = static_cast<size_t>(split_stride);
  if (!delta) delta_dtype = EI_F32;
  if (!out) out_dtype = EI_F32;
  const bool vec = H % 4 == 0 && (!delta || ss % 4 == 0) && H <= 16384;
  const int vthreads = vec_threads(N, H / 4);
  const int chunks = vec ? (H / 4 + vthreads - 1) / vthreads : 0;      // 1..4
#define EI_SN_VEC(TD, TO, C)                                                                   \
  stream_norm_vec_kernel<TD, TO, C><<<N, vthreads, 0, stream>>>(                               \
      residual, static_cast<const TD*>(delta), nsplit, ss, delta_bias, rows, w_after, b_after, \
      w_next, b_next, eps, centred, static_cast<TO*>(out), H, write_residual, conv)
#define EI_SN(TD, TO)                                                                          \
  do {                                                                                         \
    if (chunks == 1) EI_SN_VEC(TD, TO, 1);                                                     \
    else if (chunks == 2) EI_SN_VEC(TD, TO, 2);                                                \
    else if (chunks == 3 || chunks == 4) EI_SN_VEC(TD, TO, 4);                                 \
    else                                                                                       \
      stream_norm_kernel<TD, TO><<<N, threads, lds, stream>>>(                                 \
          residual, static_cast<const TD*>(delta), nsplit, ss, delta_bias, rows, w_after,      \
          b_after, w_next, b_next, eps, centred, static_cast<TO*>(out), H, write_residual);    \
  } while (0)
  if (delta_dtype == EI_F32 && out_dtype == EI_F32) EI_SN(float, float);
  else if (delta_dtype == EI_F32 && out_dtype == EI_BF16) EI_SN(float, bf16_t);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_BF16) EI_SN(bf16_t, bf16_t);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_F32) EI_SN(bf16_t, float);
  else EI_REQUIRE(false, "stream_norm: unknown dtype");
#undef EI_SN
#undef EI_SN_VEC
  EI_LAUNCH_CHECK();
}

// out [N, H] float32 = mean over the n branches of rmsnorm(x_b) * w_b; x_b [nsplit_b][N, H] of
// the type dtype[b].
extern "C" int ei_norm_mean(const void* const* x, const int* nsplit, const long long* split_stride,
                            const int* dtype, const float* const* weight, int n, float eps,
                            float* out, int N, int H, hipStream_t stream) {
  EI_REQUIRE(n >= 1 && n <= kMaxBranches, "norm_mean: 1 to 4 branches");
  EI_REQUIRE(x && nsplit && split_stride && dtype && weight && out && N > 0 && H > 0,
             "norm_mean: bad arguments");
  EI_REQUIRE(static_cast<size_t>(H) * 2 * sizeof(float) <= 64 * 1024, "norm_mean: row too wide");
  Branches branches;
  for (int b = 0; b < kMaxBranches; ++b) {
    branches.rows[b] = b < n ? x[b] : nullptr;
    branches.weight[b] = b < n ? weight[b] : nullptr;
    branches.nsplit[b] = b < n ? nsplit[b] : 0;
    branches.split_stride[b] = b < n ? split_stride[b] : 0;
    branches.dtype[b] = b < n ? dtype[b] : EI_F32;
    EI_REQUIRE(b >= n || (x[b] && weight[b] && nsplit[b] >= 1), "norm_mean: null pointer");
    EI_REQUIRE(b >= n || dtype[b] == EI_F32 || dtype[b] == EI_BF16, "norm_mean: unknown dtype");
  }
  const int threads = row_threads(H);
  const size_t lds = static_cast<size_t>(H) * 2 * sizeof(float);
  bool vec = H % 4 == 0 && H <= 16384;
  for (int b = 0; b < n; ++b)
    vec = vec && split_stride[b] % 4 == 0 && reinterpret_cast<uintptr_t>(x[b]) % 16 == 0;
  const int vthreads = vec_threads(N, H / 4);
  const int chunks = vec ? (H / 4 + vthreads - 1) / vthreads : 0;
  if (chunks == 1) norm_mean_vec_kernel<1><<<N, vthreads, 0, stream>>>(branches, n, eps, out, H);
  else if (chunks == 2) norm_mean_vec_kernel<2><<<N, vthreads, 0, stream>>>(branches, n, eps, out, H);
  else if (chunks == 3 || chunks == 4)
    norm_mean_vec_kernel<4><<<N, vthreads, 0, stream>>>(branches, n, eps, out, H);
  else
    norm_mean_kernel<<<N, threads, lds, stream>>>(branches, n, eps, out, H);
  EI_LAUNCH_CHECK();
}

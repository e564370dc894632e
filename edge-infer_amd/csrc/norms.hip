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
                              hipStream_t stream) {
  EI_REQUIRE(N > 0 && H > 0, "stream_norm: sizes must be positive");
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
#define EI_SN(TD, TO)                                                                          \
  stream_norm_kernel<TD, TO><<<N, threads, lds, stream>>>(                                     \
      residual, static_cast<const TD*>(delta), nsplit, ss, delta_bias, rows, w_after, b_after, \
      w_next, b_next, eps, centred, static_cast<TO*>(out), H, write_residual)
  if (delta_dtype == EI_F32 && out_dtype == EI_F32) EI_SN(float, float);
  else if (delta_dtype == EI_F32 && out_dtype == EI_BF16) EI_SN(float, bf16_t);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_BF16) EI_SN(bf16_t, bf16_t);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_F32) EI_SN(bf16_t, float);
  else EI_REQUIRE(false, "stream_norm: unknown dtype");
#undef EI_SN
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
  norm_mean_kernel<<<N, threads, lds, stream>>>(branches, n, eps, out, H);
  EI_LAUNCH_CHECK();
}

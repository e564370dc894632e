// Row-wise kernels of the decoder step: embedding gather, fused residual-add +
// RMSNorm (optionally on gathered rows), SiLU-gate product.  The residual stream is
// float32 in both precisions; sums of squares, the inverse RMS and the products
// are float32 and the result is rounded once to the output type.
//
// Formulas: operators/src/cuda/execution.cu:67-78 (gather),
// operators/src/cuda/rms_norm_cuda.cu:19-101 (x * rsqrt(mean(x^2) + eps) * w),
// operators/src/cuda/silu_cuda.cu:44-56 (silu(gate) * up) of the reference.
#include "common.h"

namespace {

template <typename T>
__global__ void embed_gather_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                                    float* __restrict__ out, int H, int V, float scale) {
  const int row = blockIdx.x;
  const int id = ids[row];
  float* dst = out + static_cast<size_t>(row) * H;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = 0.f;
    return;
  }
  const T* src = table + static_cast<size_t>(id) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = ei::to_f32<T>(src[i]) * scale;
}

// One block per output row.  x = residual[src] (+ sum over splits of delta[s][src]);
// optionally stored back; out[row] = x * rsqrt(mean(x^2) + eps) * weight.
template <typename TD, typename TO, bool HAS_DELTA>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                   int nsplit, size_t split_stride,
                                   const int32_t* __restrict__ rows,
                                   const float* __restrict__ weight, float eps,
                                   TO* __restrict__ out, int H, int write_residual) {
  extern __shared__ float row_values[];
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  if (src < 0) {  // padding row of a fixed-size batch: defined output, nothing else touched
    for (int i = threadIdx.x; i < H; i += blockDim.x)
      out[static_cast<size_t>(row) * H + i] = ei::from_f32<TO>(0.f);
    return;
  }
  float* res = residual + static_cast<size_t>(src) * H;
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float x = res[i];
    if (HAS_DELTA) {
      const TD* d = delta + static_cast<size_t>(src) * H + i;
      for (int s = 0; s < nsplit; ++s) x += ei::to_f32<TD>(d[s * split_stride]);
      if (write_residual) res[i] = x;
    }
    row_values[i] = x;
    sum += x * x;
  }
  const float total = ei::block_sum(sum, scratch);
  const float inv = rsqrtf(total / static_cast<float>(H) + eps);
  TO* dst = out + static_cast<size_t>(row) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    dst[i] = ei::from_f32<TO>((row_values[i] * inv) * weight[i]);
}

// The same for widths that are a multiple of 4: 16-byte accesses, the row kept in
// registers, up to 1024 threads a row so that few rows still have many loads in flight.
using ei::Vec4;

#ifndef EI_NORM_FEW_ROWS_THREADS
#define EI_NORM_FEW_ROWS_THREADS 1024   // threads a row when rows are few (a build-time knob)
#endif

template <typename TD, typename TO, bool HAS_DELTA, int CHUNKS>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                       int nsplit, size_t split_stride,
                                       const int32_t* __restrict__ rows,
                                       const float* __restrict__ weight, float eps,
                                       TO* __restrict__ out, int H, int write_residual) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  const int quads = H / 4;
  TO* dst = out + static_cast<size_t>(row) * H;
  if (src < 0) {
    const float zero[4] = {0.f, 0.f, 0.f, 0.f};
    for (int qd = threadIdx.x; qd < quads; qd += blockDim.x) Vec4<TO>::store(dst + qd * 4, zero);
    return;
  }
  float* res = residual + static_cast<size_t>(src) * H;
  float w[CHUNKS][4];                      // asked for first: it depends on nothing
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) Vec4<float>::load(weight + qd * 4, w[k]);
  }
  float x[CHUNKS][4];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    x[k][0] = x[k][1] = x[k][2] = x[k][3] = 0.f;
    if (qd < quads) {
      Vec4<float>::load(res + qd * 4, x[k]);
      if (HAS_DELTA) {
        const TD* d = delta + static_cast<size_t>(src) * H + qd * 4;
        // slices are added in slice order; eight loads are issued before the first sum so
        // that a row costs one trip to memory per eight slices
        for (int s0 = 0; s0 < nsplit; s0 += 8) {
          float v[8][4];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (s0 + u < nsplit) Vec4<TD>::load(d + (s0 + u) * split_stride, v[u]);
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (s0 + u < nsplit) {
#pragma unroll
              for (int i = 0; i < 4; ++i) x[k][i] += v[u][i];
            }
        }
        if (write_residual) Vec4<float>::store(res + qd * 4, x[k]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) sum += x[k][i] * x[k][i];
    }
  }
  const float total = ei::block_sum(sum, scratch);
  const float inv = rsqrtf(total / static_cast<float>(H) + eps);
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) {
      float y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = (x[k][i] * inv) * w[k][i];
      Vec4<TO>::store(dst + qd * 4, y);
    }
  }
}

// Where gate and up of output column `col` lie in a row of 2I: the halves [gate | up]
// (strip = 0), or strips of `strip` gate columns followed by their `strip` up columns.
// gate activations of the C interface: 0 silu, 1 the tanh form of gelu, 2 the clamped swish:
// with g = min(gate, limit) and u = clamp(up, -limit, limit) the product is
// g sigmoid(alpha g) (u + 1)
template <typename TO> __device__ __forceinline__ float gate_act(float x, int act) {
  if (act == 0) return ei::silu<TO>(x);
  return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}

template <typename TO>
__device__ __forceinline__ float gated_product(float gate, float up, int act, float limit, float alpha) {
  if (act != 2) return gate_act<TO>(gate, act) * up;
  const float g = fminf(gate, limit);
  const float u = fminf(fmaxf(up, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

__device__ __forceinline__ size_t gate_column(size_t col, int strip) {
  return strip ? (col / strip) * 2 * strip + col % strip : col;
}

template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gate_up, int nsplit, size_t split_stride,
                              TO* __restrict__ out, int I, size_t total, int strip, int act,
                              const float* __restrict__ bias, float limit, float alpha) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  const size_t up_offset = strip ? strip : I;
  for (size_t idx = start; idx < total; idx += step) {
    const size_t row = idx / I, col = idx % I;
    const TI* g = gate_up + row * 2 * I + gate_column(col, strip);
    float gate = 0.f, up = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      gate += ei::to_f32<TI>(g[s * split_stride]);
      up += ei::to_f32<TI>(g[s * split_stride + up_offset]);
    }
    if (bias) {        // laid out as a row of gate_up
      gate += bias[gate_column(col, strip)];
      up += bias[gate_column(col, strip) + up_offset];
    }
    out[idx] = ei::from_f32<TO>(gated_product<TO>(gate, up, act, limit, alpha));
  }
}

// The same for I a multiple of 8: a thread takes 8 neighbouring columns of one row with
// 16-byte (bfloat16) or 2 x 16-byte (float32) accesses.
template <typename TI, typename TO>
__global__ void swiglu_vec_kernel(const TI* __restrict__ gate_up, int nsplit, size_t split_stride,
                                  TO* __restrict__ out, int I, size_t total_octets, int strip, int act,
                                  const float* __restrict__ bias, float limit, float alpha) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  const int octets_per_row = I / 8;
  for (size_t idx = start; idx < total_octets; idx += step) {
    const size_t row = idx / octets_per_row;
    const int col = static_cast<int>(idx % octets_per_row) * 8;
    const TI* g = gate_up + row * 2 * I + gate_column(col, strip);   // strips hold whole octets
    const size_t up_offset = strip ? strip : I;
    float gate[8], up[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) gate[i] = up[i] = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += 4) {     // four slices per trip to memory
      float a[4][4], b[4][4], c[4][4], d[4][4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
          const TI* p = g + (s0 + u) * split_stride;
          Vec4<TI>::load(p, a[u]);
          Vec4<TI>::load(p + 4, b[u]);
          Vec4<TI>::load(p + up_offset, c[u]);
          Vec4<TI>::load(p + up_offset + 4, d[u]);
        }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            gate[i] += a[u][i];
            gate[i + 4] += b[u][i];
            up[i] += c[u][i];
            up[i + 4] += d[u][i];
          }
        }
    }
    if (bias) {        // laid out as a row of gate_up
      const float* b = bias + gate_column(col, strip);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        gate[i] += b[i];
        up[i] += b[up_offset + i];
      }
    }
    float y0[4], y1[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      y0[i] = gated_product<TO>(gate[i], up[i], act, limit, alpha);
      y1[i] = gated_product<TO>(gate[i + 4], up[i + 4], act, limit, alpha);
    }
    TO* dst = out + row * I + col;
    Vec4<TO>::store(dst, y0);
    Vec4<TO>::store(dst + 4, y1);
  }
}

// out[i] = sum over slices s of in[s * stride + i], in slice order.
__global__ void sum_slices_kernel(const float* __restrict__ in, int nsplit, size_t stride,
                                  float* __restrict__ out, size_t n) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < n; i += step) {
    float total = in[i];
    for (int s = 1; s < nsplit; ++s) total += in[s * stride + i];
    out[i] = total;
  }
}

// out[r, j] = bias[j] (+ out[r, j] when `accumulate`): a bias as one more slice of a sliced
// product, or added to a finished float32 product.
// operators/src/cuda/execution.cu:61-66,307-317 of the reference (the bias initialises the
// product's accumulator).
__global__ void bias_rows_kernel(const float* __restrict__ bias, float* __restrict__ out,
                                 size_t n, int width, int accumulate) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < n; i += step) {
    const float b = bias[i % width];
    out[i] = accumulate ? out[i] + b : b;
  }
}

}  // namespace

extern "C" int ei_bias_rows(const float* bias, float* out, long long rows, int width,
                            int accumulate, hipStream_t stream) {
  EI_REQUIRE(bias && out && rows > 0 && width > 0, "bias_rows: bad arguments");
  const size_t n = static_cast<size_t>(rows) * width;
  const int threads = 256;
  size_t blocks = (n + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  bias_rows_kernel<<<static_cast<unsigned>(blocks), threads, 0, stream>>>(bias, out, n, width,
                                                                         accumulate);
  EI_LAUNCH_CHECK();
}

extern "C" int ei_sum_slices(const float* in, int nsplit, long long stride, float* out,
                             long long n, hipStream_t stream) {
  EI_REQUIRE(in && out && nsplit >= 1 && n > 0 && stride >= n, "sum_slices: bad arguments");
  const int threads = 256;
  long long blocks = (n + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  sum_slices_kernel<<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
      in, nsplit, static_cast<size_t>(stride), out, static_cast<size_t>(n));
  EI_LAUNCH_CHECK();
}

extern "C" int ei_embed_gather(const int32_t* ids, const void* table, int table_dtype, float* out,
                               int N, int H, int V, float scale, hipStream_t stream) {
  EI_REQUIRE(N > 0 && H > 0 && V > 0, "embed_gather: sizes must be positive");
  EI_REQUIRE(ids && table && out, "embed_gather: null pointer");
  const int threads = H >= 1024 ? 256 : 64;
  if (table_dtype == EI_F32)
    embed_gather_kernel<float><<<N, threads, 0, stream>>>(ids, static_cast<const float*>(table),
                                                          out, H, V, scale);
  else if (table_dtype == EI_BF16)
    embed_gather_kernel<bf16_t><<<N, threads, 0, stream>>>(ids, static_cast<const bf16_t*>(table),
                                                           out, H, V, scale);
  else
    EI_REQUIRE(false, "embed_gather: unknown table dtype");
  EI_LAUNCH_CHECK();
}

template <typename TD, typename TO>
static void launch_add_rmsnorm(float* residual, const void* delta, int nsplit, size_t split_stride,
                               const int32_t* rows, const float* weight, float eps, void* out,
                               int N, int H, int write_residual, hipStream_t stream) {
  if (H % 4 == 0 && (!delta || split_stride % 4 == 0)) {
    const int quads = H / 4;
    // few rows: up to 1024 threads a row, so that many loads are in flight; many rows: 256
    // threads a row, so that several rows share a compute unit and overlap their phases
    const int most = N >= 512 && quads <= 4 * 256 ? 256 : EI_NORM_FEW_ROWS_THREADS;
    int threads = (quads + EI_WAVE - 1) / EI_WAVE * EI_WAVE;
    if (threads > most) threads = most;
    const int chunks = (quads + threads - 1) / threads;      // 1..4 for H <= 16384
#define EI_NORM_VEC(C)                                                                         \
  do {                                                                                         \
    if (delta)                                                                                 \
      add_rmsnorm_vec_kernel<TD, TO, true, C><<<N, threads, 0, stream>>>(                      \
          residual, static_cast<const TD*>(delta), nsplit, split_stride, rows, weight, eps,    \
          static_cast<TO*>(out), H, write_residual);                                           \
    else                                                                                       \
      add_rmsnorm_vec_kernel<TD, TO, false, C><<<N, threads, 0, stream>>>(                     \
          residual, nullptr, 0, 0, rows, weight, eps, static_cast<TO*>(out), H, 0);            \
  } while (0)
    if (chunks == 1) EI_NORM_VEC(1);
    else if (chunks == 2) EI_NORM_VEC(2);
    else EI_NORM_VEC(4);
#undef EI_NORM_VEC
    return;
  }
  const int threads = H >= 2048 ? 256 : (H >= 256 ? 128 : 64);
  const size_t lds = static_cast<size_t>(H) * sizeof(float);
  if (delta)
    add_rmsnorm_kernel<TD, TO, true><<<N, threads, lds, stream>>>(
        residual, static_cast<const TD*>(delta), nsplit, split_stride, rows, weight, eps,
        static_cast<TO*>(out), H, write_residual);
  else
    add_rmsnorm_kernel<TD, TO, false><<<N, threads, lds, stream>>>(
        residual, nullptr, 0, 0, rows, weight, eps, static_cast<TO*>(out), H, 0);
}

// residual: float32 [*, H].  delta: [nsplit][*, H] of delta_dtype or null.  rows: null
// (row r reads residual row r) or int32 [N] source rows (negative: padding).
extern "C" int ei_add_rmsnorm(float* residual, const void* delta, int delta_dtype, int nsplit,
                              long long split_stride, const int32_t* rows, const float* weight,
                              float eps, void* out, int out_dtype, int N, int H,
                              int write_residual, hipStream_t stream) {
  EI_REQUIRE(N > 0 && H > 0, "add_rmsnorm: sizes must be positive");
  EI_REQUIRE(H <= 16384, "add_rmsnorm: width above 16384 is not supported");
  EI_REQUIRE(residual && weight && out, "add_rmsnorm: null pointer");
  EI_REQUIRE(!delta || nsplit >= 1, "add_rmsnorm: nsplit must be at least 1");
  EI_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be positive");
  const size_t ss = static_cast<size_t>(split_stride);
  if (delta_dtype == EI_F32 && out_dtype == EI_F32)
    launch_add_rmsnorm<float, float>(residual, delta, nsplit, ss, rows, weight, eps, out, N, H,
                                     write_residual, stream);
  else if (delta_dtype == EI_F32 && out_dtype == EI_BF16)
    launch_add_rmsnorm<float, bf16_t>(residual, delta, nsplit, ss, rows, weight, eps, out, N, H,
                                      write_residual, stream);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_BF16)
    launch_add_rmsnorm<bf16_t, bf16_t>(residual, delta, nsplit, ss, rows, weight, eps, out, N, H,
                                       write_residual, stream);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_F32)
    launch_add_rmsnorm<bf16_t, float>(residual, delta, nsplit, ss, rows, weight, eps, out, N, H,
                                      write_residual, stream);
  else
    EI_REQUIRE(false, "add_rmsnorm: unknown dtype");
  EI_LAUNCH_CHECK();
}

// gate_up: [nsplit][N, 2I], out: [N, I].  strip = 0: gate columns first, then up columns;
// strip > 0 (a divisor of I): `strip` gate columns, their `strip` up columns, and so on.
extern "C" int ei_swiglu(const void* gate_up, int in_dtype, int nsplit, long long split_stride,
                         void* out, int out_dtype, int N, int I, int strip, int act,
                         const float* bias, float limit, float alpha, hipStream_t stream) {
  EI_REQUIRE(N > 0 && I > 0 && nsplit >= 1, "swiglu: sizes must be positive");
  EI_REQUIRE(act >= 0 && act <= 2, "swiglu: unknown gate activation");
  EI_REQUIRE(gate_up && out, "swiglu: null pointer");
  EI_REQUIRE(strip >= 0 && (strip == 0 || I % strip == 0), "swiglu: the strip must divide the width");
  const size_t total = static_cast<size_t>(N) * I;
  const int threads = 256;
  const size_t ss = static_cast<size_t>(split_stride);
  if (I % 8 == 0 && ss % 8 == 0 && strip % 8 == 0) {
    const size_t octets = total / 8;
    size_t vblocks = (octets + threads - 1) / threads;
    if (vblocks > ei_compute_units() * 32) vblocks = ei_compute_units() * 32;
    if (in_dtype == EI_F32 && out_dtype == EI_F32)
      swiglu_vec_kernel<float, float><<<vblocks, threads, 0, stream>>>(
          static_cast<const float*>(gate_up), nsplit, ss, static_cast<float*>(out), I, octets, strip, act, bias, limit, alpha);
    else if (in_dtype == EI_F32 && out_dtype == EI_BF16)
      swiglu_vec_kernel<float, bf16_t><<<vblocks, threads, 0, stream>>>(
          static_cast<const float*>(gate_up), nsplit, ss, static_cast<bf16_t*>(out), I, octets, strip, act, bias, limit, alpha);
    else if (in_dtype == EI_BF16 && out_dtype == EI_BF16)
      swiglu_vec_kernel<bf16_t, bf16_t><<<vblocks, threads, 0, stream>>>(
          static_cast<const bf16_t*>(gate_up), nsplit, ss, static_cast<bf16_t*>(out), I, octets, strip, act, bias, limit, alpha);
    else
      EI_REQUIRE(false, "swiglu: unsupported dtype combination");
    EI_LAUNCH_CHECK();
  }
  size_t blocks = (total + threads - 1) / threads;
  if (blocks > ei_compute_units() * 32) blocks = ei_compute_units() * 32;
  if (in_dtype == EI_F32 && out_dtype == EI_F32)
    swiglu_kernel<float, float><<<blocks, threads, 0, stream>>>(
        static_cast<const float*>(gate_up), nsplit, ss, static_cast<float*>(out), I, total, strip, act, bias, limit, alpha);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16)
    swiglu_kernel<float, bf16_t><<<blocks, threads, 0, stream>>>(
        static_cast<const float*>(gate_up), nsplit, ss, static_cast<bf16_t*>(out), I, total, strip, act, bias, limit, alpha);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16)
    swiglu_kernel<bf16_t, bf16_t><<<blocks, threads, 0, stream>>>(
        static_cast<const bf16_t*>(gate_up), nsplit, ss, static_cast<bf16_t*>(out), I, total, strip, act, bias, limit, alpha);
  else
    EI_REQUIRE(false, "swiglu: unsupported dtype combination");
  EI_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Kernels for blocks whose norm sits on a sublayer's output: residual += rmsnorm(delta) * w.
namespace {

// One block per row.  x = sum over slices of delta[row]; residual[row] += x * rsqrt(mean(x^2)
// + eps) * weight; optionally the new residual row is also written in the storage type (what
// the next sublayer's product reads).
template <typename TD, typename TO>
__global__ void norm_add_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                int nsplit, size_t split_stride, const float* __restrict__ weight,
                                float eps, TO* __restrict__ cast_out, int H,
                                const float* __restrict__ bias) {
  extern __shared__ float row_values[];
  __shared__ float scratch[16];
  const size_t base = static_cast<size_t>(blockIdx.x) * H;
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const TD* d = delta + base + i;
    float x = 0.f;
    for (int s = 0; s < nsplit; ++s) x += ei::to_f32<TD>(d[s * split_stride]);
    if (bias) x += bias[i];
    row_values[i] = x;
    sum += x * x;
  }
  const float total = ei::block_sum(sum, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(H) + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float y = residual[base + i] + (row_values[i] * inv) * weight[i];
    residual[base + i] = y;
    if (cast_out) cast_out[base + i] = ei::from_f32<TO>(y);
  }
}

// The same for widths that are a multiple of 4: 16-byte accesses, the row kept in registers,
// the slices' loads issued eight at a time (they are added in slice order).
template <typename TD, typename TO, int CHUNKS>
__global__ void norm_add_vec_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                    int nsplit, size_t split_stride,
                                    const float* __restrict__ weight, float eps,
                                    TO* __restrict__ cast_out, int H,
                                    const float* __restrict__ bias) {
  __shared__ float scratch[16];
  const size_t base = static_cast<size_t>(blockIdx.x) * H;
  const int quads = H / 4;
  float w[CHUNKS][4], r[CHUNKS][4], x[CHUNKS][4];
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) {
      Vec4<float>::load(weight + qd * 4, w[k]);
      Vec4<float>::load(residual + base + qd * 4, r[k]);
    }
  }
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    x[k][0] = x[k][1] = x[k][2] = x[k][3] = 0.f;
    if (qd < quads) {
      const TD* d = delta + base + qd * 4;
      for (int s0 = 0; s0 < nsplit; s0 += 8) {
        float v[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) Vec4<TD>::load(d + (s0 + u) * split_stride, v[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) {
#pragma unroll
            for (int i = 0; i < 4; ++i) x[k][i] += v[u][i];
          }
      }
      if (bias) {
        float b[4];
        Vec4<float>::load(bias + qd * 4, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) x[k][i] += b[i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) sum += x[k][i] * x[k][i];
    }
  }
  const float total = ei::block_sum(sum, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(H) + eps);
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) {
      float y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = r[k][i] + (x[k][i] * inv) * w[k][i];
      Vec4<float>::store(residual + base + qd * 4, y);
      if (cast_out) Vec4<TO>::store(cast_out + base + qd * 4, y);
    }
  }
}

template <typename TO>
__global__ void cast_rows_kernel(const float* __restrict__ in, TO* __restrict__ out, size_t n) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < n; i += step) out[i] = ei::from_f32<TO>(in[i]);
}

// activation kinds of the C interface
constexpr int kRelu2 = 0, kRelu = 1, kSilu = 2, kGeluTanh = 3;

__device__ __forceinline__ float activate(float x, int kind) {
  if (kind == kRelu2) {
    const float r = fmaxf(x, 0.f);
    return r * r;
  }
  if (kind == kRelu) return fmaxf(x, 0.f);
  if (kind == kSilu) return x / (1.0f + expf(-x));
  // 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3)))
  return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}

// out = act(sum over slices of in), elementwise.
template <typename TI, typename TO>
__global__ void activation_kernel(const TI* __restrict__ in, int nsplit, size_t split_stride,
                                  TO* __restrict__ out, size_t n, int kind) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < n; i += step) {
    float x = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += 8) {      // eight slices per trip to memory
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < nsplit) v[u] = ei::to_f32<TI>(in[(s0 + u) * split_stride + i]);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < nsplit) x += v[u];
    }
    out[i] = ei::from_f32<TO>(activate(x, kind));
  }
}

// The same for counts and strides that are multiples of 8: a thread takes 8 neighbours with
// 16-byte (bfloat16) or 2 x 16-byte (float32) accesses, four slices per trip to memory.
template <typename TI, typename TO>
__global__ void activation_vec_kernel(const TI* __restrict__ in, int nsplit, size_t split_stride,
                                      TO* __restrict__ out, size_t octets, int kind) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t idx = start; idx < octets; idx += step) {
    const TI* p = in + idx * 8;
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += 4) {
      float v[4][8];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) ei::VecN<TI, 8>::load(p + (s0 + u) * split_stride, v[u]);
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
#pragma unroll
          for (int i = 0; i < 8; ++i) x[i] += v[u][i];
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = activate(x[i], kind);
    ei::VecN<TO, 8>::store(out + idx * 8, x);
  }
}

}  // namespace

// residual [N, H] float32 += rmsnorm(sum of delta slices) * weight; cast_out (or null): the
// new residual rows in out_dtype.
extern "C" int ei_norm_add(float* residual, const void* delta, int delta_dtype, int nsplit,
                           long long split_stride, const float* weight, float eps, void* cast_out,
                           int out_dtype, int N, int H, const float* bias, hipStream_t stream) {
  EI_REQUIRE(N > 0 && H > 0, "norm_add: sizes must be positive");
  EI_REQUIRE(H <= 16384, "norm_add: width above 16384 is not supported");
  EI_REQUIRE(residual && delta && weight && nsplit >= 1, "norm_add: bad arguments");
  EI_REQUIRE(eps > 0.f, "norm_add: eps must be positive");
  const int threads = H >= 2048 ? 512 : (H >= 512 ? 256 : 64);
  const size_t lds = static_cast<size_t>(H) * sizeof(float);
  const size_t ss = static_cast<size_t>(split_stride);
  const bool vec = H % 4 == 0 && ss % 4 == 0;
  const int quads = H / 4;
  // few rows: up to 1024 threads a row, so that many loads are in flight; many rows: 256
  const int most = N >= 512 && quads <= 4 * 256 ? 256 : 1024;
  int vthreads = (quads + EI_WAVE - 1) / EI_WAVE * EI_WAVE;
  if (vthreads > most) vthreads = most;
  const int chunks = vec ? (quads + vthreads - 1) / vthreads : 0;      // 1..4 for H <= 16384
#define EI_NORM_ADD_VEC(TD, TO, C)                                                               \
  norm_add_vec_kernel<TD, TO, C><<<N, vthreads, 0, stream>>>(                                    \
      residual, static_cast<const TD*>(delta), nsplit, ss, weight, eps, static_cast<TO*>(cast_out), H, \
      bias)
#define EI_NORM_ADD(TD, TO)                                                                      \
  do {                                                                                           \
    if (chunks == 1) EI_NORM_ADD_VEC(TD, TO, 1);                                                 \
    else if (chunks == 2) EI_NORM_ADD_VEC(TD, TO, 2);                                            \
    else if (chunks >= 3) EI_NORM_ADD_VEC(TD, TO, 4);                                            \
    else                                                                                         \
      norm_add_kernel<TD, TO><<<N, threads, lds, stream>>>(                                      \
          residual, static_cast<const TD*>(delta), nsplit, ss, weight, eps,                      \
          static_cast<TO*>(cast_out), H, bias);                                                  \
  } while (0)
  if (delta_dtype == EI_F32 && (out_dtype == EI_F32 || !cast_out)) EI_NORM_ADD(float, float);
  else if (delta_dtype == EI_F32 && out_dtype == EI_BF16) EI_NORM_ADD(float, bf16_t);
  else if (delta_dtype == EI_BF16 && (out_dtype == EI_BF16 || !cast_out)) EI_NORM_ADD(bf16_t, bf16_t);
  else EI_REQUIRE(false, "norm_add: unsupported dtype combination");
#undef EI_NORM_ADD
#undef EI_NORM_ADD_VEC
  EI_LAUNCH_CHECK();
}

extern "C" int ei_cast_rows(const float* in, void* out, int out_dtype, long long n,
                            hipStream_t stream) {
  EI_REQUIRE(in && out && n > 0, "cast_rows: bad arguments");
  const int threads = 256;
  long long blocks = (n + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  if (out_dtype == EI_BF16)
    cast_rows_kernel<bf16_t><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
        in, static_cast<bf16_t*>(out), static_cast<size_t>(n));
  else if (out_dtype == EI_F32)
    cast_rows_kernel<float><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
        in, static_cast<float*>(out), static_cast<size_t>(n));
  else
    EI_REQUIRE(false, "cast_rows: unknown dtype");
  EI_LAUNCH_CHECK();
}

// out [n] = act(sum of `nsplit` slices of in); kind 0: relu(x)^2, 1: relu, 2: silu, 3: tanh gelu.
extern "C" int ei_activation(const void* in, int in_dtype, int nsplit, long long split_stride,
                             void* out, int out_dtype, long long n, int kind, hipStream_t stream) {
  EI_REQUIRE(in && out && n > 0 && nsplit >= 1, "activation: bad arguments");
  EI_REQUIRE(kind >= 0 && kind <= 3, "activation: unknown kind");
  const int threads = 256;
  long long blocks = (n + threads - 1) / threads;
  if (blocks > ei_compute_units() * 32) blocks = ei_compute_units() * 32;
  const size_t ss = static_cast<size_t>(split_stride);
  const bool vec = n % 8 == 0 && ss % 8 == 0 &&
                   (reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) % 16 == 0;
  if (vec) {
    blocks = (n / 8 + threads - 1) / threads;
    if (blocks > ei_compute_units() * 32) blocks = ei_compute_units() * 32;
  }
#define EI_ACT(TI, TO)                                                                         \
  do {                                                                                         \
    if (vec)                                                                                   \
      activation_vec_kernel<TI, TO><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(    \
          static_cast<const TI*>(in), nsplit, ss, static_cast<TO*>(out),                       \
          static_cast<size_t>(n / 8), kind);                                                   \
    else                                                                                       \
      activation_kernel<TI, TO><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(        \
          static_cast<const TI*>(in), nsplit, ss, static_cast<TO*>(out),                       \
          static_cast<size_t>(n), kind);                                                       \
  } while (0)
  if (in_dtype == EI_F32 && out_dtype == EI_F32) EI_ACT(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16) EI_ACT(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16) EI_ACT(bf16_t, bf16_t);
  else EI_REQUIRE(false, "activation: unsupported dtype combination");
#undef EI_ACT
  EI_LAUNCH_CHECK();
}


// ---------------------------------------------------------------------------------------
// Kernels for blocks with a norm on both sides of every sublayer, and for a stream that is
// made anew from two streams.
namespace {

// One block per row.  x = sum over slices of delta[row]; y = residual[row] + x * rsqrt(mean(x^2)
// + eps) * w_after (stored back); out[row] = y * rsqrt(mean(y^2) + eps) * w_next in the storage
// type: the norm on a sublayer's output, the addition and the next sublayer's input norm in
// one pass over the row.
template <typename TD, typename TO>
__global__ void norm_add_norm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                     int nsplit, size_t split_stride,
                                     const float* __restrict__ w_after,
                                     const float* __restrict__ w_next, float eps,
                                     TO* __restrict__ out, int H,
                                     const float* __restrict__ bias) {
  extern __shared__ float row_values[];
  __shared__ float scratch[16];
  const size_t base = static_cast<size_t>(blockIdx.x) * H;
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const TD* d = delta + base + i;
    float x = 0.f;
    for (int s = 0; s < nsplit; ++s) x += ei::to_f32<TD>(d[s * split_stride]);
    if (bias) x += bias[i];
    row_values[i] = x;
    sum += x * x;
  }
  const float inv = 1.0f / sqrtf(ei::block_sum(sum, scratch) / static_cast<float>(H) + eps);
  float sum2 = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float y = residual[base + i] + (row_values[i] * inv) * w_after[i];
    residual[base + i] = y;
    row_values[i] = y;
    sum2 += y * y;
  }
  const float inv2 = 1.0f / sqrtf(ei::block_sum(sum2, scratch) / static_cast<float>(H) + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    out[base + i] = ei::from_f32<TO>((row_values[i] * inv2) * w_next[i]);
}

// The same for widths that are a multiple of 4: 16-byte accesses, the row kept in registers,
// the slices' loads issued eight at a time (they are added in slice order).
template <typename TD, typename TO, int CHUNKS>
__global__ void norm_add_norm_vec_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                         int nsplit, size_t split_stride,
                                         const float* __restrict__ w_after,
                                         const float* __restrict__ w_next, float eps,
                                         TO* __restrict__ out, int H,
                                         const float* __restrict__ bias) {
  __shared__ float scratch[16];
  const size_t base = static_cast<size_t>(blockIdx.x) * H;
  const int quads = H / 4;
  float wa[CHUNKS][4], wn[CHUNKS][4], r[CHUNKS][4], x[CHUNKS][4];
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) {
      Vec4<float>::load(w_after + qd * 4, wa[k]);
      Vec4<float>::load(w_next + qd * 4, wn[k]);
      Vec4<float>::load(residual + base + qd * 4, r[k]);
    }
  }
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    x[k][0] = x[k][1] = x[k][2] = x[k][3] = 0.f;
    if (qd < quads) {
      const TD* d = delta + base + qd * 4;
      for (int s0 = 0; s0 < nsplit; s0 += 8) {
        float v[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) Vec4<TD>::load(d + (s0 + u) * split_stride, v[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) {
#pragma unroll
            for (int i = 0; i < 4; ++i) x[k][i] += v[u][i];
          }
      }
      if (bias) {
        float b[4];
        Vec4<float>::load(bias + qd * 4, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) x[k][i] += b[i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) sum += x[k][i] * x[k][i];
    }
  }
  const float inv = 1.0f / sqrtf(ei::block_sum(sum, scratch) / static_cast<float>(H) + eps);
  float sum2 = 0.f;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        r[k][i] += (x[k][i] * inv) * wa[k][i];
        sum2 += r[k][i] * r[k][i];
      }
      Vec4<float>::store(residual + base + qd * 4, r[k]);
    }
  }
  const float inv2 = 1.0f / sqrtf(ei::block_sum(sum2, scratch) / static_cast<float>(H) + eps);
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) {
      float y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = (r[k][i] * inv2) * wn[k][i];
      Vec4<TO>::store(out + base + qd * 4, y);
    }
  }
}

// out[r] = [a[r] | b[r]] in the storage type: two float32 streams side by side as the operand
// of one product.
template <typename TO>
__global__ void concat_cast_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                   TO* __restrict__ out, int H, size_t n) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < n; i += step) {
    const size_t row = i / (2 * H);
    const int col = static_cast<int>(i % (2 * H));
    const float v = col < H ? a[row * H + col] : b[row * H + col - H];
    out[i] = ei::from_f32<TO>(v);
  }
}

// out[r, j] = sum over slices of x[s][r, j] + vec[j]: a product's result takes the place of
// the float32 stream.
template <typename TD>
__global__ void set_rows_kernel(const TD* __restrict__ x, int nsplit, size_t split_stride,
                                const float* __restrict__ vec, float* __restrict__ out, int H,
                                size_t n) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < n; i += step) {
    float total = 0.f;
    for (int s = 0; s < nsplit; ++s) total += ei::to_f32<TD>(x[s * split_stride + i]);
    out[i] = vec ? total + vec[i % H] : total;
  }
}

}  // namespace

extern "C" int ei_norm_add_norm(float* residual, const void* delta, int delta_dtype, int nsplit,
                                long long split_stride, const float* w_after, const float* w_next,
                                float eps, void* out, int out_dtype, int N, int H,
                                const float* bias, hipStream_t stream) {
  EI_REQUIRE(N > 0 && H > 0 && nsplit >= 1, "norm_add_norm: sizes must be positive");
  EI_REQUIRE(residual && delta && w_after && w_next && out, "norm_add_norm: null pointer");
  EI_REQUIRE(static_cast<size_t>(H) * sizeof(float) <= 60 * 1024, "norm_add_norm: row too wide");
  const int threads = H >= 2048 ? 512 : (H >= 512 ? 256 : 128);
  const size_t lds = static_cast<size_t>(H) * sizeof(float);
  const size_t ss = static_cast<size_t>(split_stride);
  const bool vec = H % 4 == 0 && ss % 4 == 0;
  const int quads = H / 4;
  // few rows: up to 1024 threads a row, so that many loads are in flight; many rows: 256
  const int most = N >= 512 && quads <= 4 * 256 ? 256 : 1024;
  int vthreads = (quads + EI_WAVE - 1) / EI_WAVE * EI_WAVE;
  if (vthreads > most) vthreads = most;
  const int chunks = vec ? (quads + vthreads - 1) / vthreads : 0;
#define EI_NAN_VEC(TD, TO, C)                                                                \
  norm_add_norm_vec_kernel<TD, TO, C><<<N, vthreads, 0, stream>>>(                           \
      residual, static_cast<const TD*>(delta), nsplit, ss, w_after, w_next, eps,             \
      static_cast<TO*>(out), H, bias)
#define EI_NAN_CASE(TD, TO)                                                                  \
  do {                                                                                       \
    if (chunks == 1) EI_NAN_VEC(TD, TO, 1);                                                  \
    else if (chunks == 2) EI_NAN_VEC(TD, TO, 2);                                             \
    else if (chunks == 3 || chunks == 4) EI_NAN_VEC(TD, TO, 4);                              \
    else                                                                                     \
      norm_add_norm_kernel<TD, TO><<<N, threads, lds, stream>>>(                             \
          residual, static_cast<const TD*>(delta), nsplit, ss, w_after, w_next, eps,         \
          static_cast<TO*>(out), H, bias);                                                   \
  } while (0)
  if (delta_dtype == EI_F32 && out_dtype == EI_F32) EI_NAN_CASE(float, float);
  else if (delta_dtype == EI_F32 && out_dtype == EI_BF16) EI_NAN_CASE(float, bf16_t);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_BF16) EI_NAN_CASE(bf16_t, bf16_t);
  else EI_REQUIRE(false, "norm_add_norm: unsupported dtype combination");
#undef EI_NAN_CASE
#undef EI_NAN_VEC
  EI_LAUNCH_CHECK();
}

extern "C" int ei_concat_cast(const float* a, const float* b, void* out, int out_dtype,
                              long long rows, int H, hipStream_t stream) {
  EI_REQUIRE(a && b && out && rows > 0 && H > 0, "concat_cast: bad arguments");
  const size_t n = static_cast<size_t>(rows) * 2 * H;
  const int threads = 256;
  size_t blocks = (n + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  if (out_dtype == EI_F32)
    concat_cast_kernel<float><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
        a, b, static_cast<float*>(out), H, n);
  else if (out_dtype == EI_BF16)
    concat_cast_kernel<bf16_t><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
        a, b, static_cast<bf16_t*>(out), H, n);
  else
    EI_REQUIRE(false, "concat_cast: unknown dtype");
  EI_LAUNCH_CHECK();
}

extern "C" int ei_set_rows(const void* x, int x_dtype, int nsplit, long long split_stride,
                           const float* vec, float* out, long long rows, int H,
                           hipStream_t stream) {
  EI_REQUIRE(x && out && rows > 0 && H > 0 && nsplit >= 1, "set_rows: bad arguments");
  const size_t n = static_cast<size_t>(rows) * H;
  const int threads = 256;
  size_t blocks = (n + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  const size_t ss = static_cast<size_t>(split_stride);
  if (x_dtype == EI_F32)
    set_rows_kernel<float><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
        static_cast<const float*>(x), nsplit, ss, vec, out, H, n);
  else if (x_dtype == EI_BF16)
    set_rows_kernel<bf16_t><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
        static_cast<const bf16_t*>(x), nsplit, ss, vec, out, H, n);
  else
    EI_REQUIRE(false, "set_rows: unknown dtype");
  EI_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// x [rows, H] float32 <- x / sqrt(mean(x^2) + eps) * w, in place: a norm that sits on the
// stream itself (the one behind an embedding).  A block a row.
namespace {
__global__ void norm_rows_kernel(float* __restrict__ x, const float* __restrict__ w, float eps, int H) {
  __shared__ float scratch[16];
  float* row = x + static_cast<size_t>(blockIdx.x) * H;
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) sum += row[i] * row[i];
  const float inv = 1.0f / sqrtf(ei::block_sum(sum, scratch) / static_cast<float>(H) + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) row[i] = (row[i] * inv) * w[i];
}

// out [rows, W] *= sigmoid(gate), gate the columns col0 .. col0 + W - 1 of rows `stride` wide
// (or the sum of `nsplit` float32 slices of them).
template <typename TG, typename TO>
__global__ void gate_rows_kernel(const TG* __restrict__ gate, int nsplit, size_t split_stride,
                                 size_t stride, int col0, TO* __restrict__ out, int W, size_t total) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t idx = start; idx < total; idx += step) {
    const size_t row = idx / W, col = idx % W;
    const TG* g = gate + row * stride + col0 + col;
    float z = 0.f;
    for (int s = 0; s < nsplit; ++s) z += ei::to_f32<TG>(g[s * split_stride]);
    out[idx] = ei::from_f32<TO>(ei::to_f32<TO>(out[idx]) / (1.0f + expf(-z)));
  }
}

// x <- cap tanh(scale x / cap) (cap > 0), or scale x.
__global__ void scale_cap_kernel(float* __restrict__ x, float scale, float cap, size_t total) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < total; i += step) {
    const float v = x[i] * scale;
    x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}
}  // namespace

extern "C" int ei_norm_rows(float* x, const float* w, float eps, long long rows, int H,
                            hipStream_t stream) {
  EI_REQUIRE(x && w && rows > 0 && H > 0, "norm_rows: bad arguments");
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  norm_rows_kernel<<<static_cast<unsigned>(rows), threads, 0, stream>>>(x, w, eps, H);
  EI_LAUNCH_CHECK();
}

extern "C" int ei_gate_rows(const void* gate, int gate_dtype, int nsplit, long long split_stride,
                            long long stride, int col0, void* out, int out_dtype, long long rows,
                            int W, hipStream_t stream) {
  EI_REQUIRE(gate && out && rows > 0 && W > 0 && nsplit >= 1 && col0 >= 0 && col0 + W <= stride,
             "gate_rows: bad arguments");
  const size_t total = static_cast<size_t>(rows) * W;
  const int threads = 256;
  size_t blocks = (total + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  const size_t ss = static_cast<size_t>(split_stride), st = static_cast<size_t>(stride);
  const unsigned b = static_cast<unsigned>(blocks);
  if (gate_dtype == EI_F32 && out_dtype == EI_F32)
    gate_rows_kernel<float, float><<<b, threads, 0, stream>>>(
        static_cast<const float*>(gate), nsplit, ss, st, col0, static_cast<float*>(out), W, total);
  else if (gate_dtype == EI_F32 && out_dtype == EI_BF16)
    gate_rows_kernel<float, bf16_t><<<b, threads, 0, stream>>>(
        static_cast<const float*>(gate), nsplit, ss, st, col0, static_cast<bf16_t*>(out), W, total);
  else if (gate_dtype == EI_BF16 && out_dtype == EI_BF16)
    gate_rows_kernel<bf16_t, bf16_t><<<b, threads, 0, stream>>>(
        static_cast<const bf16_t*>(gate), nsplit, ss, st, col0, static_cast<bf16_t*>(out), W, total);
  else
    EI_REQUIRE(false, "gate_rows: unsupported dtype combination");
  EI_LAUNCH_CHECK();
}

extern "C" int ei_scale_cap(float* x, float scale, float cap, long long total, hipStream_t stream) {
  EI_REQUIRE(x && total > 0, "scale_cap: bad arguments");
  const int threads = 256;
  size_t blocks = (static_cast<size_t>(total) + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  scale_cap_kernel<<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
      x, scale, cap, static_cast<size_t>(total));
  EI_LAUNCH_CHECK();
}

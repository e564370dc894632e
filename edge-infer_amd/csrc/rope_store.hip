// Fused per-head q/k RMSNorm -> rotary encoding -> cache store.
//
// One wave per (row, head) over the packed projection [N, Q + 2*KV]: query heads
// are normed, rotated and written to q_out; key heads are normed, rotated and
// written to the cache page of (sequence, position); value heads are copied to
// the cache.  Sum of squares, inverse RMS, angles' sine/cosine (a float32 table)
// and the rotation are float32; one rounding to the storage type.
//
// Formulas of the reference: norm before rotation,
// runtime/include/execution/decoder.hpp:125-140; rotate-half pairs (i, i + d/2),
// x' = x cos - y sin, y' = x sin + y cos, operators/src/cuda/execution.cu:79-122;
// keys stored after norm and rotation, values raw, decoder.hpp:137-140.
//
// The rotation may cover only the first R <= D elements of a head (R = the table's width):
// pairs (i, i + R/2) for i < R/2, elements R..D-1 pass unrotated.  A lane's pair j of D/2 is
// then elements (j, j + R/2) below R/2 and (j + R/2, j + D/2) from there on, the latter with
// the identity as its rotation; with R = D this is the pair (j, j + D/2) throughout.
#include "common.h"

namespace {

constexpr int kMaxPairsPerLane = 4;  // head_dim up to 512

template <typename TI, typename TO>
__global__ void qk_norm_rope_store_kernel(
    const TI* __restrict__ qkv, int nsplit, size_t split_stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ rope_table,  // [max_pos, R]: cos[R/2] then sin[R/2]; null: none
    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_out, TO* __restrict__ k_pages, TO* __restrict__ v_pages,
    int N, int nq, int nkv, int D, int R, int write_cache) {
  const int heads = nq + 2 * nkv;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= N * heads) return;
  const int row = wave / heads, head = wave % heads;
  const int seq = row_seq[row];
  if (seq < 0) return;  // padding row
  const bool is_q = head < nq, is_k = !is_q && head < nq + nkv;
  if (!is_q && !write_cache) return;
  const int pos = row_pos[row];
  const int half = D / 2, rhalf = R / 2;
  const size_t width = static_cast<size_t>(nq + 2 * nkv) * D;
  const TI* src = qkv + static_cast<size_t>(row) * width + static_cast<size_t>(head) * D;

  float x[kMaxPairsPerLane], y[kMaxPairsPerLane];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < kMaxPairsPerLane; ++j) {
    const int pair = lane + j * EI_WAVE;
    x[j] = 0.f;
    y[j] = 0.f;
    if (pair < half) {
      const int i = pair < rhalf ? pair : pair + rhalf;          // the pair's first element
      const int i2 = pair < rhalf ? pair + rhalf : pair + half;  // and its second
      // slices are added in slice order, four loads per trip to memory
      for (int s0 = 0; s0 < nsplit; s0 += 4) {
        TI a[4], b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (s0 + u < nsplit) {
            a[u] = src[(s0 + u) * split_stride + i];
            b[u] = src[(s0 + u) * split_stride + i2];
          }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (s0 + u < nsplit) {
            x[j] += ei::to_f32<TI>(a[u]);
            y[j] += ei::to_f32<TI>(b[u]);
          }
      }
      sum += x[j] * x[j] + y[j] * y[j];
    }
  }

  TO* dst;
  if (is_q) {
    dst = q_out + static_cast<size_t>(row) * nq * D + static_cast<size_t>(head) * D;
  } else {
    const int page = page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE];
    if (page < 0) return;
    const int g = is_k ? head - nq : head - nq - nkv;
    TO* base = is_k ? k_pages : v_pages;
    dst = base + ((static_cast<size_t>(page) * nkv + g) * EI_PAGE + pos % EI_PAGE) * D;
  }

  const float* norm_w = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
  float inv = 1.f;
  if (norm_w) {
    sum = ei::wave_sum(sum);
    inv = rsqrtf(sum / static_cast<float>(D) + eps);
  }
  const bool rotate = rope_table != nullptr && (is_q || is_k);
  const float* trig = rotate ? rope_table + static_cast<size_t>(pos) * R : nullptr;
#pragma unroll
  for (int j = 0; j < kMaxPairsPerLane; ++j) {
    const int pair = lane + j * EI_WAVE;
    if (pair < half) {
      const int i = pair < rhalf ? pair : pair + rhalf;
      const int i2 = pair < rhalf ? pair + rhalf : pair + half;
      float a = x[j], b = y[j];
      if (norm_w) {
        a = (a * inv) * norm_w[i];
        b = (b * inv) * norm_w[i2];
      }
      if (rotate && pair < rhalf) {
        const float c = trig[pair], s = trig[pair + rhalf];
        const float ra = a * c - b * s;
        const float rb = a * s + b * c;
        a = ra;
        b = rb;
      }
      dst[i] = ei::from_f32<TO>(a);
      dst[i2] = ei::from_f32<TO>(b);
    }
  }
}

// The same for head sizes (and rotated widths) that are a multiple of 2 P: G lanes (a power of
// two) share a head, each lane takes P (4 or 8) neighbouring pairs with one or two 16-byte
// accesses (one of 8 bytes for 4 bfloat16) per half, so a wave covers 64 / G heads.
template <typename TI, typename TO, int G, int P>
__device__ __forceinline__ void qk_norm_rope_store_item(
    long long item, int sub, const TI* __restrict__ qkv, int nsplit, size_t split_stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ rope_table, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_out, TO* __restrict__ k_pages, TO* __restrict__ v_pages,
    int N, int nq, int nkv, int D, int R, int write_cache) {
  using ei::VecN;
  const int heads = nq + 2 * nkv;
  const int row = static_cast<int>(item / heads), head = static_cast<int>(item % heads);
  const bool is_q = head < nq, is_k = !is_q && head < nq + nkv;
  if (!is_q && !write_cache) return;
  // The sequence and the position are asked for first and the head's elements right after,
  // before either is needed: what depends on them (the page, the angles) is then looked up
  // while the elements are on their way.  (A padding row costs its loads.)
  const int seq = row_seq[row];
  const int pos = row_pos[row];
  const int half = D / 2, rhalf = R / 2;
  const int pair0 = sub * P;                                   // the lane's first pair
  const bool active = pair0 < half;
  const bool turned = pair0 < rhalf;                           // its pairs are rotated ones
  const int i0 = turned ? pair0 : pair0 + rhalf;               // their first elements
  const int i2 = turned ? pair0 + rhalf : pair0 + half;        // and their second ones
  const size_t width = static_cast<size_t>(heads) * D;
  const TI* src = qkv + static_cast<size_t>(row) * width + static_cast<size_t>(head) * D;
  float first_a[4][P], first_b[4][P];                          // the first four slices
  if (active) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (u < nsplit) {
        VecN<TI, P>::load(src + u * split_stride + i0, first_a[u]);
        VecN<TI, P>::load(src + u * split_stride + i2, first_b[u]);
      }
  }
  if (seq < 0) return;  // padding row

  TO* dst;
  bool stored = true;
  if (is_q) {
    dst = q_out + static_cast<size_t>(row) * nq * D + static_cast<size_t>(head) * D;
  } else {
    const int page = page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE];
    stored = page >= 0;
    const int g = is_k ? head - nq : head - nq - nkv;
    TO* base = is_k ? k_pages : v_pages;
    dst = base + ((static_cast<size_t>(stored ? page : 0) * nkv + g) * EI_PAGE + pos % EI_PAGE) * D;
  }
  const float* norm_w = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
  const bool rotate = rope_table != nullptr && (is_q || is_k);

  float x[P], y[P], wx[P], wy[P], cs[P], sn[P];
#pragma unroll
  for (int i = 0; i < P; ++i) {
    x[i] = y[i] = sn[i] = 0.f;
    wx[i] = wy[i] = cs[i] = 1.f;
  }
  if (active) {
    if (norm_w) {
      VecN<float, P>::load(norm_w + i0, wx);
      VecN<float, P>::load(norm_w + i2, wy);
    }
    if (rotate && turned) {
      const float* trig = rope_table + static_cast<size_t>(pos) * R + pair0;
      VecN<float, P>::load(trig, cs);
      VecN<float, P>::load(trig + rhalf, sn);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (u < nsplit) {
#pragma unroll
        for (int i = 0; i < P; ++i) {
          x[i] += first_a[u][i];
          y[i] += first_b[u][i];
        }
      }
    for (int s0 = 4; s0 < nsplit; s0 += 4) {       // further slices in slice order, four per trip
      float a[4][P], b[4][P];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
          VecN<TI, P>::load(src + (s0 + u) * split_stride + i0, a[u]);
          VecN<TI, P>::load(src + (s0 + u) * split_stride + i2, b[u]);
        }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
#pragma unroll
          for (int i = 0; i < P; ++i) {
            x[i] += a[u][i];
            y[i] += b[u][i];
          }
        }
    }
  }
  float inv = 1.f;
  if (norm_w) {
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < P; ++i) sum += x[i] * x[i] + y[i] * y[i];
#pragma unroll
    for (int offset = G / 2; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset, EI_WAVE);
    inv = rsqrtf(sum / static_cast<float>(D) + eps);
  }
  if (!active || !stored) return;
  float ox[P], oy[P];
#pragma unroll
  for (int i = 0; i < P; ++i) {
    float a = x[i], b = y[i];
    if (norm_w) {
      a = (a * inv) * wx[i];
      b = (b * inv) * wy[i];
    }
    if (rotate) {                      // (the identity for pairs beyond the rotated width)
      const float ra = a * cs[i] - b * sn[i];
      const float rb = a * sn[i] + b * cs[i];
      a = ra;
      b = rb;
    }
    ox[i] = a;
    oy[i] = b;
  }
  VecN<TO, P>::store(dst + i0, ox);
  VecN<TO, P>::store(dst + i2, oy);
}

template <typename TI, typename TO, int G, int P>
__global__ void qk_norm_rope_store_vec_kernel(
    const TI* __restrict__ qkv, int nsplit, size_t split_stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ rope_table, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_out, TO* __restrict__ k_pages, TO* __restrict__ v_pages,
    int N, int nq, int nkv, int D, int R, int write_cache) {
  const long long item = (static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x) / G;
  const int sub = threadIdx.x % G;
  if (item >= static_cast<long long>(N) * (nq + 2 * nkv)) return;   // the same for all lanes of a group
  qk_norm_rope_store_item<TI, TO, G, P>(item, sub, qkv, nsplit, split_stride, q_norm_w, k_norm_w,
                                        eps, rope_table, row_pos, row_seq, page_table, table_width,
                                        q_out, k_pages, v_pages, N, nq, nkv, D, R, write_cache);
}

}  // namespace

// qkv: [nsplit][N, (nq + 2 nkv) * D] of in_dtype.  q_out: [N, nq * D] of out_dtype.
// k_pages / v_pages: [n_pages, nkv, 64, D] of out_dtype for this cache entry.
// page_table: int32 [n_seqs, table_width], logical page -> physical page.
extern "C" int ei_qk_norm_rope_store(
    const void* qkv, int in_dtype, int nsplit, long long split_stride, const float* q_norm_w,
    const float* k_norm_w, float eps, const float* rope_table, int rot_dim,
    const int32_t* row_pos, const int32_t* row_seq, const int32_t* page_table, int table_width,
    void* q_out, void* k_pages, void* v_pages, int out_dtype, int N, int nq, int nkv, int D,
    int write_cache, hipStream_t stream) {
  EI_REQUIRE(N > 0 && nq > 0 && nkv > 0 && D > 0, "qk_norm_rope_store: sizes must be positive");
  EI_REQUIRE(D % 2 == 0, "qk_norm_rope_store: head_dim must be even");
  EI_REQUIRE(D / 2 <= kMaxPairsPerLane * EI_WAVE, "qk_norm_rope_store: head_dim above 512");
  EI_REQUIRE(qkv && row_pos && row_seq && q_out, "qk_norm_rope_store: null pointer");
  EI_REQUIRE(!write_cache || (k_pages && v_pages && page_table && table_width > 0),
             "qk_norm_rope_store: cache pointers missing");
  EI_REQUIRE(nsplit >= 1, "qk_norm_rope_store: nsplit must be at least 1");
  // the rotated width R: the table's row length, even, at most the head size (D without a table)
  const int R = rope_table ? rot_dim : D;
  EI_REQUIRE(R >= 2 && R % 2 == 0 && R <= D,
             "qk_norm_rope_store: the rotated width must be even and at most head_dim");
  const int heads = nq + 2 * nkv;
  const int threads = 256;
  const size_t ss = static_cast<size_t>(split_stride);
  // vector kernel: P pairs a lane (8 for bfloat16 in and out where the sizes allow, else 4),
  // G = lanes a head (the power of two at or above D / 2P)
  const bool aligned = (reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(q_out) |
                        reinterpret_cast<uintptr_t>(k_pages) | reinterpret_cast<uintptr_t>(v_pages) |
                        reinterpret_cast<uintptr_t>(q_norm_w) | reinterpret_cast<uintptr_t>(k_norm_w) |
                        reinterpret_cast<uintptr_t>(rope_table)) % 16 == 0;
  if (D % 8 == 0 && R % 8 == 0 && ss % 4 == 0 && aligned) {
    const bool wide = in_dtype == EI_BF16 && out_dtype == EI_BF16 && D % 16 == 0 && R % 16 == 0 &&
                      ss % 8 == 0;
    const int per_lane = wide ? 16 : 8;            // elements of a head a lane takes
    int G = 2;
    while (G * per_lane < D) G *= 2;
    const long long items = static_cast<long long>(N) * heads;
    const long long blocks = (items * G + threads - 1) / threads;
    EI_REQUIRE(blocks < (1ll << 31), "qk_norm_rope_store: too many rows");
#define EI_ROPE_VEC(TI, TO, GG, PP)                                                               \
  qk_norm_rope_store_vec_kernel<TI, TO, GG, PP><<<static_cast<unsigned>(blocks), threads, 0, stream>>>( \
      static_cast<const TI*>(qkv), nsplit, ss, q_norm_w, k_norm_w, eps, rope_table, row_pos,      \
      row_seq, page_table, table_width, static_cast<TO*>(q_out), static_cast<TO*>(k_pages),       \
      static_cast<TO*>(v_pages), N, nq, nkv, D, R, write_cache)
#define EI_ROPE_VEC_G(TI, TO, PP)                                                                 \
  do {                                                                                            \
    if (G == 2) EI_ROPE_VEC(TI, TO, 2, PP);                                                       \
    else if (G == 4) EI_ROPE_VEC(TI, TO, 4, PP);                                                  \
    else if (G == 8) EI_ROPE_VEC(TI, TO, 8, PP);                                                  \
    else if (G == 16) EI_ROPE_VEC(TI, TO, 16, PP);                                                \
    else if (G == 32) EI_ROPE_VEC(TI, TO, 32, PP);                                                \
    else EI_ROPE_VEC(TI, TO, 64, PP);                                                             \
  } while (0)
    if (wide)
      EI_ROPE_VEC_G(bf16_t, bf16_t, 8);
    else if (in_dtype == EI_F32 && out_dtype == EI_F32)
      EI_ROPE_VEC_G(float, float, 4);
    else if (in_dtype == EI_F32 && out_dtype == EI_BF16)
      EI_ROPE_VEC_G(float, bf16_t, 4);
    else if (in_dtype == EI_BF16 && out_dtype == EI_BF16)
      EI_ROPE_VEC_G(bf16_t, bf16_t, 4);
    else
      EI_REQUIRE(false, "qk_norm_rope_store: unsupported dtype combination");
#undef EI_ROPE_VEC_G
#undef EI_ROPE_VEC
    EI_LAUNCH_CHECK();
  }
  const long long waves = static_cast<long long>(N) * heads;
  const long long blocks = (waves * EI_WAVE + threads - 1) / threads;
  EI_REQUIRE(blocks < (1ll << 31), "qk_norm_rope_store: too many rows");
#define EI_ROPE_LAUNCH(TI, TO)                                                                   \
  qk_norm_rope_store_kernel<TI, TO><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(      \
      static_cast<const TI*>(qkv), nsplit, ss, q_norm_w, k_norm_w, eps, rope_table, row_pos,     \
      row_seq, page_table, table_width, static_cast<TO*>(q_out), static_cast<TO*>(k_pages),      \
      static_cast<TO*>(v_pages), N, nq, nkv, D, R, write_cache)
  if (in_dtype == EI_F32 && out_dtype == EI_F32)
    EI_ROPE_LAUNCH(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16)
    EI_ROPE_LAUNCH(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16)
    EI_ROPE_LAUNCH(bf16_t, bf16_t);
  else
    EI_REQUIRE(false, "qk_norm_rope_store: unsupported dtype combination");
#undef EI_ROPE_LAUNCH
  EI_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Queries and keys normed over the whole projection (one RMS norm over all heads of q, one
// over all heads of k, weights of those widths; or no norm), no rotation, and values whose
// head size may differ from the keys'.  One block a row; sums in float32, one rounding.
namespace {

// The same for rows of at most 4 x 256 16-byte pieces whose widths are all multiples of 4: a
// thread keeps its pieces in registers between the sums of squares and the stores, and the two
// sums cross the block together.
template <typename TI, typename TO, int CH>
__global__ void __launch_bounds__(256)
projection_norm_store_reg_kernel(
    const TI* __restrict__ qkv, int nsplit, size_t split_stride, const float* __restrict__ bias,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ page_table, int table_width, TO* __restrict__ q_out,
    TO* __restrict__ k_pages, TO* __restrict__ v_pages, int nq, int nkv, int D, int DV,
    int write_cache) {
  __shared__ float sums[2][4];
  const int row = blockIdx.x;
  const int seq = row_seq[row];
  if (seq < 0) return;                      // padding row of a fixed-size batch
  const int QW = nq * D, KW = nkv * D, VW = nkv * DV, W = QW + KW + VW;
  const TI* src = qkv + static_cast<size_t>(row) * W;
  float x[CH][4];
  float q_sq = 0.f, k_sq = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (threadIdx.x + c * 256) * 4;
    x[c][0] = x[c][1] = x[c][2] = x[c][3] = 0.f;
    if (i < W) {
      if (bias) ei::Vec4<float>::load(bias + i, x[c]);
      for (int s0 = 0; s0 < nsplit; s0 += 8) {
        float v[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) ei::Vec4<TI>::load(src + (s0 + u) * split_stride + i, v[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) {
#pragma unroll
            for (int e = 0; e < 4; ++e) x[c][e] += v[u][e];
          }
      }
      const float sq = x[c][0] * x[c][0] + x[c][1] * x[c][1] + x[c][2] * x[c][2] + x[c][3] * x[c][3];
      if (i < QW) q_sq += sq;
      else if (i < QW + KW) k_sq += sq;
    }
  }
  q_sq = ei::wave_sum(q_sq);
  k_sq = ei::wave_sum(k_sq);
  if (threadIdx.x % EI_WAVE == 0) {
    sums[0][threadIdx.x / EI_WAVE] = q_sq;
    sums[1][threadIdx.x / EI_WAVE] = k_sq;
  }
  __syncthreads();
  const float q_total = sums[0][0] + sums[0][1] + sums[0][2] + sums[0][3];
  const float k_total = sums[1][0] + sums[1][1] + sums[1][2] + sums[1][3];
  const float q_inv = q_norm_w ? 1.0f / sqrtf(q_total / static_cast<float>(QW) + eps) : 1.f;
  const float k_inv = k_norm_w ? 1.0f / sqrtf(k_total / static_cast<float>(KW) + eps) : 1.f;
  const int pos = row_pos[row];
  const int phys = write_cache ? page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE] : -1;
  const int in_page = pos % EI_PAGE;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (threadIdx.x + c * 256) * 4;
    if (i >= W) continue;
    float w[4];
    if (i < QW) {
      if (q_norm_w) {
        ei::Vec4<float>::load(q_norm_w + i, w);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[c][e] = (x[c][e] * q_inv) * w[e];
      }
      ei::Vec4<TO>::store(q_out + static_cast<size_t>(row) * QW + i, x[c]);
    } else if (phys >= 0 && i < QW + KW) {
      const int at = i - QW, head = at / D, d = at % D;
      if (k_norm_w) {
        ei::Vec4<float>::load(k_norm_w + at, w);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[c][e] = (x[c][e] * k_inv) * w[e];
      }
      ei::Vec4<TO>::store(
          k_pages + ((static_cast<size_t>(phys) * nkv + head) * EI_PAGE + in_page) * D + d, x[c]);
    } else if (phys >= 0) {
      const int at = i - QW - KW, head = at / DV, d = at % DV;
      ei::Vec4<TO>::store(
          v_pages + ((static_cast<size_t>(phys) * nkv + head) * EI_PAGE + in_page) * DV + d, x[c]);
    }
  }
}

template <typename TI, typename TO, bool VEC>
__global__ void projection_norm_store_kernel(
    const TI* __restrict__ qkv, int nsplit, size_t split_stride, const float* __restrict__ bias,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ page_table, int table_width, TO* __restrict__ q_out,
    TO* __restrict__ k_pages, TO* __restrict__ v_pages, int nq, int nkv, int D, int DV,
    int write_cache) {
  extern __shared__ __attribute__((aligned(16))) float row_values[];     // the row's q, k and v sums
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int seq = row_seq[row];
  if (seq < 0) return;                      // padding row of a fixed-size batch
  const int QW = nq * D, KW = nkv * D, VW = nkv * DV, W = QW + KW + VW;
  const TI* src = qkv + static_cast<size_t>(row) * W;
  float q_sq = 0.f, k_sq = 0.f;
  if constexpr (VEC) {      // every width a multiple of 4: 16-byte pieces, 8 slices per trip
    for (int i = threadIdx.x * 4; i < W; i += blockDim.x * 4) {
      float x[4] = {0.f, 0.f, 0.f, 0.f};
      if (bias) ei::Vec4<float>::load(bias + i, x);
      for (int s0 = 0; s0 < nsplit; s0 += 8) {
        float v[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) ei::Vec4<TI>::load(src + (s0 + u) * split_stride + i, v[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) {
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] += v[u][e];
          }
      }
      ei::Vec4<float>::store(row_values + i, x);
      const float sq = x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
      if (i < QW) q_sq += sq;
      else if (i < QW + KW) k_sq += sq;
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float x = bias ? bias[i] : 0.f;
      for (int s0 = 0; s0 < nsplit; s0 += 8) {      // eight slices per trip to memory
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) v[u] = ei::to_f32<TI>(src[(s0 + u) * split_stride + i]);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < nsplit) x += v[u];
      }
      row_values[i] = x;
      if (i < QW) q_sq += x * x;
      else if (i < QW + KW) k_sq += x * x;
    }
  }
  const float q_total = ei::block_sum(q_sq, scratch);
  const float k_total = ei::block_sum(k_sq, scratch);
  const float q_inv = q_norm_w ? 1.0f / sqrtf(q_total / static_cast<float>(QW) + eps) : 1.f;
  const float k_inv = k_norm_w ? 1.0f / sqrtf(k_total / static_cast<float>(KW) + eps) : 1.f;
  const int pos = row_pos[row];
  const int phys = write_cache ? page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE] : -1;
  const int in_page = pos % EI_PAGE;
  if constexpr (VEC) {
    for (int i = threadIdx.x * 4; i < W; i += blockDim.x * 4) {
      float x[4], w[4] = {1.f, 1.f, 1.f, 1.f};
      ei::Vec4<float>::load(row_values + i, x);
      if (i < QW) {
        if (q_norm_w) {
          ei::Vec4<float>::load(q_norm_w + i, w);
#pragma unroll
          for (int e = 0; e < 4; ++e) x[e] = (x[e] * q_inv) * w[e];
        }
        ei::Vec4<TO>::store(q_out + static_cast<size_t>(row) * QW + i, x);
      } else if (phys >= 0 && i < QW + KW) {
        const int at = i - QW, head = at / D, d = at % D;
        if (k_norm_w) {
          ei::Vec4<float>::load(k_norm_w + at, w);
#pragma unroll
          for (int e = 0; e < 4; ++e) x[e] = (x[e] * k_inv) * w[e];
        }
        ei::Vec4<TO>::store(
            k_pages + ((static_cast<size_t>(phys) * nkv + head) * EI_PAGE + in_page) * D + d, x);
      } else if (phys >= 0) {
        const int at = i - QW - KW, head = at / DV, d = at % DV;
        ei::Vec4<TO>::store(
            v_pages + ((static_cast<size_t>(phys) * nkv + head) * EI_PAGE + in_page) * DV + d, x);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < QW; i += blockDim.x) {
    const float y = q_norm_w ? (row_values[i] * q_inv) * q_norm_w[i] : row_values[i];
    q_out[static_cast<size_t>(row) * QW + i] = ei::from_f32<TO>(y);
  }
  if (phys < 0) return;
  for (int i = threadIdx.x; i < KW; i += blockDim.x) {
    const int head = i / D, d = i % D;
    const float x = row_values[QW + i];
    const float y = k_norm_w ? (x * k_inv) * k_norm_w[i] : x;
    k_pages[((static_cast<size_t>(phys) * nkv + head) * EI_PAGE + in_page) * D + d] =
        ei::from_f32<TO>(y);
  }
  for (int i = threadIdx.x; i < VW; i += blockDim.x) {
    const int head = i / DV, d = i % DV;
    v_pages[((static_cast<size_t>(phys) * nkv + head) * EI_PAGE + in_page) * DV + d] =
        ei::from_f32<TO>(row_values[QW + KW + i]);
  }
}

}  // namespace

// qkv: [nsplit][N, nq * D + nkv * D + nkv * DV] of in_dtype; q_out: [N, nq * D]; key pages
// [n_pages, nkv, 64, D], value pages [n_pages, nkv, 64, DV] of out_dtype; q_norm_w [nq * D] and
// k_norm_w [nkv * D] float32, or both null (no norm); bias: float32 [row width] added to the
// sums, or null.
extern "C" int ei_projection_norm_store(
    const void* qkv, int in_dtype, int nsplit, long long split_stride, const float* bias,
    const float* q_norm_w,
    const float* k_norm_w, float eps, const int32_t* row_pos, const int32_t* row_seq,
    const int32_t* page_table, int table_width, void* q_out, void* k_pages, void* v_pages,
    int out_dtype, int N, int nq, int nkv, int D, int DV, int write_cache, hipStream_t stream) {
  EI_REQUIRE(N > 0 && nq > 0 && nkv > 0 && D > 0 && DV > 0,
             "projection_norm_store: sizes must be positive");
  EI_REQUIRE(qkv && row_pos && row_seq && q_out, "projection_norm_store: null pointer");
  EI_REQUIRE((q_norm_w == nullptr) == (k_norm_w == nullptr),
             "projection_norm_store: both norm weights or neither");
  EI_REQUIRE(!write_cache || (k_pages && v_pages && page_table && table_width > 0),
             "projection_norm_store: cache pointers missing");
  EI_REQUIRE(nsplit >= 1, "projection_norm_store: nsplit must be at least 1");
  const long long width = static_cast<long long>(nq) * D + static_cast<long long>(nkv) * (D + DV);
  EI_REQUIRE(width * 4 <= 160 * 1024 - 1024, "projection_norm_store: the row does not fit in LDS");
  const size_t lds = static_cast<size_t>(width) * sizeof(float);
  const int threads = width >= 2048 ? 512 : 256;
  const size_t ss = static_cast<size_t>(split_stride);
  const bool aligned = (reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(q_out) |
                        reinterpret_cast<uintptr_t>(k_pages) | reinterpret_cast<uintptr_t>(v_pages) |
                        reinterpret_cast<uintptr_t>(q_norm_w) | reinterpret_cast<uintptr_t>(k_norm_w) |
                        reinterpret_cast<uintptr_t>(bias)) % 16 == 0;
  const bool vec = D % 4 == 0 && DV % 4 == 0 && ss % 4 == 0 && aligned;
#define EI_PNS_V(TI, TO, VV)                                                                    \
  do {                                                                                          \
    if (lds > 64 * 1024)                                                                        \
      (void)hipFuncSetAttribute(                                                                \
          reinterpret_cast<const void*>(&projection_norm_store_kernel<TI, TO, VV>),             \
          hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));                   \
    projection_norm_store_kernel<TI, TO, VV><<<N, threads, lds, stream>>>(                      \
        static_cast<const TI*>(qkv), nsplit, ss, bias, q_norm_w, k_norm_w, eps, row_pos,        \
        row_seq, page_table, table_width, static_cast<TO*>(q_out), static_cast<TO*>(k_pages),   \
        static_cast<TO*>(v_pages), nq, nkv, D, DV, write_cache);                                \
  } while (0)
#define EI_PNS_R(TI, TO, CC)                                                                    \
  projection_norm_store_reg_kernel<TI, TO, CC><<<N, 256, 0, stream>>>(                          \
      static_cast<const TI*>(qkv), nsplit, ss, bias, q_norm_w, k_norm_w, eps, row_pos, row_seq, \
      page_table, table_width, static_cast<TO*>(q_out), static_cast<TO*>(k_pages),              \
      static_cast<TO*>(v_pages), nq, nkv, D, DV, write_cache)
#define EI_PNS(TI, TO)                                   \
  do {                                                   \
    if (vec && width <= 1024) EI_PNS_R(TI, TO, 1);       \
    else if (vec && width <= 2048) EI_PNS_R(TI, TO, 2);  \
    else if (vec && width <= 4096) EI_PNS_R(TI, TO, 4);  \
    else if (vec) EI_PNS_V(TI, TO, true);                \
    else EI_PNS_V(TI, TO, false);                        \
  } while (0)
  if (in_dtype == EI_F32 && out_dtype == EI_F32) EI_PNS(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16) EI_PNS(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16) EI_PNS(bf16_t, bf16_t);
  else EI_REQUIRE(false, "projection_norm_store: unsupported dtype combination");
#undef EI_PNS
#undef EI_PNS_R
#undef EI_PNS_V
  EI_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// The store for heads whose values have a width of their own, whose rotation works out its
// angles from frequencies (angle = position * f_i as a float64 product, taken modulo 2 pi and
// rounded to float32 once, cosine and sine taken here: no table, no longest position, and the
// float32 angle is the nearest one at any position), and whose values may be mixed with the values that
// an earlier layer of the same step computed for the same token.
//
// proj: rows `row_stride` wide that begin with [q: nq * D | k: nkv * D | v: nkv * DV]
// (whatever follows is another kernel's).  One wave a (row, head).  Query and key heads:
// optional RMS norm over the head with a weight [D], then the rotation of the first R
// elements in pairs (i, i + R/2), then queries to q_out and keys to their page.  Value heads:
// v_mode 0: stored as they are; 1: also written, in float32, to v_first [N, nkv * DV];
// 2: v <- (1 - lambda) v + lambda v_first before the store (lambda one float on the device).
// temp_every > 0: a query at position p is multiplied by 1 + temp_coef ln(p' + 1), p' the whole
// part of (p + 1) / temp_every.  gate_out: the float32 sums of the nq columns from `gate_at` on
// (one number a query head) go to gate_out [N, nq] for the attention kernel's output gate.
// nkv may be 0 for rows that hold queries only (a layer that reads another layer's keys).
namespace {

constexpr int kHeadStoreMax = 8;  // elements a lane: head sizes up to 512

template <typename TI>
__device__ __forceinline__ float sliced(const TI* p, int nsplit, size_t split_stride) {
  float v = 0.f;
  for (int s = 0; s < nsplit; ++s) v += ei::to_f32<TI>(p[s * split_stride]);
  return v;
}

template <typename TI, typename TO>
__global__ void head_store_kernel(
    const TI* __restrict__ proj, int nsplit, size_t split_stride, size_t row_stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const double* __restrict__ freqs, int R, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_out, TO* __restrict__ k_pages, TO* __restrict__ v_pages,
    float* __restrict__ v_first, int v_mode, const float* __restrict__ v_lambda,
    int N, int nq, int nkv, int D, int DV, int write_cache, float temp_coef, int temp_every,
    float* __restrict__ gate_out, size_t gate_at) {
  const int heads = nq + 2 * nkv;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= N * heads) return;
  const int row = wave / heads, head = wave % heads;
  const int seq = row_seq[row];
  if (seq < 0) return;  // padding row
  const int pos = row_pos[row];
  const TI* src_row = proj + static_cast<size_t>(row) * row_stride;
  size_t page_slot = 0;   // (page, position in the page) of this row, if the cache is written
  if (write_cache)
    page_slot = static_cast<size_t>(page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE]);

  if (head >= nq + nkv) {   // a value head
    const int h = head - nq - nkv;
    const TI* src = src_row + static_cast<size_t>(nq + nkv) * D + static_cast<size_t>(h) * DV;
    float* first = v_first ? v_first + static_cast<size_t>(row) * nkv * DV + static_cast<size_t>(h) * DV
                           : nullptr;
    const float lambda = v_mode == 2 ? *v_lambda : 0.f;
    TO* dst = write_cache
                  ? v_pages + ((page_slot * nkv + h) * EI_PAGE + pos % EI_PAGE) * static_cast<size_t>(DV)
                  : nullptr;
    for (int e = lane; e < DV; e += EI_WAVE) {
      float v = sliced(src + e, nsplit, split_stride);
      if (v_mode == 1) first[e] = v;
      else if (v_mode == 2) v = (1.0f - lambda) * v + lambda * first[e];
      if (dst) dst[e] = ei::from_f32<TO>(v);
    }
    return;
  }
  const bool is_q = head < nq;
  if (!is_q && !write_cache) return;
  const TI* src = src_row + static_cast<size_t>(head) * D;
  const float* w = is_q ? q_norm_w : k_norm_w;
  const int rhalf = R / 2;
  float x[kHeadStoreMax], y[kHeadStoreMax];   // a lane's elements and their partners in the rotation
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < kHeadStoreMax; ++j) {
    const int e = lane + j * EI_WAVE;
    x[j] = y[j] = 0.f;
    if (e < D) {
      x[j] = sliced(src + e, nsplit, split_stride);
      sum += x[j] * x[j];
      if (e < R) y[j] = sliced(src + (e < rhalf ? e + rhalf : e - rhalf), nsplit, split_stride);
    }
  }
  float inv = 1.0f;
  if (w) inv = 1.0f / sqrtf(ei::wave_sum(sum) / static_cast<float>(D) + eps);
  const float warm = (is_q && temp_every > 0)
      ? 1.0f + temp_coef * logf(static_cast<float>((pos + 1) / temp_every) + 1.0f) : 1.0f;
  if (is_q && gate_out && lane == 0)
    gate_out[static_cast<size_t>(row) * nq + head] = sliced(src_row + gate_at + head, nsplit, split_stride);
  TO* dst = is_q ? q_out + (static_cast<size_t>(row) * nq + head) * D
                 : k_pages + ((page_slot * nkv + (head - nq)) * EI_PAGE + pos % EI_PAGE) * static_cast<size_t>(D);
#pragma unroll
  for (int j = 0; j < kHeadStoreMax; ++j) {
    const int e = lane + j * EI_WAVE;
    if (e >= D) continue;
    float v = w ? (x[j] * inv) * w[e] : x[j];
    if (e < R) {
      const int partner = e < rhalf ? e + rhalf : e - rhalf;
      const float p = w ? (y[j] * inv) * w[partner] : y[j];
      const double turns = static_cast<double>(pos) * freqs[e < rhalf ? e : e - rhalf] *
                           0.15915494309189535;       // in units of 2 pi
      const float angle = static_cast<float>((turns - floor(turns)) * 6.283185307179586);
      float sn, cs;
      sincosf(angle, &sn, &cs);
      v = e < rhalf ? v * cs - p * sn : v * cs + p * sn;
    }
    dst[e] = ei::from_f32<TO>(v * warm);
  }
}


template <typename TI>
__device__ __forceinline__ void sliced8(const TI* p, int nsplit, size_t split_stride, float (&v)[8]) {
  ei::VecN<TI, 8>::load(p, v);
  for (int s = 1; s < nsplit; ++s) {
    float more[8];
    ei::VecN<TI, 8>::load(p + s * split_stride, more);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] += more[i];
  }
}

// The same in 16-byte pieces, for head sizes, rotated halves and strides that are multiples of
// 8: a lane takes 8 neighbouring elements, the G lanes of a head (G the power of two at or
// above the widest head's eighth) add their squares by shuffles, and a wave takes 64 / G
// (row, head) pairs.
template <typename TI, typename TO>
__global__ void head_store_vec_kernel(
    const TI* __restrict__ proj, int nsplit, size_t split_stride, size_t row_stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const double* __restrict__ freqs, int R, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_out, TO* __restrict__ k_pages, TO* __restrict__ v_pages,
    float* __restrict__ v_first, int v_mode, const float* __restrict__ v_lambda,
    int N, int nq, int nkv, int D, int DV, int write_cache, int G, float temp_coef, int temp_every,
    float* __restrict__ gate_out, size_t gate_at) {
  const int heads = nq + 2 * nkv;
  const size_t thread = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t item = thread / G;
  const int j = static_cast<int>(thread % G);                 // which eighth of the head
  const bool in_range = item < static_cast<size_t>(N) * heads;
  const int row = in_range ? static_cast<int>(item / heads) : 0;
  const int head = in_range ? static_cast<int>(item % heads) : 0;
  const int seq = in_range ? row_seq[row] : -1;
  const bool is_q = head < nq, is_v = head >= nq + nkv;
  // (every lane stays for the shuffles; `live` says whether it has anything to do)
  const bool live = seq >= 0 && (is_q || write_cache || (is_v && v_mode == 1)) &&
                    j * 8 < (is_v ? DV : D);
  const int pos = seq >= 0 ? row_pos[row] : 0;
  const TI* src_row = proj + static_cast<size_t>(row) * row_stride;
  size_t page = 0;
  if (live && write_cache)
    page = static_cast<size_t>(page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE]);
  float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (is_v) {
    if (!live) return;          // (value heads take no part in any shuffle: whole groups leave)
    const int h = head - nq - nkv;
    sliced8(src_row + static_cast<size_t>(nq + nkv) * D + static_cast<size_t>(h) * DV + j * 8, nsplit,
            split_stride, x);
    if (v_mode) {
      float* first = v_first + static_cast<size_t>(row) * nkv * DV + static_cast<size_t>(h) * DV + j * 8;
      if (v_mode == 1) {
        ei::VecN<float, 8>::store(first, x);
      } else {
        const float lambda = *v_lambda;
        float kept[8];
        ei::VecN<float, 8>::load(first, kept);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = (1.0f - lambda) * x[i] + lambda * kept[i];
      }
    }
    if (write_cache)
      ei::VecN<TO, 8>::store(
          v_pages + ((page * nkv + h) * EI_PAGE + pos % EI_PAGE) * static_cast<size_t>(DV) + j * 8, x);
    return;
  }
  const TI* src = src_row + static_cast<size_t>(head) * D;
  const float* w = is_q ? q_norm_w : k_norm_w;
  const int e0 = j * 8, rhalf = R / 2;
  const bool turns = live && e0 < R;
  const int partner0 = e0 < rhalf ? e0 + rhalf : e0 - rhalf;
  float y[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (live) sliced8(src + e0, nsplit, split_stride, x);
  if (turns) sliced8(src + partner0, nsplit, split_stride, y);
  float inv = 1.0f;
  if (w) {                      // (uniform: every lane of the wave takes the shuffles)
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += x[i] * x[i];
    for (int offset = G / 2; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset, EI_WAVE);
    inv = 1.0f / sqrtf(sum / static_cast<float>(D) + eps);
  }
  if (!live) return;
  if (w) {
    float wx[8];
    ei::VecN<float, 8>::load(w + e0, wx);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = (x[i] * inv) * wx[i];
    if (turns) {
      ei::VecN<float, 8>::load(w + partner0, wx);
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = (y[i] * inv) * wx[i];
    }
  }
  if (turns) {
    const int f0 = e0 < rhalf ? e0 : e0 - rhalf;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const double whole = static_cast<double>(pos) * freqs[f0 + i] * 0.15915494309189535;
      const float angle = static_cast<float>((whole - floor(whole)) * 6.283185307179586);
      float sn, cs;
      sincosf(angle, &sn, &cs);
      x[i] = e0 < rhalf ? x[i] * cs - y[i] * sn : x[i] * cs + y[i] * sn;
    }
  }
  if (is_q && temp_every > 0) {
    const float warm = 1.0f + temp_coef * logf(static_cast<float>((pos + 1) / temp_every) + 1.0f);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] *= warm;
  }
  if (is_q && gate_out && j == 0)
    gate_out[static_cast<size_t>(row) * nq + head] = sliced(src_row + gate_at + head, nsplit, split_stride);
  TO* dst = is_q ? q_out + (static_cast<size_t>(row) * nq + head) * D
                 : k_pages + ((page * nkv + (head - nq)) * EI_PAGE + pos % EI_PAGE) * static_cast<size_t>(D);
  ei::VecN<TO, 8>::store(dst + e0, x);
}

}  // namespace

extern "C" int ei_head_store(
    const void* proj, int in_dtype, int nsplit, long long split_stride, long long row_stride,
    const float* q_norm_w, const float* k_norm_w, float eps, const double* freqs, int rot_dim,
    const int32_t* row_pos, const int32_t* row_seq, const int32_t* page_table, int table_width,
    void* q_out, void* k_pages, void* v_pages, int out_dtype, float* v_first, int v_mode,
    const float* v_lambda, int N, int nq, int nkv, int D, int DV, int write_cache,
    float temp_coef, int temp_every, float* gate_out, long long gate_at, hipStream_t stream) {
  EI_REQUIRE(N > 0 && nq > 0 && nkv >= 0 && D > 0 && DV > 0, "head_store: sizes must be positive");
  EI_REQUIRE(nkv > 0 || !write_cache, "head_store: rows without keys cannot write the cache");
  EI_REQUIRE(temp_every >= 0, "head_store: negative temperature step");
  EI_REQUIRE(!gate_out || (gate_at >= 0 && row_stride >= gate_at + nq),
             "head_store: rows narrower than the gate's columns");
  EI_REQUIRE(D <= kHeadStoreMax * EI_WAVE, "head_store: head_dim above 512");
  EI_REQUIRE(proj && row_pos && row_seq && q_out && nsplit >= 1, "head_store: bad arguments");
  EI_REQUIRE(row_stride >= static_cast<long long>(nq + nkv) * D + static_cast<long long>(nkv) * DV,
             "head_store: rows narrower than the projections");
  EI_REQUIRE(!write_cache || (k_pages && v_pages && page_table && table_width > 0),
             "head_store: cache pointers missing");
  EI_REQUIRE((q_norm_w == nullptr) == (k_norm_w == nullptr), "head_store: both norm weights or neither");
  const int R = freqs ? rot_dim : 0;
  EI_REQUIRE(R % 2 == 0 && R >= 0 && R <= D, "head_store: the rotated width must be even and at most head_dim");
  EI_REQUIRE(v_mode >= 0 && v_mode <= 2 && (v_mode == 0 || v_first) && (v_mode != 2 || v_lambda),
             "head_store: value mixing needs its buffer and its weight");
  const int heads = nq + 2 * nkv;
  const int threads = 256;
  const size_t waves = static_cast<size_t>(N) * heads;
  const unsigned blocks = static_cast<unsigned>((waves * EI_WAVE + threads - 1) / threads);
  const size_t ss = static_cast<size_t>(split_stride), rs = static_cast<size_t>(row_stride);
  // 16-byte pieces where every head, rotated half and stride is a multiple of 8
  const auto aligned16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = D % 8 == 0 && DV % 8 == 0 && R % 16 == 0 && rs % 8 == 0 && (nsplit == 1 || ss % 8 == 0) &&
                   aligned16(proj) && aligned16(q_out) && aligned16(k_pages) && aligned16(v_pages) &&
                   aligned16(v_first) && aligned16(q_norm_w) && aligned16(k_norm_w);
  if (vec) {
    int G = 1;
    while (G * 8 < (D > DV ? D : DV)) G *= 2;
    const size_t lanes = waves * G;
    const unsigned vblocks = static_cast<unsigned>((lanes + threads - 1) / threads);
#define EI_HSV(TI, TO)                                                                         \
  head_store_vec_kernel<TI, TO><<<vblocks, threads, 0, stream>>>(                              \
      static_cast<const TI*>(proj), nsplit, ss, rs, q_norm_w, k_norm_w, eps, freqs, R, row_pos, \
      row_seq, page_table, table_width, static_cast<TO*>(q_out), static_cast<TO*>(k_pages),    \
      static_cast<TO*>(v_pages), v_first, v_mode, v_lambda, N, nq, nkv, D, DV, write_cache, G,  \
      temp_coef, temp_every, gate_out, static_cast<size_t>(gate_at))
    if (in_dtype == EI_F32 && out_dtype == EI_F32) EI_HSV(float, float);
    else if (in_dtype == EI_F32 && out_dtype == EI_BF16) EI_HSV(float, bf16_t);
    else if (in_dtype == EI_BF16 && out_dtype == EI_BF16) EI_HSV(bf16_t, bf16_t);
    else EI_REQUIRE(false, "head_store: unsupported dtype combination");
#undef EI_HSV
    EI_LAUNCH_CHECK();
  }
#define EI_HS(TI, TO)                                                                          \
  head_store_kernel<TI, TO><<<blocks, threads, 0, stream>>>(                                   \
      static_cast<const TI*>(proj), nsplit, ss, rs, q_norm_w, k_norm_w, eps, freqs, R, row_pos, \
      row_seq, page_table, table_width, static_cast<TO*>(q_out), static_cast<TO*>(k_pages),    \
      static_cast<TO*>(v_pages), v_first, v_mode, v_lambda, N, nq, nkv, D, DV, write_cache,     \
      temp_coef, temp_every, gate_out, static_cast<size_t>(gate_at))
  if (in_dtype == EI_F32 && out_dtype == EI_F32) EI_HS(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16) EI_HS(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16) EI_HS(bf16_t, bf16_t);
  else EI_REQUIRE(false, "head_store: unsupported dtype combination");
#undef EI_HS
  EI_LAUNCH_CHECK();
}

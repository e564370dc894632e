// Routed feed-forward (mixture of experts): router, and the experts of every row's choice.
//
// Router: logits z = W_router x in float32 (W_router is kept in float32; x is read as stored),
// the `top` experts of largest logit (of equal logits the one of lower index), and their
// weights softmax(z over the chosen ones only); or (`mode` 1) the scores s = softmax(z) over all
// router outputs, the `top` outputs of largest s + correction (a learned number per output,
// null: none), and the weights s of the chosen, not renormalised.  Experts: for row r and its
// choice k with expert e and weight p,  y_r += p W_down,e (silu(W_gate,e x_r) * (W_up,e x_r)).
// A router may have more outputs than there are experts: an output beyond the experts is an
// identity expert, which adds p x_r and has no matrices.
//
// Two forms of the experts.  One takes a (row, choice) pair at a time and streams the expert's
// matrices for it: any type and any sizes.  The other (bfloat16, widths that are multiples of
// 64) lays the pairs out by expert on the device and runs every expert's pairs against its
// matrices as tiles on the matrix cores.  The matrices of all experts lie stacked: gate and up
// [E, F, W], down [E, W, F].
#include "common.h"
#include <float.h>

namespace {

constexpr int kMaxTop = 64;
constexpr int kRouteMax = 8;      // experts a lane holds: up to 512 experts

// A block of four waves a row: the waves share the experts' logits out, the first wave chooses.
template <typename TX>
__global__ void __launch_bounds__(256)
moe_route_kernel(const TX* __restrict__ x, const float* __restrict__ w_router,
                 const int32_t* __restrict__ row_seq, int32_t* __restrict__ expert,
                 float* __restrict__ weight, int N, int W, int E, int top, int mode,
                 const float* __restrict__ correction) {
  __shared__ float logits[kRouteMax * EI_WAVE];
  const int wave = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  const int row = blockIdx.x;
  int32_t* e_out = expert + static_cast<size_t>(row) * top;
  float* w_out = weight + static_cast<size_t>(row) * top;
  if (row_seq && row_seq[row] < 0) {            // a padding row: no expert has anything to add
    for (int k = threadIdx.x; k < top; k += blockDim.x) { e_out[k] = 0; w_out[k] = 0.f; }
    return;
  }
  const TX* xr = x + static_cast<size_t>(row) * W;
  for (int e = wave; e < E; e += 4) {
    const float* wr = w_router + static_cast<size_t>(e) * W;
    float sum = 0.f;
    if (W % 4 == 0) {
#pragma unroll 4
      for (int i = lane * 4; i < W; i += EI_WAVE * 4) {
        float xv[4], wv[4];
        ei::Vec4<TX>::load(xr + i, xv);
        ei::Vec4<float>::load(wr + i, wv);
        sum += xv[0] * wv[0];
        sum += xv[1] * wv[1];
        sum += xv[2] * wv[2];
        sum += xv[3] * wv[3];
      }
    } else {
      for (int i = lane; i < W; i += EI_WAVE) sum += ei::to_f32<TX>(xr[i]) * wr[i];
    }
    sum = ei::wave_sum(sum);
    if (!(sum > -FLT_MAX)) sum = -FLT_MAX;      // (a NaN chooses nothing ahead of a number)
    if (lane == 0) logits[e] = sum;
  }
  __syncthreads();
  if (wave != 0) return;
  float z[kRouteMax];
#pragma unroll
  for (int j = 0; j < kRouteMax; ++j) z[j] = lane + j * EI_WAVE < E ? logits[lane + j * EI_WAVE] : -FLT_MAX;
  float score[kRouteMax];                        // mode 1: the softmax over all outputs
  if (mode == 1) {
    float top_z = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < kRouteMax; ++j) top_z = fmaxf(top_z, z[j]);
    top_z = ei::wave_max(top_z);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < kRouteMax; ++j) {
      score[j] = lane + j * EI_WAVE < E ? expf(z[j] - top_z) : 0.f;
      sum += score[j];
    }
    sum = ei::wave_sum(sum);
#pragma unroll
    for (int j = 0; j < kRouteMax; ++j) {
      const int e = lane + j * EI_WAVE;
      score[j] = score[j] / sum;
      // what the choice goes by from here on
      z[j] = e < E ? score[j] + (correction ? correction[e] : 0.f) : -FLT_MAX;
    }
  }
  unsigned taken = 0;                            // bit j: this lane's expert lane + 64 j is chosen
  float total = 0.f, largest = 0.f;
  float mine = 0.f;                              // lane k keeps the k-th choice
  int mine_e = 0;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < kRouteMax; ++j) {
      const int e = lane + j * EI_WAVE;
      if (e < E && !(taken >> j & 1u) && z[j] > best) { best = z[j]; best_e = e; }
    }
    for (int offset = EI_WAVE / 2; offset > 0; offset >>= 1) {
      const float other = __shfl_xor(best, offset, EI_WAVE);
      const int other_e = __shfl_xor(best_e, offset, EI_WAVE);
      if (other > best || (other == best && other_e < best_e)) { best = other; best_e = other_e; }
    }
    float chosen_score = 0.f;                    // mode 1: the score of the choice, from its lane
    if (best_e % EI_WAVE == lane) {
      taken |= 1u << (best_e / EI_WAVE);
      if (mode == 1) {
#pragma unroll
        for (int j = 0; j < kRouteMax; ++j)
          if (j == best_e / EI_WAVE) chosen_score = score[j];
      }
    }
    if (mode == 1) chosen_score = __shfl(chosen_score, best_e % EI_WAVE, EI_WAVE);
    if (k == 0) largest = best;
    total += expf(best - largest);
    if (lane == k) { mine = mode == 1 ? chosen_score : best; mine_e = best_e; }
  }
  if (lane < top) {
    e_out[lane] = mine_e;
    w_out[lane] = mode == 1 ? mine : expf(mine - largest) / total;
  }
}

// act [N * top, F] = silu(W_gate,e x) * (W_up,e x) for every (row, choice).  A block a pair and
// a strip of 16 outputs; a wave takes four outputs at a time.
template <typename T>
__global__ void __launch_bounds__(256)
moe_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ w_gate, const T* __restrict__ w_up,
                   const int32_t* __restrict__ expert, const float* __restrict__ weight,
                   T* __restrict__ act, int W, int F, int top, int E) {
  const int pair = blockIdx.x;
  if (weight[pair] == 0.f) return;              // a padding row's choice
  const int row = pair / top, e = expert[pair];
  if (e >= E) return;                           // an identity expert has no product
  const int wave = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  const int f0 = blockIdx.y * 16 + wave * 4;
  if (f0 >= F) return;
  const T* xr = x + static_cast<size_t>(row) * W;
  const T* g = w_gate + (static_cast<size_t>(e) * F + f0) * W;
  const T* u = w_up + (static_cast<size_t>(e) * F + f0) * W;
  const int nf = min(4, F - f0);
  float sg[4] = {0.f, 0.f, 0.f, 0.f}, su[4] = {0.f, 0.f, 0.f, 0.f};
  if (W % 8 == 0) {
    for (int i = lane * 8; i < W; i += EI_WAVE * 8) {
      float xv[8];
      ei::VecN<T, 8>::load(xr + i, xv);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (q < nf) {
          float a[8], b[8];
          ei::VecN<T, 8>::load(g + static_cast<size_t>(q) * W + i, a);
          ei::VecN<T, 8>::load(u + static_cast<size_t>(q) * W + i, b);
#pragma unroll
          for (int v = 0; v < 8; ++v) { sg[q] += a[v] * xv[v]; su[q] += b[v] * xv[v]; }
        }
      }
    }
  } else {
    for (int i = lane; i < W; i += EI_WAVE) {
      const float xv = ei::to_f32<T>(xr[i]);
      for (int q = 0; q < nf; ++q) {
        sg[q] += ei::to_f32<T>(g[static_cast<size_t>(q) * W + i]) * xv;
        su[q] += ei::to_f32<T>(u[static_cast<size_t>(q) * W + i]) * xv;
      }
    }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float gate = ei::wave_sum(sg[q]), up = ei::wave_sum(su[q]);
    if (lane == 0 && q < nf)
      act[static_cast<size_t>(pair) * F + f0 + q] = ei::from_f32<T>(gate / (1.0f + expf(-gate)) * up);
  }
}

// out [N, W] float32 = sum over a row's choices of weight * W_down,e act.  A block a row and a
// strip of 16 columns; a wave takes four columns at a time.
template <typename T>
__global__ void __launch_bounds__(256)
moe_down_kernel(const T* __restrict__ act, const T* __restrict__ w_down,
                const int32_t* __restrict__ expert, const float* __restrict__ weight,
                float* __restrict__ out, int W, int F, int top, int E, const T* __restrict__ x) {
  const int row = blockIdx.x;
  const int wave = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  const int c0 = blockIdx.y * 16 + wave * 4;
  if (c0 >= W) return;
  const int nc = min(4, W - c0);
  float total[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < top; ++k) {
    const int pair = row * top + k;
    const float p = weight[pair];
    if (p == 0.f) continue;
    if (expert[pair] >= E) {                    // an identity expert: the row itself
      for (int q = 0; q < nc; ++q)
        total[q] += p * ei::to_f32<T>(x[static_cast<size_t>(row) * W + c0 + q]);
      continue;
    }
    const T* a = act + static_cast<size_t>(pair) * F;
    const T* d = w_down + (static_cast<size_t>(expert[pair]) * W + c0) * F;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    if (F % 8 == 0) {
      for (int i = lane * 8; i < F; i += EI_WAVE * 8) {
        float av[8];
        ei::VecN<T, 8>::load(a + i, av);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (q < nc) {
            float dv[8];
            ei::VecN<T, 8>::load(d + static_cast<size_t>(q) * F + i, dv);
#pragma unroll
            for (int v = 0; v < 8; ++v) s[q] += dv[v] * av[v];
          }
        }
      }
    } else {
      for (int i = lane; i < F; i += EI_WAVE) {
        const float av = ei::to_f32<T>(a[i]);
        for (int q = 0; q < nc; ++q) s[q] += ei::to_f32<T>(d[static_cast<size_t>(q) * F + i]) * av;
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) total[q] += p * ei::wave_sum(s[q]);
  }
  if (lane == 0)
    for (int q = 0; q < nc; ++q) out[static_cast<size_t>(row) * W + c0 + q] = total[q];
}


// ---------------------------------------------------------------------------------------
// The experts as grouped matrix products on the matrix cores (bfloat16, K a multiple of 64).
//
// moe_group: the (row, choice) pairs counted and laid out by expert: `sorted` [P] holds the
// pairs of expert 0, then those of expert 1, ...; `place` [P] is where a pair went (-1: a pair
// of weight 0, which is left out; -2: a pair of an identity expert, an output of the router
// beyond the E experts); `starts` [E + 1] are the experts' first places.  Which place
// a pair gets inside its expert's span depends on the order of the atomics; every pair is
// computed for itself, so no result depends on it.
__global__ void __launch_bounds__(1024)
moe_group_kernel(const int32_t* __restrict__ expert, const float* __restrict__ weight,
                 int32_t* __restrict__ sorted, int32_t* __restrict__ place,
                 int32_t* __restrict__ starts, int P, int E) {
  __shared__ int counts[kRouteMax * EI_WAVE], cursor[kRouteMax * EI_WAVE];
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x)
    if (weight[p] != 0.f && expert[p] < E) atomicAdd(&counts[expert[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      starts[e] = at;
      cursor[e] = at;
      at += counts[e];
    }
    starts[E] = at;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    int q = -1;
    if (weight[p] != 0.f) {
      if (expert[p] < E) {
        q = atomicAdd(&cursor[expert[p]], 1);
        sorted[q] = p;
      } else {
        q = -2;
      }
    }
    place[p] = q;
  }
}

typedef __bf16 moe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float moe_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileN = 64, kTileK = 64;      // (kTileK: the least K-tile; K must be a multiple)

// One tile of MB * 16 places of one expert against 64 rows of its matrix (GATED: of its gate
// and of its up matrix).  GATED: the rows of `a` are gathered (row = pair / top) and
// silu(gate) * up goes to `out_act` [P, N] at the pairs' places; else the rows of `a` are the
// places themselves and the float32 products go to `out_sum` [P, N].  A wave owns 16 rows of
// the matrix, which it reads from global memory straight into operand registers one K-tile
// ahead; the places' rows travel through LDS (16-byte chunks stored at chunk ^ row % 8).  KT is
// the K-tile: 64 for the large tiles of prompts, 256 for the small ones of decoding, where a
// wave has little to multiply and lives on how many loads of the matrix it keeps in flight.
template <int MB, bool GATED, int KT>
__global__ void __launch_bounds__(256)
moe_gemm_kernel(const bf16_t* __restrict__ a, const int32_t* __restrict__ sorted,
                const int32_t* __restrict__ starts, const bf16_t* __restrict__ w1,
                const bf16_t* __restrict__ w2, bf16_t* __restrict__ out_act,
                float* __restrict__ out_sum, int E, int N, int K, int top) {
  constexpr int TM = MB * 16;
  constexpr int PER_THREAD = TM * (KT / 8) / 256 > 0 ? TM * (KT / 8) / 256 : 1;
  __shared__ __attribute__((aligned(16))) bf16_t xs[TM * KT];
  __shared__ int tile_info[2];
  if (threadIdx.x == 0) {       // which expert's tile this block is
    int t = blockIdx.x, found = -1, m0 = 0;
    for (int e = 0; e < E; ++e) {
      const int count = starts[e + 1] - starts[e];
      const int tiles = (count + TM - 1) / TM;
      if (t < tiles) { found = e; m0 = t * TM; break; }
      t -= tiles;
    }
    tile_info[0] = found;
    tile_info[1] = m0;
  }
  __syncthreads();
  const int e = tile_info[0];
  if (e < 0) return;
  const int first = starts[e] + tile_info[1];                 // the tile's first place
  const int valid = min(TM, starts[e + 1] - first);           // places of the tile that exist
  const int wave = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  const int r16 = lane % 16, quarter = lane / 16;
  const int n_wave = blockIdx.y * kTileN + wave * 16;         // the wave's first matrix row
  const int n_row = min(n_wave + r16, N - 1);                 // (clamped: rows beyond N are not stored)
  const bf16_t* w1_row = w1 + (static_cast<size_t>(e) * N + n_row) * K + quarter * 8;
  const bf16_t* w2_row = GATED ? w2 + (static_cast<size_t>(e) * N + n_row) * K + quarter * 8 : nullptr;
  // the chunks of the places' rows that this thread carries into LDS
  const bf16_t* src[PER_THREAD];
  int dst[PER_THREAD];
#pragma unroll
  for (int i = 0; i < PER_THREAD; ++i) {
    const int index = threadIdx.x + i * 256;
    const int row = index / (KT / 8), chunk = index % (KT / 8);
    const int at = first + min(row, valid - 1);               // (clamped: such rows are not stored)
    const size_t source_row = GATED ? static_cast<size_t>(sorted[at] / top) : static_cast<size_t>(at);
    src[i] = a + source_row * K + chunk * 8;
    dst[i] = row * KT + ((chunk ^ (row % 8)) * 8);
  }
  const bool carries = threadIdx.x < TM * (KT / 8);      // (tiles of fewer chunks than threads)
  moe_f32x4 acc1[MB], acc2[GATED ? MB : 1];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    acc1[mb] = moe_f32x4{0.f, 0.f, 0.f, 0.f};
    if (GATED) acc2[mb] = moe_f32x4{0.f, 0.f, 0.f, 0.f};
  }
  uint4 x_next[PER_THREAD];
  constexpr int STEPS = KT / 32;
  moe_bf16x8 wa[STEPS], wb[GATED ? STEPS : 1], wa_next[STEPS], wb_next[GATED ? STEPS : 1];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i)
      if (carries) x_next[i] = *reinterpret_cast<const uint4*>(src[i] + k0);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      wa_next[s] = *reinterpret_cast<const moe_bf16x8*>(w1_row + k0 + s * 32);
      if (GATED) wb_next[s] = *reinterpret_cast<const moe_bf16x8*>(w2_row + k0 + s * 32);
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += KT) {
    __syncthreads();                       // everybody has read the tile before
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i)
      if (carries) *reinterpret_cast<uint4*>(&xs[dst[i]]) = x_next[i];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      wa[s] = wa_next[s];
      if (GATED) wb[s] = wb_next[s];
    }
    __syncthreads();
    if (k0 + KT < K) fetch(k0 + KT);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int row = mb * 16 + r16, chunk = s * 4 + quarter;
        const moe_bf16x8 xf = *reinterpret_cast<const moe_bf16x8*>(
            &xs[row * KT + ((chunk ^ (row % 8)) * 8)]);
        acc1[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[s], xf, acc1[mb], 0, 0, 0);
        if (GATED) acc2[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[s], xf, acc2[mb], 0, 0, 0);
      }
    }
  }
  // lane (r16, quarter) holds, of place mb * 16 + r16, the matrix rows n_wave + 4 quarter + i
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int row = mb * 16 + r16;
    if (row >= valid) continue;
    const size_t at = static_cast<size_t>(first + row) * N;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n_wave + 4 * quarter + i;
      if (n >= N) continue;
      if (GATED) {
        const float gate = acc1[mb][i], up = acc2[mb][i];
        out_act[at + n] = ei::f32_to_bf16(gate / (1.0f + expf(-gate)) * up);
      } else {
        out_sum[at + n] = acc1[mb][i];
      }
    }
  }
}

// out [rows, W] = sum over a row's choices of weight * the choice's product row.
__global__ void moe_combine_kernel(const float* __restrict__ sums, const int32_t* __restrict__ place,
                                   const float* __restrict__ weight, float* __restrict__ out,
                                   int W, int top, size_t total, const bf16_t* __restrict__ x) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t idx = start; idx < total; idx += step) {
    const size_t row = idx / W, col = idx % W;
    float sum = 0.f;
    for (int k = 0; k < top; ++k) {
      const int q = place[row * top + k];
      if (q >= 0) sum += weight[row * top + k] * sums[static_cast<size_t>(q) * W + col];
      else if (q == -2) sum += weight[row * top + k] * ei::bf16_to_f32(x[idx]);   // identity
    }
    out[idx] = sum;
  }
}

}  // namespace

extern "C" int ei_moe_route(const void* x, int x_dtype, const float* w_router, const int32_t* row_seq,
                            int32_t* expert, float* weight, int N, int W, int E, int top,
                            int mode, const float* correction, hipStream_t stream) {
  EI_REQUIRE(x && w_router && expert && weight && N > 0 && W > 0, "moe_route: bad arguments");
  EI_REQUIRE(E >= 1 && E <= kRouteMax * EI_WAVE && top >= 1 && top <= E && top <= kMaxTop,
             "moe_route: up to 512 experts, of which 1 to 64 are chosen");
  EI_REQUIRE(mode == 0 || mode == 1, "moe_route: unknown mode");
  const int threads = 256;
  const unsigned blocks = static_cast<unsigned>(N);
  if (x_dtype == EI_F32)
    moe_route_kernel<float><<<blocks, threads, 0, stream>>>(static_cast<const float*>(x), w_router,
                                                            row_seq, expert, weight, N, W, E, top,
                                                            mode, correction);
  else if (x_dtype == EI_BF16)
    moe_route_kernel<bf16_t><<<blocks, threads, 0, stream>>>(static_cast<const bf16_t*>(x), w_router,
                                                             row_seq, expert, weight, N, W, E, top,
                                                            mode, correction);
  else
    EI_REQUIRE(false, "moe_route: unknown dtype");
  EI_LAUNCH_CHECK();
}

extern "C" int ei_moe_experts(const void* x, const void* w_gate, const void* w_up, const void* w_down,
                              int dtype, const int32_t* expert, const float* weight, void* act,
                              float* out, int N, int W, int F, int E, int top, hipStream_t stream) {
  EI_REQUIRE(x && w_gate && w_up && w_down && expert && weight && act && out, "moe_experts: null pointer");
  EI_REQUIRE(N > 0 && W > 0 && F > 0 && top >= 1, "moe_experts: sizes must be positive");
  EI_REQUIRE(static_cast<long long>(N) * top <= 0x7fffffffLL && (F + 15) / 16 <= 65535 &&
                 (W + 15) / 16 <= 65535, "moe_experts: too large for one launch");
  const dim3 grid_up(N * top, (F + 15) / 16), grid_down(N, (W + 15) / 16);
#define EI_MOE(T)                                                                              \
  do {                                                                                         \
    moe_gate_up_kernel<T><<<grid_up, 256, 0, stream>>>(                                        \
        static_cast<const T*>(x), static_cast<const T*>(w_gate), static_cast<const T*>(w_up),  \
        expert, weight, static_cast<T*>(act), W, F, top, E);                                   \
    moe_down_kernel<T><<<grid_down, 256, 0, stream>>>(                                         \
        static_cast<const T*>(act), static_cast<const T*>(w_down), expert, weight, out, W, F, top, \
        E, static_cast<const T*>(x));                                                          \
  } while (0)
  if (dtype == EI_F32) EI_MOE(float);
  else if (dtype == EI_BF16) EI_MOE(bf16_t);
  else EI_REQUIRE(false, "moe_experts: unknown dtype");
#undef EI_MOE
  EI_LAUNCH_CHECK();
}

// Whether `ei_moe_experts_grouped` takes these sizes.
extern "C" int ei_moe_grouped_supported(int dtype, int W, int F, int E) {
  return dtype == EI_BF16 && W % kTileK == 0 && F % kTileK == 0 && E <= kRouteMax * EI_WAVE ? 1 : 0;
}

// The experts as grouped products.  Scratch: sorted, place [P] and starts [E + 1] int32,
// act [P, F] bfloat16, sums [P, W] float32, with P = N * top.
extern "C" int ei_moe_experts_grouped(const void* x, const void* w_gate, const void* w_up,
                                      const void* w_down, const int32_t* expert, const float* weight,
                                      int32_t* sorted, int32_t* place, int32_t* starts, void* act,
                                      float* sums, float* out, int N, int W, int F, int E, int top,
                                      hipStream_t stream) {
  EI_REQUIRE(x && w_gate && w_up && w_down && expert && weight && sorted && place && starts && act &&
                 sums && out, "moe_experts_grouped: null pointer");
  EI_REQUIRE(N > 0 && top >= 1 && E >= 1 && ei_moe_grouped_supported(EI_BF16, W, F, E),
             "moe_experts_grouped: sizes it does not take");
  const long long pairs = static_cast<long long>(N) * top;
  EI_REQUIRE(pairs <= 0x3fffffffLL, "moe_experts_grouped: too many rows for one launch");
  const int P = static_cast<int>(pairs);
  moe_group_kernel<<<1, 1024, 0, stream>>>(expert, weight, sorted, place, starts, P, E);
  const bf16_t* xb = static_cast<const bf16_t*>(x);
  const bf16_t* g = static_cast<const bf16_t*>(w_gate);
  const bf16_t* u = static_cast<const bf16_t*>(w_up);
  const bf16_t* d = static_cast<const bf16_t*>(w_down);
  bf16_t* ab = static_cast<bf16_t*>(act);
  // tiles of 32 places while an expert has few (decoding), of 128 for prompts
  if (P <= 32 * E) {
    const unsigned tiles = static_cast<unsigned>((P + 31) / 32 + E);
    const dim3 grid_up(tiles, (F + kTileN - 1) / kTileN), grid_down(tiles, (W + kTileN - 1) / kTileN);
    // (the long K-tile where few experts are at work and their waves cannot fill the chip:
    // measured at 2, 16 and 128 pairs over 8 experts of 2,816 x 2,048)
    const bool few = P <= 4;
    if (few && W % 256 == 0)
      moe_gemm_kernel<2, true, 256><<<grid_up, 256, 0, stream>>>(xb, sorted, starts, g, u, ab, nullptr, E, F, W, top);
    else
      moe_gemm_kernel<2, true, 64><<<grid_up, 256, 0, stream>>>(xb, sorted, starts, g, u, ab, nullptr, E, F, W, top);
    if (few && F % 256 == 0)
      moe_gemm_kernel<2, false, 256><<<grid_down, 256, 0, stream>>>(ab, sorted, starts, d, nullptr, nullptr, sums, E, W, F, top);
    else
      moe_gemm_kernel<2, false, 64><<<grid_down, 256, 0, stream>>>(ab, sorted, starts, d, nullptr, nullptr, sums, E, W, F, top);
  } else {
    const unsigned tiles = static_cast<unsigned>((P + 127) / 128 + E);
    moe_gemm_kernel<8, true, 64><<<dim3(tiles, (F + kTileN - 1) / kTileN), 256, 0, stream>>>(
        xb, sorted, starts, g, u, ab, nullptr, E, F, W, top);
    moe_gemm_kernel<8, false, 64><<<dim3(tiles, (W + kTileN - 1) / kTileN), 256, 0, stream>>>(
        ab, sorted, starts, d, nullptr, nullptr, sums, E, W, F, top);
  }
  const size_t total = static_cast<size_t>(N) * W;
  size_t blocks = (total + 255) / 256;
  if (blocks > static_cast<size_t>(ei_compute_units()) * 16) blocks = static_cast<size_t>(ei_compute_units()) * 16;
  moe_combine_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(sums, place, weight, out, W, top, total, xb);
  EI_LAUNCH_CHECK();
}

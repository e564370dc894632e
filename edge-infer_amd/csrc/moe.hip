// Routed feed-forward (mixture of experts): router, and the experts of every row's choice.
//
// Router: logits z = W_router x in float32 (W_router is kept in float32; x is read as stored),
// the `top` experts of largest logit (of equal logits the one of lower index), and their
// weights softmax(z over the chosen ones only).  Experts: for row r and its choice k with expert
// e and weight p,  y_r += p W_down,e (silu(W_gate,e x_r) * (W_up,e x_r)).
//
// These kernels take a row's experts one (row, choice) pair at a time and stream the expert's
// matrices for it: the form for few rows (decoding), and a correct one for any number.  The
// matrices of all experts lie stacked: gate and up [E, F, W], down [E, W, F].
#include "common.h"
#include <float.h>

namespace {

constexpr int kMaxTop = 64;
constexpr int kRouteMax = 8;      // experts a lane holds: up to 512 experts

// A wave a row.
template <typename TX>
__global__ void moe_route_kernel(const TX* __restrict__ x, const float* __restrict__ w_router,
                                 const int32_t* __restrict__ row_seq, int32_t* __restrict__ expert,
                                 float* __restrict__ weight, int N, int W, int E, int top) {
  const int wave_in_block = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  const int row = blockIdx.x * (blockDim.x / EI_WAVE) + wave_in_block;
  if (row >= N) return;
  int32_t* e_out = expert + static_cast<size_t>(row) * top;
  float* w_out = weight + static_cast<size_t>(row) * top;
  if (row_seq && row_seq[row] < 0) {            // a padding row: no expert has anything to add
    for (int k = lane; k < top; k += EI_WAVE) { e_out[k] = 0; w_out[k] = 0.f; }
    return;
  }
  const TX* xr = x + static_cast<size_t>(row) * W;
  float z[kRouteMax];
#pragma unroll
  for (int j = 0; j < kRouteMax; ++j) z[j] = -FLT_MAX;
  for (int e = 0; e < E; ++e) {
    const float* wr = w_router + static_cast<size_t>(e) * W;
    float sum = 0.f;
    for (int i = lane; i < W; i += EI_WAVE) sum += ei::to_f32<TX>(xr[i]) * wr[i];
    sum = ei::wave_sum(sum);
    if (!(sum > -FLT_MAX)) sum = -FLT_MAX;      // (a NaN chooses nothing ahead of a number)
    if (e % EI_WAVE == lane) {
#pragma unroll
      for (int j = 0; j < kRouteMax; ++j)
        if (j == e / EI_WAVE) z[j] = sum;
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
    if (best_e % EI_WAVE == lane) taken |= 1u << (best_e / EI_WAVE);
    if (k == 0) largest = best;
    total += expf(best - largest);
    if (lane == k) { mine = best; mine_e = best_e; }
  }
  if (lane < top) {
    e_out[lane] = mine_e;
    w_out[lane] = expf(mine - largest) / total;
  }
}

// act [N * top, F] = silu(W_gate,e x) * (W_up,e x) for every (row, choice).  A block a pair and
// a strip of 16 outputs; a wave takes four outputs at a time.
template <typename T>
__global__ void __launch_bounds__(256)
moe_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ w_gate, const T* __restrict__ w_up,
                   const int32_t* __restrict__ expert, const float* __restrict__ weight,
                   T* __restrict__ act, int W, int F, int top) {
  const int pair = blockIdx.x;
  if (weight[pair] == 0.f) return;              // a padding row's choice
  const int row = pair / top, e = expert[pair];
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
                float* __restrict__ out, int W, int F, int top) {
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

}  // namespace

extern "C" int ei_moe_route(const void* x, int x_dtype, const float* w_router, const int32_t* row_seq,
                            int32_t* expert, float* weight, int N, int W, int E, int top,
                            hipStream_t stream) {
  EI_REQUIRE(x && w_router && expert && weight && N > 0 && W > 0, "moe_route: bad arguments");
  EI_REQUIRE(E >= 1 && E <= kRouteMax * EI_WAVE && top >= 1 && top <= E && top <= kMaxTop,
             "moe_route: up to 512 experts, of which 1 to 64 are chosen");
  const int threads = 256;
  const unsigned blocks = static_cast<unsigned>((N + 3) / 4);
  if (x_dtype == EI_F32)
    moe_route_kernel<float><<<blocks, threads, 0, stream>>>(static_cast<const float*>(x), w_router,
                                                            row_seq, expert, weight, N, W, E, top);
  else if (x_dtype == EI_BF16)
    moe_route_kernel<bf16_t><<<blocks, threads, 0, stream>>>(static_cast<const bf16_t*>(x), w_router,
                                                             row_seq, expert, weight, N, W, E, top);
  else
    EI_REQUIRE(false, "moe_route: unknown dtype");
  EI_LAUNCH_CHECK();
}

extern "C" int ei_moe_experts(const void* x, const void* w_gate, const void* w_up, const void* w_down,
                              int dtype, const int32_t* expert, const float* weight, void* act,
                              float* out, int N, int W, int F, int top, hipStream_t stream) {
  EI_REQUIRE(x && w_gate && w_up && w_down && expert && weight && act && out, "moe_experts: null pointer");
  EI_REQUIRE(N > 0 && W > 0 && F > 0 && top >= 1, "moe_experts: sizes must be positive");
  EI_REQUIRE(static_cast<long long>(N) * top <= 0x7fffffffLL && (F + 15) / 16 <= 65535 &&
                 (W + 15) / 16 <= 65535, "moe_experts: too large for one launch");
  const dim3 grid_up(N * top, (F + 15) / 16), grid_down(N, (W + 15) / 16);
#define EI_MOE(T)                                                                              \
  do {                                                                                         \
    moe_gate_up_kernel<T><<<grid_up, 256, 0, stream>>>(                                        \
        static_cast<const T*>(x), static_cast<const T*>(w_gate), static_cast<const T*>(w_up),  \
        expert, weight, static_cast<T*>(act), W, F, top);                                      \
    moe_down_kernel<T><<<grid_down, 256, 0, stream>>>(                                         \
        static_cast<const T*>(act), static_cast<const T*>(w_down), expert, weight, out, W, F, top); \
  } while (0)
  if (dtype == EI_F32) EI_MOE(float);
  else if (dtype == EI_BF16) EI_MOE(bf16_t);
  else EI_REQUIRE(false, "moe_experts: unknown dtype");
#undef EI_MOE
  EI_LAUNCH_CHECK();
}

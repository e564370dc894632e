// A short causal convolution over time that is added to what it reads: for every channel c of
// a row at step index t of its sequence,
//
//   out_t[c] = h_t[c] + sum_j w[j, c] * h_(t - T + 1 + j)[c],    j = 0 .. T - 1,
//
// (the filter lies tap by tap, [T, W], so that neighbouring channels' weights are neighbours) with rows before the sequence's start being zero.  The last T - 1 inputs of a sequence are
// its state: a float32 table with two versions of every sequence's row, [tables rows]
// [parts][T - 1][W]; a step reads the row `seq_in` names and writes the whole part `part` of
// the row `seq_out` names, so a prompt may arrive whole, in portions of any size or token by
// token.  Inputs older than the step's own rows come from the state.  Arithmetic is float32;
// the result is rounded once to the rows' type.
#include "common.h"

namespace {

// VEC channels a thread (8: 16-byte accesses of bfloat16 rows, for widths that are multiples
// of 8; 1: any width).
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
input_conv_kernel(const T* __restrict__ h, const float* __restrict__ w,
                  const float* state, float* state_out, int part,
                  int parts, int taps, const int32_t* __restrict__ row_pos,
                  const int32_t* __restrict__ row_seq, const int32_t* __restrict__ seq_in,
                  const int32_t* __restrict__ seq_out, const int32_t* __restrict__ seq_start,
                  const int32_t* __restrict__ seq_count, const int32_t* __restrict__ seq_row0,
                  T* __restrict__ out, int N, int W, int n_seqs) {
  const int tail = taps - 1;
  const int WV = W / VEC;                                             // channel groups of a row
  const size_t row_floats = static_cast<size_t>(parts) * tail * W;   // of one state row
  const size_t part_at = static_cast<size_t>(part) * tail * W;
  const size_t index = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t conv_items = static_cast<size_t>(N) * WV;

  auto load_row = [&](const T* p, float (&x)[VEC]) {
    if constexpr (VEC == 8) ei::VecN<T, 8>::load(p, x);
    else x[0] = ei::to_f32<T>(p[0]);
  };
  auto load_state = [&](const float* p, float (&x)[VEC]) {
    if constexpr (VEC == 8) ei::VecN<float, 8>::load(p, x);
    else x[0] = p[0];
  };
  if (index < conv_items) {
    const int row = static_cast<int>(index / WV), c = static_cast<int>(index % WV) * VEC;
    const int seq = row_seq[row];
    if (seq < 0) return;                       // a padding row
    const int t = row_pos[row] - seq_start[seq];
    const int row0 = seq_row0[seq];
    const float* old = state ? state + static_cast<size_t>(seq_in[seq]) * row_floats + part_at : nullptr;
    float acc[VEC];
    load_row(h + static_cast<size_t>(row) * W + c, acc);
    for (int j = 0; j < taps; ++j) {
      const int at = t - tail + j;             // the step's row that tap j meets
      float x[VEC];
      if (at >= 0) load_row(h + static_cast<size_t>(row0 + at) * W + c, x);
      else load_state(old + static_cast<size_t>(tail + at) * W + c, x);
      float wj[VEC];
      load_state(w + static_cast<size_t>(j) * W + c, wj);
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] += wj[i] * x[i];
    }
    if constexpr (VEC == 8) ei::VecN<T, 8>::store(out + static_cast<size_t>(row) * W + c, acc);
    else out[static_cast<size_t>(row) * W + c] = ei::from_f32<T>(acc[0]);
    return;
  }
  // the threads beyond the rows renew the state: entry k of the new tail is the input at step
  // index count - tail + k, which is one of the step's rows or an entry of the old tail
  const size_t item = index - conv_items;
  if (tail == 0 || item >= static_cast<size_t>(n_seqs) * tail * WV) return;
  const int seq = static_cast<int>(item / (static_cast<size_t>(tail) * WV));
  const int k = static_cast<int>(item / WV % tail), c = static_cast<int>(item % WV) * VEC;
  const int count = seq_count[seq];
  if (count <= 0) return;                      // a padding sequence
  const int at = count - tail + k;
  float x[VEC];
  if (at >= 0) load_row(h + static_cast<size_t>(seq_row0[seq] + at) * W + c, x);
  else load_state(state + static_cast<size_t>(seq_in[seq]) * row_floats + part_at +
                  static_cast<size_t>(tail + at) * W + c, x);
  float* dst = state_out + static_cast<size_t>(seq_out[seq]) * row_floats + part_at +
               static_cast<size_t>(k) * W + c;
  if constexpr (VEC == 8) ei::VecN<float, 8>::store(dst, x);
  else dst[0] = x[0];
}

}  // namespace

// h, out: [N, W] of `dtype` (out may not be h: later rows read earlier ones); w: [taps, W]
// float32; state: float32 rows of parts * (taps - 1) * W (null when taps is 1).
extern "C" int ei_input_conv(const void* h, int dtype, const float* w, float* state, int part,
                             int parts, int taps, const int32_t* row_pos, const int32_t* row_seq,
                             const int32_t* seq_in, const int32_t* seq_out,
                             const int32_t* seq_start, const int32_t* seq_count,
                             const int32_t* seq_row0, void* out, int N, int W, int n_seqs,
                             hipStream_t stream) {
  EI_REQUIRE(h && w && out && h != out && N > 0 && W > 0 && n_seqs > 0, "input_conv: bad arguments");
  EI_REQUIRE(taps >= 1 && taps <= 64 && parts >= 1 && part >= 0 && part < parts,
             "input_conv: 1 to 64 taps, and a part of the state that exists");
  EI_REQUIRE(row_pos && row_seq && seq_start && seq_count && seq_row0, "input_conv: row metadata missing");
  EI_REQUIRE(taps == 1 || (state && seq_in && seq_out), "input_conv: state missing");
  const auto aligned16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = W % 8 == 0 && aligned16(h) && aligned16(out) && aligned16(state) && aligned16(w);
  const int per = vec ? 8 : 1;
  const size_t items = (static_cast<size_t>(N) + static_cast<size_t>(n_seqs) * (taps - 1)) * (W / per);
  const unsigned blocks = static_cast<unsigned>((items + 255) / 256);
#define EI_IC(T, VEC)                                                                          \
  input_conv_kernel<T, VEC><<<blocks, 256, 0, stream>>>(                                       \
      static_cast<const T*>(h), w, state, state, part, parts, taps, row_pos, row_seq, seq_in,  \
      seq_out, seq_start, seq_count, seq_row0, static_cast<T*>(out), N, W, n_seqs)
  if (dtype == EI_F32) {
    if (vec) EI_IC(float, 8); else EI_IC(float, 1);
  } else if (dtype == EI_BF16) {
    if (vec) EI_IC(bf16_t, 8); else EI_IC(bf16_t, 1);
  }
  else
    EI_REQUIRE(false, "input_conv: unknown dtype");
#undef EI_IC
  EI_LAUNCH_CHECK();
}

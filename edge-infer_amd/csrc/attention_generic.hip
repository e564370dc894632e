// Causal grouped-query attention over the paged cache, any key head size up to 1024 and value
// head size up to 512 (the two may differ), any head and group counts, float32 or bfloat16
// storage, float32 arithmetic throughout (scores, running maximum, exponentials,
// sums and the value accumulation).  One kernel serves prefill (many positions of a
// sequence) and decode (one position, the key range split over several blocks and
// merged by a second kernel).
//
// Mathematics of the reference: s_t = (q . k_t) / sqrt(d) for keys t <= p (and
// t > p - window when a window is set), streaming softmax with a running maximum,
// o = sum w_t v_t / sum w_t; query head h reads kv head h / (nq / nkv).
// Options beyond the reference: `chunk` (a query at p sees key t only if t / chunk == p / chunk),
// `slopes` (per query head: the score is lowered by slope * (p - t)), `sinks` (per query head:
// exp(sink) joins the denominator; it has no key and no value), `key_heads` (a query row is
// key_heads * D wide and meets the keys of all kv heads of a position laid end to end, which is
// how scores mixed over heads are taken: a mix of scores is the score of mixed queries;
// values still come from the row's own kv head), `values_in_keys` (the values are the first DV
// elements of the key rows: a latent that serves as key and value is cached once), `gate` (per
// row and head: the output is multiplied by sigmoid(gate)), `pool` (with a window w: besides the
// tokens of its window a query at p sees entry b of a second paged cache, which holds one key and
// value for every block of `pool` positions, if b pool + pool - 1 <= p - w; tokens and blocks
// share one softmax), `pool_only` (the tokens are left out: the kernel takes the pooled entries
// alone and leaves every row's unnormalised sums, maximum and sum of weights in part_o and
// part_ml, slice 0 of one, for a kernel that takes them in as one more slice of its own softmax).
// operators/src/cuda/execution.cu:137-179, runtime/src/qwen.cpp:374-402,
// split merge: operators/src/cuda/kernels/gather_fa_variable.cu:14-118.
#include "common.h"

namespace {

constexpr int kRows = 16;     // query rows (positions x heads of one kv group) per block
constexpr int kThreads = 256;
constexpr float kLowest = -1.0e30f;
constexpr int kAcc = 32;      // a lane holds every 16th value element: values up to 16 * kAcc wide

// Work item: `npos` consecutive packed rows starting at `row0`, all of sequence `seq`.
template <typename T>
__global__ void __launch_bounds__(kThreads)
attn_generic_kernel(const T* __restrict__ q, const T* __restrict__ k_pages,
                    const T* __restrict__ v_pages, const int32_t* __restrict__ item_seq,
                    const int32_t* __restrict__ item_row0, const int32_t* __restrict__ item_npos,
                    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ page_table,
                    int table_width, T* __restrict__ out, float* __restrict__ part_o,
                    float* __restrict__ part_ml, int nq, int nkv, int D, int DV, int Gb,
                    int head_blocks, int BC, int window, int chunk,
                    const float* __restrict__ slopes, const float* __restrict__ sinks,
                    float scale, int n_splits, int KH, int values_in_keys,
                    const float* __restrict__ gate, int pool, const T* __restrict__ pool_k,
                    const T* __restrict__ pool_v, const int32_t* __restrict__ pool_table,
                    int pool_only) {
  extern __shared__ float lds[];
  const int DQ = KH * D;                  // width of a query row and of a key as it is met
  float* Qs = lds;                        // [kRows][DQ]
  float* Ks = Qs + kRows * DQ;            // [BC][DQ + 1]
  float* Vs = Ks + BC * (DQ + 1);         // [BC][DV]
  float* Ps = Vs + BC * DV;               // [kRows][BC + 1]

  const int item = blockIdx.x;
  const int g = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
  const int split = blockIdx.z;
  const int seq = item_seq[item];
  const int npos = item_npos[item];
  const int row0 = item_row0[item];
  const int G = nq / nkv;
  const int t = threadIdx.x;
  const int r = t / 16, cc = t % 16;
  const int pi = r / Gb, hi = r % Gb;
  const int head_in_group = hb * Gb + hi;
  const bool row_valid = seq >= 0 && pi < npos && head_in_group < G;
  const int head = g * G + head_in_group;
  const int row = row0 + pi;
  const int pos_r = row_valid ? row_pos[row] : -1;
  const float slope = (slopes && row_valid) ? slopes[head] : 0.f;
  const int chunk_r = (chunk > 0 && row_valid) ? pos_r / chunk : 0;

  // (the pooled entries alone, and the item's last row sees none: nothing to meet)
  bool idle = false;
  if (pool_only && seq >= 0 && npos > 0) {
    const int before = row_pos[row0 + npos - 1] - window + 1;
    idle = before < pool;
  }
  // query rows, pre-scaled
  for (int idx = t; idx < kRows * DQ && !idle; idx += kThreads) {
    const int rr = idx / DQ, d = idx % DQ;
    const int ppi = rr / Gb, hhi = hb * Gb + rr % Gb;
    float v = 0.f;
    if (seq >= 0 && ppi < npos && hhi < G)
      v = ei::to_f32<T>(q[(static_cast<size_t>(row0 + ppi) * nq + g * G + hhi) * DQ + d]) * scale;
    Qs[idx] = v;
  }

  float m_r = kLowest, l_r = 0.f;
  float acc[kAcc];
#pragma unroll
  for (int k = 0; k < kAcc; ++k) acc[k] = 0.f;
  const int nd = (DV + 15) / 16;
  const int nj = BC / 16;

  // pooled blocks that this row sees: those wholly before its window
  const int blocks_r = (pool > 0 && window > 0 && row_valid && pos_r - window + 1 > 0)
                           ? (pos_r - window + 1) / pool : 0;
  // One chunk of BC keys (chunk `ch` of a page whose first key is key0; keys beyond last_key
  // hold stale bytes) against the block's rows: scores, running maximum and sum, values.
  auto walk = [&](const T* kp, const T* vp, int DVS, int phys, int ch, int key0, int last_key,
                  bool pooled) {
      __syncthreads();
      for (int idx = t; idx < BC * DQ; idx += kThreads) {
        const int c = idx / DQ, d = idx % DQ;
        const bool live = key0 + c <= last_key;  // later slots hold stale bytes
        // with key_heads > 1 the piece d / D of the key lies in that kv head's page part
        const T* src = KH > 1 ? k_pages + (static_cast<size_t>(phys) * nkv + d / D) * EI_PAGE * D
                              : kp;
        const size_t off = static_cast<size_t>(ch * BC + c) * D + (KH > 1 ? d % D : d);
        Ks[c * (DQ + 1) + d] = live ? ei::to_f32<T>(src[off]) : 0.f;
      }
      for (int idx = t; idx < BC * DV; idx += kThreads) {
        const int c = idx / DV, d = idx % DV;
        const bool live = key0 + c <= last_key;
        const size_t off = static_cast<size_t>(ch * BC + c) * DVS + d;
        Vs[c * DV + d] = live ? ei::to_f32<T>(vp[off]) : 0.f;
      }
      __syncthreads();
      float s[4];
      float row_max = kLowest;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s[j] = -INFINITY;
        if (j < nj) {
          const int c = cc + 16 * j;
          const int key = key0 + c;
          const bool visible =
              pooled ? (row_valid && key < blocks_r)
                     : (row_valid && key <= pos_r && (window <= 0 || key > pos_r - window) &&
                        (chunk <= 0 || key / chunk == chunk_r));
          if (visible) {
            float dot = 0.f;
            const float* qr = Qs + r * DQ;
            const float* kr = Ks + c * (DQ + 1);
            for (int d = 0; d < DQ; ++d) dot += qr[d] * kr[d];
            if (!pooled) dot -= slope * static_cast<float>(pos_r - key);
            s[j] = dot;
            row_max = fmaxf(row_max, dot);
          }
        }
      }
#pragma unroll
      for (int offset = 8; offset > 0; offset >>= 1)
        row_max = fmaxf(row_max, __shfl_xor(row_max, offset, 16));
      const float m_new = fmaxf(m_r, row_max);
      const float alpha = expf(m_r - m_new);
      float row_sum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j < nj) {
          const float p_val = expf(s[j] - m_new);  // -inf -> 0
          Ps[r * (BC + 1) + cc + 16 * j] = p_val;
          row_sum += p_val;
        }
      }
#pragma unroll
      for (int offset = 8; offset > 0; offset >>= 1) row_sum += __shfl_xor(row_sum, offset, 16);
      l_r = l_r * alpha + row_sum;
      m_r = m_new;
      __syncthreads();
      const float* pr = Ps + r * (BC + 1);
#pragma unroll
      for (int k = 0; k < kAcc; ++k) {
        if (k < nd) {
          const int d = cc + 16 * k;
          float a = acc[k] * alpha;
          if (d < DV)
            for (int c = 0; c < BC; ++c) a += pr[c] * Vs[c * DV + d];
          acc[k] = a;
        }
      }
  };

  if (seq >= 0 && npos > 0 && !idle) {
    const int hi_key = row_pos[row0 + npos - 1];
    int lo_key = window > 0 ? max(0, row_pos[row0] - window + 1) : 0;
    if (chunk > 0) lo_key = max(lo_key, row_pos[row0] / chunk * chunk);
    const int lo_page = lo_key / EI_PAGE, hi_page = hi_key / EI_PAGE;
    const int total_pages = hi_page - lo_page + 1;
    const int per = (total_pages + n_splits - 1) / n_splits;
    const int p_begin = lo_page + split * per;
    const int p_end = min(lo_page + (split + 1) * per, hi_page + 1);
    const int chunks_per_page = EI_PAGE / BC;
    for (int p = p_begin; p < p_end && !pool_only; ++p) {
      const int phys = page_table[static_cast<size_t>(seq) * table_width + p];
      if (phys < 0) continue;  // a page the window has released: every key in it is masked
      const T* kp = k_pages + (static_cast<size_t>(phys) * nkv + g) * EI_PAGE * D;
      const int DVS = values_in_keys ? D : DV;      // distance between two keys' values
      const T* vp = values_in_keys
                        ? kp
                        : v_pages + (static_cast<size_t>(phys) * nkv + g) * EI_PAGE * DV;
      for (int ch = 0; ch < chunks_per_page; ++ch) {
        const int key0 = p * EI_PAGE + ch * BC;
        if (key0 > hi_key) break;
        if (key0 + BC <= lo_key) continue;   // wholly before what any row of the item sees
        walk(kp, vp, DVS, phys, ch, key0, hi_key, false);
      }
    }
    if (pool > 0 && window > 0) {
      // the pooled blocks that the item's last row sees (its other rows see fewer): entries
      // 0 .. seen - 1 of the pooled cache, whose pages the slices take in turn
      const int before = hi_key - window + 1;
      const int seen = before > 0 ? before / pool : 0;
      const int pool_pages = (seen + EI_PAGE - 1) / EI_PAGE;
      for (int p = split; p < pool_pages; p += n_splits) {
        const int phys = pool_table[static_cast<size_t>(seq) * table_width + p];
        if (phys < 0) continue;
        const T* kp = pool_k + (static_cast<size_t>(phys) * nkv + g) * EI_PAGE * D;
        const T* vp = pool_v + (static_cast<size_t>(phys) * nkv + g) * EI_PAGE * DV;
        for (int ch = 0; ch < chunks_per_page; ++ch) {
          const int key0 = p * EI_PAGE + ch * BC;
          if (key0 >= seen) break;
          walk(kp, vp, DV, phys, ch, key0, seen - 1, true);
        }
      }
    }
  }

  if (!row_valid) return;
  if (sinks && split == 0 && !pool_only) {
    // the sink is one more term of the denominator: exp(sink), on the row's running scale
    const float sink = sinks[head];
    const float m_new = fmaxf(m_r, sink);
    const float alpha = expf(m_r - m_new);
    l_r = l_r * alpha + expf(sink - m_new);
#pragma unroll
    for (int k = 0; k < kAcc; ++k) acc[k] *= alpha;
    m_r = m_new;
  }
  if (n_splits == 1 && !pool_only) {
    float inv = l_r > 0.f ? 1.f / l_r : 0.f;
    if (gate) inv *= 1.0f / (1.0f + expf(-gate[static_cast<size_t>(row) * nq + head]));
    T* dst = out + (static_cast<size_t>(row) * nq + head) * DV;
#pragma unroll
    for (int k = 0; k < kAcc; ++k)
      if (k < nd && cc + 16 * k < DV) dst[cc + 16 * k] = ei::from_f32<T>(acc[k] * inv);
  } else {
    const size_t slot = (static_cast<size_t>(row) * nq + head) * n_splits + split;
    float* dst = part_o + slot * DV;
#pragma unroll
    for (int k = 0; k < kAcc; ++k)
      if (k < nd && cc + 16 * k < DV) dst[cc + 16 * k] = acc[k];
    if (cc == 0) {
      part_ml[slot * 2] = m_r;
      part_ml[slot * 2 + 1] = l_r;
    }
  }
}

// One wave per (row, head): o = sum_s o_s e^{m_s - m} / sum_s l_s e^{m_s - m}.
template <typename T>
__global__ void attn_merge_kernel(const float* __restrict__ part_o,
                                  const float* __restrict__ part_ml,
                                  const int32_t* __restrict__ row_seq, T* __restrict__ out, int nq,
                                  int D, int n_splits, int total,
                                  const float* __restrict__ gate) {
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= total) return;
  const int row = wave / nq;
  if (row_seq && row_seq[row] < 0) return;
  const float* ml = part_ml + static_cast<size_t>(wave) * n_splits * 2;
  float m = kLowest;
  for (int s = 0; s < n_splits; ++s) m = fmaxf(m, ml[2 * s]);
  float l = 0.f;
  for (int s = 0; s < n_splits; ++s) l += ml[2 * s + 1] * expf(ml[2 * s] - m);
  float inv = l > 0.f ? 1.f / l : 0.f;
  if (gate) inv *= 1.0f / (1.0f + expf(-gate[wave]));
  const float* po = part_o + static_cast<size_t>(wave) * n_splits * D;
  for (int d = lane; d < D; d += EI_WAVE) {
    float o = 0.f;
    for (int s = 0; s < n_splits; ++s) o += po[static_cast<size_t>(s) * D + d] * expf(ml[2 * s] - m);
    out[static_cast<size_t>(wave) * D + d] = ei::from_f32<T>(o * inv);
  }
}

int chunk_keys(int D) { return D <= 64 ? 64 : (D <= 128 ? 32 : 16); }

}  // namespace

// Heads of one kv group that share a block (at most 16) for a head count ratio G.
extern "C" int ei_attn_heads_per_block(int G) { return G < kRows ? G : kRows; }
// Positions of one sequence that a prefill work item holds.
extern "C" int ei_attn_positions_per_item(int G) {
  const int gb = G < kRows ? G : kRows;
  return kRows / gb;
}

// q: [N, nq, D], out: [N, nq, DV]; key pages: [n_pages, nkv, 64, D], value pages:
// [n_pages, nkv, 64, DV]; items: see the kernel.  chunk 0, slopes and sinks null: none.
// n_splits > 1 needs part_o [N, nq, n_splits, DV] and part_ml [N, nq, n_splits, 2]
// float32 and items that hold one position each (decode); the merge follows.
extern "C" int ei_attention(const void* q, const void* k_pages, const void* v_pages, int dtype,
                            const int32_t* item_seq, const int32_t* item_row0,
                            const int32_t* item_npos, int n_items, const int32_t* row_pos,
                            const int32_t* row_seq, const int32_t* page_table, int table_width,
                            void* out, float* part_o, float* part_ml, int N, int nq, int nkv,
                            int D, int DV, int window, int chunk, const float* slopes,
                            const float* sinks, float scale, int n_splits, int key_heads,
                            int values_in_keys, const float* gate, int pool, const void* pool_k,
                            const void* pool_v, const int32_t* pool_table, int pool_only,
                            hipStream_t stream) {
  EI_REQUIRE(n_items > 0 && N > 0 && nq > 0 && nkv > 0, "attention: sizes must be positive");
  EI_REQUIRE(nq % nkv == 0, "attention: query heads must be a multiple of kv heads");
  EI_REQUIRE(key_heads == 1 || key_heads == nkv,
             "attention: a query meets the keys of its own kv head or of all of them");
  const int DQ = key_heads * D;
  EI_REQUIRE(D >= 1 && DQ <= 1024 && DV >= 1 && DV <= 16 * kAcc,
             "attention: keys of at most 1024 and values of at most 512 elements a head");
  EI_REQUIRE(!values_in_keys || DV <= D, "attention: values inside keys cannot be wider than them");
  EI_REQUIRE(values_in_keys || v_pages, "attention: null pointer");
  EI_REQUIRE(chunk >= 0, "attention: negative chunk");
  EI_REQUIRE(q && k_pages && out && item_seq && item_row0 && item_npos && row_pos &&
                 page_table && table_width > 0,
             "attention: null pointer");
  EI_REQUIRE(n_splits >= 1 && n_splits <= 64, "attention: splits must be between 1 and 64");
  EI_REQUIRE((n_splits == 1 && !pool_only) || (part_o && part_ml), "attention: split scratch missing");
  EI_REQUIRE(!pool_only || (pool > 0 && n_splits == 1 && !gate),
             "attention: the pooled entries alone are taken in one slice, without a gate");
  EI_REQUIRE(window >= 0, "attention: negative window");
  EI_REQUIRE(pool >= 0 && (pool == 0 || (window > 0 && pool_k && pool_v && pool_table &&
                                         key_heads == 1 && !values_in_keys)),
             "attention: pooled blocks need a window, their cache and keys of one kv head");
  const int G = nq / nkv;
  const int Gb = G < kRows ? G : kRows;
  const int head_blocks = (G + Gb - 1) / Gb;
  const int BC = chunk_keys(DQ > DV ? DQ : DV);
  const size_t lds =
      sizeof(float) * (static_cast<size_t>(kRows) * DQ + static_cast<size_t>(BC) * (DQ + 1) +
                       static_cast<size_t>(BC) * DV + static_cast<size_t>(kRows) * (BC + 1));
  if (lds > 64 * 1024) {      // beyond the default bound of a launch: ask for it, once
    static bool raised = false;
    if (!raised) {
      const int most = 160 * 1024;
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_generic_kernel<float>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess ||
          hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_generic_kernel<bf16_t>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess) {
        (void)hipGetLastError();
        EI_REQUIRE(false, "attention: the device refuses the LDS these head sizes need");
      }
      raised = true;
    }
  }
  EI_REQUIRE(lds <= 160 * 1024, "attention: head sizes too large for the LDS");
  EI_REQUIRE(static_cast<long long>(nkv) * head_blocks <= 65535, "attention: too many heads");
  dim3 grid(n_items, nkv * head_blocks, n_splits);
  if (dtype == EI_F32) {
    attn_generic_kernel<float><<<grid, kThreads, lds, stream>>>(
        static_cast<const float*>(q), static_cast<const float*>(k_pages),
        static_cast<const float*>(v_pages), item_seq, item_row0, item_npos, row_pos, page_table,
        table_width, static_cast<float*>(out), part_o, part_ml, nq, nkv, D, DV, Gb, head_blocks,
        BC, window, chunk, slopes, sinks, scale, n_splits, key_heads, values_in_keys, gate, pool,
        static_cast<const float*>(pool_k), static_cast<const float*>(pool_v), pool_table, pool_only);
  } else if (dtype == EI_BF16) {
    attn_generic_kernel<bf16_t><<<grid, kThreads, lds, stream>>>(
        static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages),
        static_cast<const bf16_t*>(v_pages), item_seq, item_row0, item_npos, row_pos, page_table,
        table_width, static_cast<bf16_t*>(out), part_o, part_ml, nq, nkv, D, DV, Gb, head_blocks,
        BC, window, chunk, slopes, sinks, scale, n_splits, key_heads, values_in_keys, gate, pool,
        static_cast<const bf16_t*>(pool_k), static_cast<const bf16_t*>(pool_v), pool_table, pool_only);
  } else {
    EI_REQUIRE(false, "attention: unknown dtype");
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    ei_set_error(hipGetErrorString(e));
    return static_cast<int>(e);
  }
  if (n_splits > 1) {
    const int total = N * nq;
    const int threads = 256;
    const int blocks = (total * EI_WAVE + threads - 1) / threads;
    if (dtype == EI_F32)
      attn_merge_kernel<float><<<blocks, threads, 0, stream>>>(
          part_o, part_ml, row_seq, static_cast<float*>(out), nq, DV, n_splits, total, gate);
    else
      attn_merge_kernel<bf16_t><<<blocks, threads, 0, stream>>>(
          part_o, part_ml, row_seq, static_cast<bf16_t*>(out), nq, DV, n_splits, total, gate);
  }
  EI_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// The pooled cache: entry b holds the means of the cached keys and of the cached values of the
// positions b P .. b P + P - 1 of a sequence, for every kv head.  A wave a (row, kv head): the
// row at position p with (p + 1) % P == 0 completes block p / P, whose keys all lie in the
// token cache by then (this step's store has run), and writes the block's entry; every other
// row has nothing to do.  Sums are float32, in the order of the positions, divided by P.
namespace {

template <typename T>
__global__ void pool_store_kernel(const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                                  const int32_t* __restrict__ row_pos,
                                  const int32_t* __restrict__ row_seq,
                                  const int32_t* __restrict__ page_table,
                                  const int32_t* __restrict__ pool_table, int table_width,
                                  T* __restrict__ pool_k, T* __restrict__ pool_v, int N, int nkv,
                                  int D, int DV, int P, int pieces,
                                  const int32_t* __restrict__ row_list) {
  // a wave a (row, kv head, piece of 64 elements of [key | value]); eight positions' loads
  // are issued before the first is added
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= N * nkv * pieces) return;
  const int piece = wave % pieces, g = wave / pieces % nkv;
  // (row_list: the rows that end a block, as the host has worked them out; -1: none)
  const int row = row_list ? row_list[wave / pieces / nkv] : wave / pieces / nkv;
  if (row < 0) return;
  const int seq = row_seq[row];
  if (seq < 0) return;
  const int pos = row_pos[row];
  if ((pos + 1) % P != 0) return;
  const int e = piece * EI_WAVE + lane;
  if (e >= D + DV) return;
  const int block = pos / P;
  const int32_t* pages = page_table + static_cast<size_t>(seq) * table_width;
  const int dst_page = pool_table[static_cast<size_t>(seq) * table_width + block / EI_PAGE];
  if (dst_page < 0) return;
  const size_t dst = (static_cast<size_t>(dst_page) * nkv + g) * EI_PAGE + block % EI_PAGE;
  const bool key = e < D;
  const int width = key ? D : DV, at = key ? e : e - D;
  const T* source = key ? k_pages : v_pages;
  float sum = 0.f;
  for (int j0 = 0; j0 < P; j0 += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      v[u] = 0.f;
      const int p = block * P + j0 + u;
      if (j0 + u < P) {
        const int phys = pages[p / EI_PAGE];
        if (phys >= 0)
          v[u] = ei::to_f32<T>(source[((static_cast<size_t>(phys) * nkv + g) * EI_PAGE + p % EI_PAGE) *
                                      width + at]);
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) sum += v[u];
  }
  (key ? pool_k : pool_v)[dst * width + at] = ei::from_f32<T>(sum / static_cast<float>(P));
}

}  // namespace

// k_pages [pages, nkv, 64, D], v_pages [pages, nkv, 64, DV] hold the tokens; pool_k, pool_v the
// same shapes for the pooled entries, found through pool_table as tokens are through page_table.
// row_list (or null): n_listed rows to look at instead of all N (a prompt step's rows that end a
// block, known to the host; entries of -1 are skipped).
extern "C" int ei_pool_store(const void* k_pages, const void* v_pages, int dtype,
                             const int32_t* row_pos, const int32_t* row_seq,
                             const int32_t* page_table, const int32_t* pool_table, int table_width,
                             void* pool_k, void* pool_v, int N, int nkv, int D, int DV, int P,
                             const int32_t* row_list, int n_listed, hipStream_t stream) {
  EI_REQUIRE(k_pages && v_pages && row_pos && row_seq && page_table && pool_table && pool_k && pool_v,
             "pool_store: null pointer");
  EI_REQUIRE(N > 0 && nkv > 0 && D > 0 && DV > 0 && P >= 1 && table_width > 0,
             "pool_store: sizes must be positive");
  const int pieces = (D + DV + EI_WAVE - 1) / EI_WAVE;
  EI_REQUIRE(!row_list || n_listed > 0, "pool_store: an empty list of rows");
  // N rows, or only the listed ones among them
  const size_t waves = static_cast<size_t>(row_list ? n_listed : N) * nkv * pieces;
  if (row_list) N = n_listed;
  EI_REQUIRE(waves * EI_WAVE / 256 < 0x7fffffffULL, "pool_store: too many rows for one launch");
  const unsigned blocks = static_cast<unsigned>((waves * EI_WAVE + 255) / 256);
  if (dtype == EI_F32)
    pool_store_kernel<float><<<blocks, 256, 0, stream>>>(
        static_cast<const float*>(k_pages), static_cast<const float*>(v_pages), row_pos, row_seq,
        page_table, pool_table, table_width, static_cast<float*>(pool_k),
        static_cast<float*>(pool_v), N, nkv, D, DV, P, pieces, row_list);
  else if (dtype == EI_BF16)
    pool_store_kernel<bf16_t><<<blocks, 256, 0, stream>>>(
        static_cast<const bf16_t*>(k_pages), static_cast<const bf16_t*>(v_pages), row_pos, row_seq,
        page_table, pool_table, table_width, static_cast<bf16_t*>(pool_k),
        static_cast<bf16_t*>(pool_v), N, nkv, D, DV, P, pieces, row_list);
  else
    EI_REQUIRE(false, "pool_store: unknown dtype");
  EI_LAUNCH_CHECK();
}

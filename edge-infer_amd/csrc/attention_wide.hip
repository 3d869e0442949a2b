// bfloat16 attention over the paged cache on the matrix cores for wide keys: key rows of up to
// 1024 elements (a latent with its rotated part, or the keys of all kv heads of a position laid
// end to end for scores mixed over heads) and values of up to 512, which may be the first
// elements of the key rows.  One kernel serves prompts (several positions of a sequence a
// block) and decoding (one position, the key range cut into slices that a second kernel
// merges).  Mathematics and options as in attention_generic.hip: causal, optional window,
// a sink per head in the softmax's denominator, a sigmoid gate per row and head on the output;
// float32 scores, maxima, sums and accumulators, the softmax's weights rounded to bfloat16
// only as the operand of the value product.
//
// A block is four waves and up to 64 query rows (positions x heads of one kv group, 16 a
// wave).  Keys come in tiles of 32 through LDS, as stored (a row a key, padded by 16 bytes),
// the values of the tile transposed (a row a value element, 32 keys wide).  Scores are taken
// transposed, S^T = K Q^T with v_mfma_f32_16x16x32_bf16: the key tile is the A operand (lane
// (key, c) reads 16 bytes of the key's row), the wave's query rows, held in registers for the
// whole walk, the B operand; lane (c, n) then holds the scores of keys 4c .. 4c + 3 of either
// half of the tile for query row n, which is, with the keys of a tile taken in the order
// {4c .. 4c + 3, 16 + 4c .. 16 + 4c + 3}, exactly the B operand of O^T = V^T P^T; the A operand
// of that product is two 8-byte reads of a row of the transposed values.  A lane's
// accumulators all belong to query row n, so the rescaling needs no exchange.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kThreads = 256;
constexpr int kRows = 64;         // query rows of a block
constexpr int kKeys = 32;         // keys of a tile
constexpr int kPadK = 8;          // elements of padding of a key row in LDS
constexpr int kVtRow = kKeys + 8; // elements of a row of the transposed values in LDS
constexpr float kLowest = -1.0e30f;

template <int NK, int NDV>
__global__ void __launch_bounds__(kThreads)
attn_wide_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
                 const bf16_t* __restrict__ v_pages, const int32_t* __restrict__ item_seq,
                 const int32_t* __restrict__ item_row0, const int32_t* __restrict__ item_npos,
                 const int32_t* __restrict__ row_pos, const int32_t* __restrict__ page_table,
                 int table_width, bf16_t* __restrict__ out, float* __restrict__ part_o,
                 float* __restrict__ part_ml, int nq, int nkv, int D, int DV, int KH,
                 int values_in_keys, int HB, int head_blocks, int window,
                 const float* __restrict__ sinks, const float* __restrict__ gate, float scale,
                 int n_splits) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int DQ = KH * D;
  const int k_row = DQ + kPadK;                               // elements
  bf16_t* Kt = reinterpret_cast<bf16_t*>(lds_raw);            // [kKeys][k_row]
  bf16_t* Vt = Kt + kKeys * k_row;                            // [DV][kVtRow]
  const int nk = DQ / 32, ndv = DV / 16;

  const int item = blockIdx.x;
  const int g = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
  const int split = blockIdx.z;
  const int seq = item_seq[item];
  const int npos = item_npos[item];
  if (seq < 0 || npos <= 0) return;
  const int row0 = item_row0[item];
  const int G = nq / nkv;
  const int t = threadIdx.x;
  const int wave = t / EI_WAVE, lane = t % EI_WAVE;
  const int n = lane % 16, c = lane / 16;
  const int rho = wave * 16 + n;                              // the block's query row
  const int pi = rho / HB, head_in_group = hb * HB + rho % HB;
  const bool valid = pi < npos && head_in_group < G;
  const int head = g * G + head_in_group;
  const int row = row0 + (valid ? pi : 0);
  const int pos = valid ? row_pos[row] : -1;
  const bool wave_live = __ballot(valid) != 0ull;

  // the wave's query rows as the B operand: lane (n, c) holds q[row n][j * 32 + c * 8 .. + 8]
  bf16x8 q_reg[NK];
#pragma unroll
  for (int j = 0; j < NK; ++j) {
    uint4 z = uint4{0u, 0u, 0u, 0u};
    if (valid && j < nk)
      z = *reinterpret_cast<const uint4*>(q + (static_cast<size_t>(row) * nq + head) * DQ + j * 32 +
                                          c * 8);
    q_reg[j] = *reinterpret_cast<bf16x8*>(&z);
  }

  float m_run = kLowest, l_run = 0.f;
  f32x4 acc[NDV];
#pragma unroll
  for (int d = 0; d < NDV; ++d) acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int hi_key = row_pos[row0 + npos - 1];
  const int lo_key = window > 0 ? max(0, row_pos[row0] - window + 1) : 0;
  const int lo_page = lo_key / EI_PAGE, hi_page = hi_key / EI_PAGE;
  const int per = (hi_page - lo_page + 1 + n_splits - 1) / n_splits;
  const int p_begin = lo_page + split * per;
  const int p_end = min(lo_page + (split + 1) * per, hi_page + 1);
  const int k_chunks = DQ / 8, v_chunks = DV / 8;

  for (int p = p_begin; p < p_end; ++p) {
    const int phys = page_table[static_cast<size_t>(seq) * table_width + p];
    if (phys < 0) continue;          // a page the window has released: every key in it is masked
    for (int half = 0; half < EI_PAGE / kKeys; ++half) {
      const int key0 = p * EI_PAGE + half * kKeys;
      if (key0 > hi_key) break;
      if (key0 + kKeys <= lo_key) continue;
      __syncthreads();
      // keys as stored; with values inside the keys, their first DV elements transposed as well.
      // Neighbouring lanes take neighbouring keys: their 2-byte writes of the transposed values
      // then fall into 32 banks, two lanes a word, instead of into two banks.  The loads of a
      // batch are unconditional, from clamped places (a live key of the tile, the last chunk),
      // so that they travel together instead of each waiting behind a branch.
      // (the widest query rows leave no registers for it: two waves a SIMD count for more there)
      constexpr int kBatch = NK > 18 ? 1 : 5;
      const int last_live = min(kKeys - 1, hi_key - key0);
      const int k_total = kKeys * k_chunks;
      for (int base = 0; base < k_total; base += kThreads * kBatch) {
        uint4 val[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int ch = min(base + u * kThreads + t, k_total - 1);
          const int key = min(ch % kKeys, last_live), col = (ch / kKeys) * 8;
          const int kh = KH > 1 ? col / D : g, dd = KH > 1 ? col % D : col;
          val[u] = *reinterpret_cast<const uint4*>(
              k_pages + ((static_cast<size_t>(phys) * nkv + kh) * EI_PAGE + half * kKeys + key) * D + dd);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int ch = base + u * kThreads + t;
          if (ch < k_total) {
            const int key = ch % kKeys, col = (ch / kKeys) * 8;
            const uint4 v = key <= last_live ? val[u] : uint4{0u, 0u, 0u, 0u};   // stale slots: zeros
            *reinterpret_cast<uint4*>(Kt + key * k_row + col) = v;
            if (values_in_keys && col < DV) {
              const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                Vt[(col + 2 * i) * kVtRow + key] = static_cast<bf16_t>(w[i] & 0xffffu);
                Vt[(col + 2 * i + 1) * kVtRow + key] = static_cast<bf16_t>(w[i] >> 16);
              }
            }
          }
        }
      }
      if (!values_in_keys) {
        const int v_total = kKeys * v_chunks;
        for (int base = 0; base < v_total; base += kThreads * kBatch) {
          uint4 val[kBatch];
#pragma unroll
          for (int u = 0; u < kBatch; ++u) {
            const int ch = min(base + u * kThreads + t, v_total - 1);
            const int key = min(ch % kKeys, last_live), col = (ch / kKeys) * 8;
            val[u] = *reinterpret_cast<const uint4*>(
                v_pages + ((static_cast<size_t>(phys) * nkv + g) * EI_PAGE + half * kKeys + key) * DV + col);
          }
#pragma unroll
          for (int u = 0; u < kBatch; ++u) {
            const int ch = base + u * kThreads + t;
            if (ch < v_total) {
              const int key = ch % kKeys, col = (ch / kKeys) * 8;
              const uint4 v = key <= last_live ? val[u] : uint4{0u, 0u, 0u, 0u};
              const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                Vt[(col + 2 * i) * kVtRow + key] = static_cast<bf16_t>(w[i] & 0xffffu);
                Vt[(col + 2 * i + 1) * kVtRow + key] = static_cast<bf16_t>(w[i] >> 16);
              }
            }
          }
        }
      }
      __syncthreads();
      if (!wave_live) continue;

      f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < NK; ++j) {
        if (j < nk) {
          const bf16x8 a0 = *reinterpret_cast<const bf16x8*>(Kt + n * k_row + j * 32 + c * 8);
          const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(Kt + (16 + n) * k_row + j * 32 + c * 8);
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, q_reg[j], s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, q_reg[j], s1, 0, 0, 0);
        }
      }
      // lane (c, n): s0[r] is the score of key key0 + 4c + r, s1[r] of key0 + 16 + 4c + r, for row n
      float sc[8];
      float tile_max = kLowest;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const int key = key0 + (r < 4 ? 4 * c + r : 16 + 4 * c + (r - 4));
        const bool visible = valid && key <= pos && (window <= 0 || key > pos - window);
        const float s = r < 4 ? s0[r] : s1[r - 4];
        sc[r] = visible ? s * scale : -INFINITY;
        tile_max = fmaxf(tile_max, sc[r]);
      }
      tile_max = ei::rows_max(tile_max);
      const float m_new = fmaxf(m_run, tile_max);
      const float alpha = expf(m_run - m_new);
      float tile_sum = 0.f;
      bf16x8 p_reg;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const float pv = expf(sc[r] - m_new);      // -inf -> 0
        tile_sum += pv;
        p_reg[r] = static_cast<__bf16>(pv);
      }
      tile_sum = ei::rows_sum(tile_sum);
      l_run = l_run * alpha + tile_sum;
      m_run = m_new;
#pragma unroll
      for (int d = 0; d < NDV; ++d) {
        if (d < ndv) {
          const bf16_t* vr = Vt + (d * 16 + n) * kVtRow + 4 * c;
          const uint2 lo = *reinterpret_cast<const uint2*>(vr);
          const uint2 hi = *reinterpret_cast<const uint2*>(vr + 16);
          const uint4 both = uint4{lo.x, lo.y, hi.x, hi.y};
          f32x4 a = acc[d];
          a[0] *= alpha; a[1] *= alpha; a[2] *= alpha; a[3] *= alpha;
          acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, both), p_reg,
                                                          a, 0, 0, 0);
        }
      }
    }
  }

  if (!valid) return;
  if (sinks && split == 0) {
    const float sink = sinks[head];
    const float m_new = fmaxf(m_run, sink);
    const float alpha = expf(m_run - m_new);
    l_run = l_run * alpha + expf(sink - m_new);
#pragma unroll
    for (int d = 0; d < NDV; ++d) {
      acc[d][0] *= alpha; acc[d][1] *= alpha; acc[d][2] *= alpha; acc[d][3] *= alpha;
    }
    m_run = m_new;
  }
  // lane (c, n) holds out[row n][d * 16 + 4c .. + 4]
  if (n_splits == 1) {
    float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    if (gate) inv *= 1.0f / (1.0f + expf(-gate[static_cast<size_t>(row) * nq + head]));
    bf16_t* dst = out + (static_cast<size_t>(row) * nq + head) * DV + 4 * c;
#pragma unroll
    for (int d = 0; d < NDV; ++d) {
      if (d < ndv) {
        const float y[4] = {acc[d][0] * inv, acc[d][1] * inv, acc[d][2] * inv, acc[d][3] * inv};
        ei::Vec4<bf16_t>::store(dst + d * 16, y);
      }
    }
  } else {
    const size_t slot = (static_cast<size_t>(row) * nq + head) * n_splits + split;
    float* dst = part_o + slot * DV + 4 * c;
#pragma unroll
    for (int d = 0; d < NDV; ++d) {
      if (d < ndv) {
        const float y[4] = {acc[d][0], acc[d][1], acc[d][2], acc[d][3]};
        ei::Vec4<float>::store(dst + d * 16, y);
      }
    }
    if (c == 0) {
      part_ml[slot * 2] = m_run;
      part_ml[slot * 2 + 1] = l_run;
    }
  }
}

// One wave per (row, head): o = sum_s o_s e^{m_s - m} / sum_s l_s e^{m_s - m}, times the gate.
// Lane s works out slice s's weight once (at most 64 slices); the lanes then share them.
__global__ void wide_merge_kernel(const float* __restrict__ part_o,
                                  const float* __restrict__ part_ml,
                                  const int32_t* __restrict__ row_seq, bf16_t* __restrict__ out,
                                  int nq, int DV, int n_splits, int total,
                                  const float* __restrict__ gate) {
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= total) return;
  const int row = wave / nq;
  if (row_seq && row_seq[row] < 0) return;
  const float* ml = part_ml + static_cast<size_t>(wave) * n_splits * 2;
  const float m_own = lane < n_splits ? ml[2 * lane] : kLowest;
  const float l_own = lane < n_splits ? ml[2 * lane + 1] : 0.f;
  const float m = ei::wave_max(m_own);
  float weight = lane < n_splits ? expf(m_own - m) : 0.f;
  const float l = ei::wave_sum(l_own * weight);
  float inv = l > 0.f ? 1.f / l : 0.f;
  if (gate) inv *= 1.0f / (1.0f + expf(-gate[wave]));
  weight *= inv;
  const float* po = part_o + static_cast<size_t>(wave) * n_splits * DV;
  for (int d = lane * 4; d < DV; d += EI_WAVE * 4) {       // DV is a multiple of 16
    float o[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < n_splits; ++s) {
      float x[4];
      ei::Vec4<float>::load(po + static_cast<size_t>(s) * DV + d, x);
      const float w = __shfl(weight, s, EI_WAVE);
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] += x[e] * w;
    }
    ei::Vec4<bf16_t>::store(out + static_cast<size_t>(wave) * DV + d, o);
  }
}

struct Launch {
  int nk, ndv;
  const void* function;
};

template <int NK, int NDV>
const void* kernel_of() {
  return reinterpret_cast<const void*>(&attn_wide_kernel<NK, NDV>);
}

int heads_per_block(int G) { return G < kRows ? G : kRows; }

}  // namespace

// Whether the kernel takes these sizes: key rows (as a query meets them) a multiple of 32 up
// to 1024, the stored key head size a multiple of 8, values a multiple of 16 up to 512.
extern "C" int ei_attn_wide_supported(int DQ, int D, int DV) {
  return DQ >= 32 && DQ <= 1024 && DQ % 32 == 0 && D % 8 == 0 && DV >= 16 && DV <= 512 &&
         DV % 16 == 0;
}

// Positions of one sequence that a work item may hold, for G query heads a kv group.
extern "C" int ei_attn_wide_positions(int G) {
  const int hb = heads_per_block(G);
  return kRows / hb;
}

// q: [N, nq, key_heads * D]; key pages [pages, nkv, 64, D]; value pages [pages, nkv, 64, DV] (not
// read with values_in_keys); out [N, nq, DV]; all bfloat16.  Items as in ei_attention, with at
// most ei_attn_wide_positions positions each.  n_splits > 1: items of one position, scratch
// part_o [N, nq, n_splits, DV] and part_ml [N, nq, n_splits, 2], merged here.
extern "C" int ei_attention_wide(const void* q, const void* k_pages, const void* v_pages,
                                 const int32_t* item_seq, const int32_t* item_row0,
                                 const int32_t* item_npos, int n_items, const int32_t* row_pos,
                                 const int32_t* row_seq, const int32_t* page_table,
                                 int table_width, void* out, float* part_o, float* part_ml, int N,
                                 int nq, int nkv, int D, int DV, int window, const float* sinks,
                                 float scale, int n_splits, int key_heads, int values_in_keys,
                                 const float* gate, hipStream_t stream) {
  EI_REQUIRE(n_items > 0 && N > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention_wide: bad sizes");
  EI_REQUIRE(key_heads == 1 || key_heads == nkv,
             "attention_wide: a query meets the keys of its own kv head or of all of them");
  const int DQ = key_heads * D;
  EI_REQUIRE(ei_attn_wide_supported(DQ, D, DV), "attention_wide: head sizes not supported");
  EI_REQUIRE(!values_in_keys || DV <= D, "attention_wide: values inside keys cannot be wider");
  EI_REQUIRE(q && k_pages && out && item_seq && item_row0 && item_npos && row_pos && page_table &&
                 table_width > 0 && (values_in_keys || v_pages),
             "attention_wide: null pointer");
  EI_REQUIRE(n_splits >= 1 && n_splits <= 64, "attention_wide: splits must be between 1 and 64");
  EI_REQUIRE(n_splits == 1 || (part_o && part_ml), "attention_wide: split scratch missing");
  EI_REQUIRE(window >= 0, "attention_wide: negative window");
  const int G = nq / nkv;
  const int HB = heads_per_block(G);
  const int head_blocks = (G + HB - 1) / HB;
  EI_REQUIRE(static_cast<long long>(nkv) * head_blocks <= 65535, "attention_wide: too many heads");
  static const Launch table[] = {
      {4, 4, kernel_of<4, 4>()},     {8, 8, kernel_of<8, 8>()},     {16, 4, kernel_of<16, 4>()},
      {16, 8, kernel_of<16, 8>()},   {18, 16, kernel_of<18, 16>()}, {18, 32, kernel_of<18, 32>()},
      {32, 8, kernel_of<32, 8>()},   {32, 32, kernel_of<32, 32>()},
  };
  const int nk = DQ / 32, ndv = DV / 16;
  const Launch* chosen = nullptr;
  for (const Launch& entry : table)
    if (entry.nk >= nk && entry.ndv >= ndv) {
      chosen = &entry;
      break;
    }
  EI_REQUIRE(chosen != nullptr, "attention_wide: no kernel for these head sizes");
  const size_t lds = sizeof(bf16_t) * (static_cast<size_t>(kKeys) * (DQ + kPadK) +
                                       static_cast<size_t>(DV) * kVtRow);
  EI_REQUIRE(lds <= 160 * 1024, "attention_wide: head sizes too large for the LDS");
  if (lds > 64 * 1024) {        // beyond the default bound of a launch: ask for it, once a kernel
    static bool raised[sizeof(table) / sizeof(table[0])] = {false};
    const int index = static_cast<int>(chosen - table);
    if (!raised[index]) {
      if (hipFuncSetAttribute(chosen->function, hipFuncAttributeMaxDynamicSharedMemorySize,
                              160 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        EI_REQUIRE(false, "attention_wide: the device refuses the LDS these head sizes need");
      }
      raised[index] = true;
    }
  }
  dim3 grid(n_items, nkv * head_blocks, n_splits);
  const bf16_t* qp = static_cast<const bf16_t*>(q);
  const bf16_t* kp = static_cast<const bf16_t*>(k_pages);
  const bf16_t* vp = static_cast<const bf16_t*>(v_pages);
  bf16_t* op = static_cast<bf16_t*>(out);
  void* args[] = {&qp, &kp, &vp, &item_seq, &item_row0, &item_npos, &row_pos, &page_table,
                  &table_width, &op, &part_o, &part_ml, &nq, &nkv, &D, &DV, &key_heads,
                  &values_in_keys, const_cast<int*>(&HB), const_cast<int*>(&head_blocks), &window,
                  &sinks, &gate, &scale, &n_splits};
  hipError_t e = hipLaunchKernel(chosen->function, grid, dim3(kThreads), args, lds, stream);
  if (e != hipSuccess) {
    ei_set_error(hipGetErrorString(e));
    return static_cast<int>(e);
  }
  if (n_splits > 1) {
    const int total = N * nq;
    const int threads = 256;
    const int blocks = (total * EI_WAVE + threads - 1) / threads;
    wide_merge_kernel<<<blocks, threads, 0, stream>>>(part_o, part_ml, row_seq, op, nq, DV,
                                                      n_splits, total, gate);
  }
  EI_LAUNCH_CHECK();
}

// Per-head operations around attention over a compressed (latent) cache, and the mixing of
// queries over heads.  All sums, norms, angles and rotations are float32; inputs may be the
// float32 slices of a sliced product (they are added in slice order while they are read).
//
//   latent_down_store  one row of a fused down-projection [queries' latent | keys' latent |
//                      rotated key part | gate logits]: RMS norm of the two latents, the
//                      queries' latent out in the storage type, the keys' latent and the
//                      rotated key part into the row's cache page (one row of
//                      kv_rank + rot_dim elements a position), the gate logits out as float32
//   head_matmul        Y[n, h, :] = X[n, h, :] . M[h] for one matrix [in, out] a head
//   rotate_pairs       neighbouring elements (2i, 2i + 1) of a part of every head turn by
//                      position * frequency[i]
//   mix_heads          queries mixed over heads with a matrix T [heads, heads], kept apart by
//                      the kv head they meet: out[n, h, c, :] = sum over heads g of kv head c of
//                      T[h, g] q[n, g, :]
#include "common.h"

namespace {

template <typename TI>
__device__ __forceinline__ float sliced(const TI* p, int nsplit, size_t split_stride) {
  float x = 0.f;
  for (int s = 0; s < nsplit; ++s) x += ei::to_f32<TI>(p[s * split_stride]);
  return x;
}

template <typename TI, typename TO>
__global__ void latent_down_store_kernel(
    const TI* __restrict__ proj, int nsplit, size_t split_stride, int P,
    const float* __restrict__ q_norm_w, const float* __restrict__ c_norm_w, float eps,
    const float* __restrict__ freq, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_latent, TO* __restrict__ k_pages, float* __restrict__ gate_out, int q_rank,
    int kv_rank, int rot_dim, int n_gate, int write_cache) {
  extern __shared__ float row_values[];      // [P]
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int seq = row_seq[row];
  if (seq < 0) return;                       // a padding row of a fixed-size batch
  const TI* src = proj + static_cast<size_t>(row) * P;
  float sum_q = 0.f, sum_c = 0.f;
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    const float x = sliced<TI>(src + i, nsplit, split_stride);
    row_values[i] = x;
    if (i < q_rank) sum_q += x * x;
    else if (i < q_rank + kv_rank) sum_c += x * x;
  }
  const float inv_q =
      1.0f / sqrtf(ei::block_sum(sum_q, scratch) / static_cast<float>(q_rank) + eps);
  const float inv_c =
      1.0f / sqrtf(ei::block_sum(sum_c, scratch) / static_cast<float>(kv_rank) + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
    q_latent[static_cast<size_t>(row) * q_rank + i] =
        ei::from_f32<TO>((row_values[i] * inv_q) * q_norm_w[i]);
  for (int h = threadIdx.x; h < n_gate; h += blockDim.x)
    gate_out[static_cast<size_t>(row) * n_gate + h] = row_values[q_rank + kv_rank + rot_dim + h];
  if (!write_cache) return;
  const int pos = row_pos[row];
  const int page = page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE];
  if (page < 0) return;
  const int width = kv_rank + rot_dim;
  TO* dst = k_pages + (static_cast<size_t>(page) * EI_PAGE + pos % EI_PAGE) * width;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x)
    dst[i] = ei::from_f32<TO>((row_values[q_rank + i] * inv_c) * c_norm_w[i]);
  const float* turn = row_values + q_rank + kv_rank;
  for (int i = threadIdx.x; i < rot_dim / 2; i += blockDim.x) {
    const float angle = static_cast<float>(pos) * freq[i];
    float sn, cs;
    sincosf(angle, &sn, &cs);
    const float u = turn[2 * i], v = turn[2 * i + 1];
    dst[kv_rank + 2 * i] = ei::from_f32<TO>(u * cs - v * sn);
    dst[kv_rank + 2 * i + 1] = ei::from_f32<TO>(v * cs + u * sn);
  }
}

constexpr int kTileRows = 16;
constexpr int kTileK = 128;
constexpr int kCols = 64;            // output columns of a block
constexpr int kParts = 4;            // threads that share a column, each a quarter of a K tile

// Block: head blockIdx.y, rows blockIdx.x * 16 .., output columns blockIdx.z * 64 + t % 64; the
// four threads of a column take a quarter of every K tile each (all its weights requested at
// once, so that a step of few rows is not a chain of trips to memory) and add up through LDS.
template <typename TI, typename TW, typename TO>
__global__ void __launch_bounds__(256)
head_matmul_kernel(const TI* __restrict__ x, int nsplit, size_t split_stride, long long x_row,
                   int x_head, int x_first, const TW* __restrict__ m, TO* __restrict__ y,
                   long long y_row, int y_head, int y_first, int N, int K, int J) {
  __shared__ float xs[kTileRows][kTileK];
  __shared__ float sums[kParts][kTileRows][kCols];
  const int h = blockIdx.y;
  const int row0 = blockIdx.x * kTileRows;
  const int col = threadIdx.x % kCols, part = threadIdx.x / kCols;
  const int j = blockIdx.z * kCols + col;
  const TW* mh = m + static_cast<size_t>(h) * K * J;
  float acc[kTileRows];
#pragma unroll
  for (int r = 0; r < kTileRows; ++r) acc[r] = 0.f;
  constexpr int kQuarter = kTileK / kParts;
  for (int k0 = 0; k0 < K; k0 += kTileK) {
    const int kn = min(kTileK, K - k0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < kTileRows * kTileK; idx += 256) {
      const int r = idx / kTileK, k = idx % kTileK;
      float v = 0.f;
      if (row0 + r < N && k < kn)
        v = sliced<TI>(x + static_cast<size_t>(row0 + r) * x_row + h * x_head + x_first + k0 + k,
                       nsplit, split_stride);
      xs[r][k] = v;
    }
    __syncthreads();
    if (j < J) {
      const int k_lo = part * kQuarter, k_hi = min(kn, k_lo + kQuarter);
      // the thread's whole quarter of the tile is requested before any of it is used
      // (every load is unconditional, from a clamped place, so that none waits for a branch;
      // beyond the tile's end x holds zeros)
      TW w[kQuarter];
      const int last = K - 1 - k0;
#pragma unroll
      for (int u = 0; u < kQuarter; ++u)
        w[u] = mh[static_cast<size_t>(k0 + min(k_lo + u, last)) * J + j];
#pragma unroll
      for (int u = 0; u < kQuarter; ++u) {
        const float wu = ei::to_f32<TW>(w[u]);
#pragma unroll
        for (int r = 0; r < kTileRows; ++r) acc[r] += xs[r][k_lo + u] * wu;
      }
      (void)k_hi;
    }
  }
#pragma unroll
  for (int r = 0; r < kTileRows; ++r) sums[part][r][col] = acc[r];
  __syncthreads();
  // thread (part, col) finishes rows part, part + 4, ...
  if (j < J) {
    for (int r = part; r < kTileRows; r += kParts) {
      if (row0 + r < N) {
        const float total = (sums[0][r][col] + sums[1][r][col]) + (sums[2][r][col] + sums[3][r][col]);
        y[static_cast<size_t>(row0 + r) * y_row + h * y_head + y_first + j] = ei::from_f32<TO>(total);
      }
    }
  }
}

template <typename TI, typename TO>
__global__ void rotate_pairs_kernel(const TI* __restrict__ x, int nsplit, size_t split_stride,
                                    long long x_row, int x_head, int x_first,
                                    const float* __restrict__ freq,
                                    const int32_t* __restrict__ row_pos, TO* __restrict__ y,
                                    long long y_row, int y_head, int y_first, int heads, int half,
                                    size_t total) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t idx = start; idx < total; idx += step) {
    const int i = static_cast<int>(idx % half);
    const int h = static_cast<int>((idx / half) % heads);
    const size_t row = idx / (static_cast<size_t>(half) * heads);
    const TI* src = x + row * x_row + h * x_head + x_first + 2 * i;
    const float u = sliced<TI>(src, nsplit, split_stride);
    const float v = sliced<TI>(src + 1, nsplit, split_stride);
    const float angle = static_cast<float>(row_pos[row]) * freq[i];
    float sn, cs;
    sincosf(angle, &sn, &cs);
    TO* dst = y + row * y_row + h * y_head + y_first + 2 * i;
    dst[0] = ei::from_f32<TO>(u * cs - v * sn);
    dst[1] = ei::from_f32<TO>(v * cs + u * sn);
  }
}

template <typename T>
__global__ void mix_heads_kernel(const T* __restrict__ q, const float* __restrict__ talk,
                                 T* __restrict__ out, int heads, int kv_heads, int D,
                                 size_t total) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  const int share = heads / kv_heads;
  for (size_t idx = start; idx < total; idx += step) {
    const int d = static_cast<int>(idx % D);
    const int c = static_cast<int>((idx / D) % kv_heads);
    const int h = static_cast<int>((idx / (static_cast<size_t>(D) * kv_heads)) % heads);
    const size_t row = idx / (static_cast<size_t>(D) * kv_heads * heads);
    const T* src = q + (row * heads + static_cast<size_t>(c) * share) * D + d;
    const float* t = talk + static_cast<size_t>(h) * heads + c * share;
    float sum = 0.f;
    for (int g = 0; g < share; ++g) sum += t[g] * ei::to_f32<T>(src[static_cast<size_t>(g) * D]);
    out[idx] = ei::from_f32<T>(sum);
  }
}

// The same for head sizes that are a multiple of 8: a thread makes 8 neighbouring elements
// (16-byte accesses in bfloat16).
template <typename T>
__global__ void mix_heads_vec_kernel(const T* __restrict__ q, const float* __restrict__ talk,
                                     T* __restrict__ out, int heads, int kv_heads, int D,
                                     size_t total_octets) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  const int share = heads / kv_heads;
  const int octets = D / 8;
  for (size_t idx = start; idx < total_octets; idx += step) {
    const int d = static_cast<int>(idx % octets) * 8;
    const int c = static_cast<int>((idx / octets) % kv_heads);
    const int h = static_cast<int>((idx / (static_cast<size_t>(octets) * kv_heads)) % heads);
    const size_t row = idx / (static_cast<size_t>(octets) * kv_heads * heads);
    const T* src = q + (row * heads + static_cast<size_t>(c) * share) * D + d;
    const float* t = talk + static_cast<size_t>(h) * heads + c * share;
    float sum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = 0.f;
    for (int g = 0; g < share; ++g) {
      float x[8];
      ei::VecN<T, 8>::load(src + static_cast<size_t>(g) * D, x);
      const float w = t[g];
#pragma unroll
      for (int e = 0; e < 8; ++e) sum[e] += w * x[e];
    }
    ei::VecN<T, 8>::store(out + idx * 8, sum);
  }
}

inline unsigned capped_blocks(size_t n, int threads) {
  size_t blocks = (n + threads - 1) / threads;
  const size_t most = static_cast<size_t>(ei_compute_units()) * 16;
  return static_cast<unsigned>(blocks > most ? most : (blocks < 1 ? 1 : blocks));
}

}  // namespace

// proj: [nsplit][N, q_rank + kv_rank + rot_dim + n_gate]; k_pages: [pages, 1, 64, kv_rank + rot_dim].
extern "C" int ei_latent_down_store(const void* proj, int in_dtype, int nsplit,
                                    long long split_stride, const float* q_norm_w,
                                    const float* c_norm_w, float eps, const float* freq,
                                    const int32_t* row_pos, const int32_t* row_seq,
                                    const int32_t* page_table, int table_width, void* q_latent,
                                    void* k_pages, float* gate_out, int out_dtype, int N, int q_rank,
                                    int kv_rank, int rot_dim, int n_gate, int write_cache,
                                    hipStream_t stream) {
  EI_REQUIRE(N > 0 && q_rank > 0 && kv_rank > 0 && rot_dim >= 0 && rot_dim % 2 == 0 && n_gate >= 0,
             "latent_down_store: bad sizes");
  EI_REQUIRE(proj && q_norm_w && c_norm_w && row_pos && row_seq && q_latent && nsplit >= 1,
             "latent_down_store: null pointer");
  EI_REQUIRE(rot_dim == 0 || freq, "latent_down_store: a rotation needs its frequencies");
  EI_REQUIRE(n_gate == 0 || gate_out, "latent_down_store: gate logits need a place");
  EI_REQUIRE(!write_cache || (k_pages && page_table && table_width > 0),
             "latent_down_store: the cache is missing");
  const int P = q_rank + kv_rank + rot_dim + n_gate;
  const size_t lds = static_cast<size_t>(P) * sizeof(float);
  EI_REQUIRE(lds <= 60 * 1024, "latent_down_store: row too wide");
  // few rows: up to 1024 threads a row, so that a row's loads are in flight together
  const int threads = N <= 64 ? (P >= 768 ? 1024 : 512) : 256;
  const size_t ss = static_cast<size_t>(split_stride);
#define EI_LDS_CASE(TI, TO)                                                                     \
  latent_down_store_kernel<TI, TO><<<N, threads, lds, stream>>>(                                \
      static_cast<const TI*>(proj), nsplit, ss, P, q_norm_w, c_norm_w, eps, freq, row_pos,      \
      row_seq, page_table, table_width, static_cast<TO*>(q_latent), static_cast<TO*>(k_pages),  \
      gate_out, q_rank, kv_rank, rot_dim, n_gate, write_cache)
  if (in_dtype == EI_F32 && out_dtype == EI_F32) EI_LDS_CASE(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16) EI_LDS_CASE(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16) EI_LDS_CASE(bf16_t, bf16_t);
  else EI_REQUIRE(false, "latent_down_store: unsupported dtype combination");
#undef EI_LDS_CASE
  EI_LAUNCH_CHECK();
}

// x: [nsplit][N, x_row] read at x_head * h + x_first + 0..K; m: [heads, K, J] of the storage
// type; y: [N, y_row] written at y_head * h + y_first + 0..J.
extern "C" int ei_head_matmul(const void* x, int x_dtype, int nsplit, long long split_stride,
                              long long x_row, int x_head, int x_first, const void* m,
                              int m_dtype, void* y, int y_dtype, long long y_row, int y_head,
                              int y_first, int N, int heads, int K, int J, hipStream_t stream) {
  EI_REQUIRE(N > 0 && heads > 0 && K > 0 && J > 0 && nsplit >= 1, "head_matmul: bad sizes");
  EI_REQUIRE(x && m && y, "head_matmul: null pointer");
  EI_REQUIRE(x_first >= 0 && y_first >= 0 &&
                 static_cast<long long>(heads - 1) * x_head + x_first + K <= x_row &&
                 static_cast<long long>(heads - 1) * y_head + y_first + J <= y_row,
             "head_matmul: a head's part lies outside its row");
  EI_REQUIRE(heads <= 65535 && (J + kCols - 1) / kCols <= 65535,
             "head_matmul: too many heads or columns");
  dim3 grid((N + kTileRows - 1) / kTileRows, heads, (J + kCols - 1) / kCols);
  const size_t ss = static_cast<size_t>(split_stride);
#define EI_HM_CASE(TI, TW, TO)                                                                  \
  head_matmul_kernel<TI, TW, TO><<<grid, 256, 0, stream>>>(                                     \
      static_cast<const TI*>(x), nsplit, ss, x_row, x_head, x_first, static_cast<const TW*>(m), \
      static_cast<TO*>(y), y_row, y_head, y_first, N, K, J)
  if (x_dtype == EI_F32 && m_dtype == EI_F32 && y_dtype == EI_F32) EI_HM_CASE(float, float, float);
  else if (x_dtype == EI_F32 && m_dtype == EI_BF16 && y_dtype == EI_BF16) EI_HM_CASE(float, bf16_t, bf16_t);
  else if (x_dtype == EI_BF16 && m_dtype == EI_BF16 && y_dtype == EI_BF16) EI_HM_CASE(bf16_t, bf16_t, bf16_t);
  else EI_REQUIRE(false, "head_matmul: unsupported dtype combination");
#undef EI_HM_CASE
  EI_LAUNCH_CHECK();
}

extern "C" int ei_rotate_pairs(const void* x, int x_dtype, int nsplit, long long split_stride,
                               long long x_row, int x_head, int x_first, const float* freq,
                               const int32_t* row_pos, void* y, int y_dtype, long long y_row,
                               int y_head, int y_first, int N, int heads, int rot_dim,
                               hipStream_t stream) {
  EI_REQUIRE(N > 0 && heads > 0 && rot_dim > 0 && rot_dim % 2 == 0 && nsplit >= 1,
             "rotate_pairs: bad sizes");
  EI_REQUIRE(x && y && freq && row_pos, "rotate_pairs: null pointer");
  EI_REQUIRE(x_first >= 0 && y_first >= 0 &&
                 static_cast<long long>(heads - 1) * x_head + x_first + rot_dim <= x_row &&
                 static_cast<long long>(heads - 1) * y_head + y_first + rot_dim <= y_row,
             "rotate_pairs: a head's part lies outside its row");
  const int half = rot_dim / 2;
  const size_t total = static_cast<size_t>(N) * heads * half;
  const size_t ss = static_cast<size_t>(split_stride);
  const unsigned blocks = capped_blocks(total, 256);
#define EI_RP_CASE(TI, TO)                                                                     \
  rotate_pairs_kernel<TI, TO><<<blocks, 256, 0, stream>>>(                                     \
      static_cast<const TI*>(x), nsplit, ss, x_row, x_head, x_first, freq, row_pos,            \
      static_cast<TO*>(y), y_row, y_head, y_first, heads, half, total)
  if (x_dtype == EI_F32 && y_dtype == EI_F32) EI_RP_CASE(float, float);
  else if (x_dtype == EI_F32 && y_dtype == EI_BF16) EI_RP_CASE(float, bf16_t);
  else if (x_dtype == EI_BF16 && y_dtype == EI_BF16) EI_RP_CASE(bf16_t, bf16_t);
  else EI_REQUIRE(false, "rotate_pairs: unsupported dtype combination");
#undef EI_RP_CASE
  EI_LAUNCH_CHECK();
}

// q: [N, heads, D]; talk: float32 [heads, heads]; out: [N, heads, kv_heads, D].
extern "C" int ei_mix_heads(const void* q, int dtype, const float* talk, void* out, int N,
                            int heads, int kv_heads, int D, hipStream_t stream) {
  EI_REQUIRE(N > 0 && heads > 0 && kv_heads > 0 && D > 0 && heads % kv_heads == 0,
             "mix_heads: bad sizes");
  EI_REQUIRE(q && talk && out, "mix_heads: null pointer");
  const size_t total = static_cast<size_t>(N) * heads * kv_heads * D;
  if (D % 8 == 0) {
    const size_t octets = total / 8;
    const unsigned vblocks = capped_blocks(octets, 256);
    if (dtype == EI_F32)
      mix_heads_vec_kernel<float><<<vblocks, 256, 0, stream>>>(
          static_cast<const float*>(q), talk, static_cast<float*>(out), heads, kv_heads, D, octets);
    else if (dtype == EI_BF16)
      mix_heads_vec_kernel<bf16_t><<<vblocks, 256, 0, stream>>>(
          static_cast<const bf16_t*>(q), talk, static_cast<bf16_t*>(out), heads, kv_heads, D, octets);
    else
      EI_REQUIRE(false, "mix_heads: unknown dtype");
    EI_LAUNCH_CHECK();
  }
  const unsigned blocks = capped_blocks(total, 256);
  if (dtype == EI_F32)
    mix_heads_kernel<float><<<blocks, 256, 0, stream>>>(
        static_cast<const float*>(q), talk, static_cast<float*>(out), heads, kv_heads, D, total);
  else if (dtype == EI_BF16)
    mix_heads_kernel<bf16_t><<<blocks, 256, 0, stream>>>(
        static_cast<const bf16_t*>(q), talk, static_cast<bf16_t*>(out), heads, kv_heads, D, total);
  else
    EI_REQUIRE(false, "mix_heads: unknown dtype");
  EI_LAUNCH_CHECK();
}

// Matrix memory with exponential gates (the mLSTM cell): per head and sequence a state
// S [key size, value size], a normaliser n [key size] and a running maximum m of the log gates,
// all float32, carried from token to token.
//
// For token t with log input gate i_t and log forget gate f_t (m_0 = 0, S_0 = 0, n_0 = 0):
//   m_t = max(f_t + m_{t-1}, i_t)
//   S_t = e^(f_t + m_{t-1} - m_t) S_{t-1} + e^(i_t - m_t) k_t v_t^T     (n_t alike, with k_t alone)
//   o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + bottom_eps)
// The gates come from two columns a head of the fused projection: with a cap c,
//   i_t = c tanh((x_i + b_i) / c),   f_t = logsigmoid(c tanh((x_f + b_f) / c)).
//
// `mlstm_walk`: a block of one wave per (sequence, head, block of columns of S) walks the
// sequence's rows of the step in order.  A thread owns 8 neighbouring rows of one, two or four
// neighbouring columns of S in registers (and the same rows of n, which all its columns share);
// the L = key size / 8 lanes that share the columns add their partial dot products with DPP
// adds (a row swap for L = 32).  A wave that is alone on its SIMD pays for every instruction of
// a token in full, so a launch of few blocks takes one column a thread (the fewest instructions
// a token); where the chip is full anyway, four columns a thread read and update k, q and n
// once for four columns (the fewest instructions in all).  Tokens come through LDS in tiles of 16: q, k
// (16 bytes a load where the projection is bfloat16), the block's columns of v, and the three
// factors of every token.  A lane a token works those out: with F_t the sum of the tile's log
// forget gates up to t, m_t = F_t + max(m before the tile, max over s <= t of (i_s - F_s)), a
// prefix sum and a prefix maximum over the lanes, so nothing but S itself is a chain.
// The state is read from one row of the table and written, whole, to another (the table has two
// versions a sequence).
// `mlstm_out`: a wave a (row, head): RMS norm of the read-out, a weight as wide as all heads,
// a sigmoid gate from the projection, one rounding.
#include "common.h"

namespace {

constexpr int kThreads = EI_WAVE;   // a block is one wave
constexpr int kTile = 16;           // tokens in LDS at a time
constexpr int kOwn = 8;             // rows of a column that a thread owns
constexpr int kMostCols = 4;        // most columns of S that a thread owns (1, 2 or 4)

template <typename TI>
__device__ __forceinline__ float sliced(const TI* p, int nsplit, size_t split_stride) {
  float x = 0.f;
  for (int s = 0; s < nsplit; ++s) x += ei::to_f32<TI>(p[s * split_stride]);
  return x;
}

__device__ __forceinline__ float log_sigmoid(float z) {
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

#define EI_DPP_ADD(v, ctrl)                                                                     \
  ((v) + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), \
                                                                (ctrl), 0xf, 0xf, false)))

// Sum over each aligned group of L neighbouring lanes (L a power of two up to 32), every lane
// of the group getting it: quad permutes, mirrors of half rows and rows, a swap of
// neighbouring rows.
__device__ __forceinline__ float group_sum(float v, int L) {
  if (L >= 2) v = EI_DPP_ADD(v, 0xb1);     // quad_perm [1,0,3,2]
  if (L >= 4) v = EI_DPP_ADD(v, 0x4e);     // quad_perm [2,3,0,1]
  if (L >= 8) v = EI_DPP_ADD(v, 0x141);    // row_half_mirror
  if (L >= 16) v = EI_DPP_ADD(v, 0x140);   // row_mirror
  if (L >= 32) {
    const ei::ei_u32x2 r =
        __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r.x) + __uint_as_float(r.y);
  }
  return v;
}

// Floats of one head's state: S^T [vdim, dim], n [dim], m, padded to a multiple of 4 so that
// every head's part starts at a 16-byte boundary.
__host__ __device__ inline size_t head_state_floats(int dim, int vdim) {
  return (static_cast<size_t>(vdim) * dim + dim + 1 + 3) / 4 * 4;
}

// Column offsets of the fused projection [q | k | v | i | f | g].
struct Columns {
  int q, k, v, i, f, g, width;
};

__host__ __device__ inline Columns columns_of(int heads, int dim, int vdim) {
  Columns c;
  c.q = 0;
  c.k = heads * dim;
  c.v = 2 * heads * dim;
  c.i = c.v + heads * vdim;
  c.f = c.i + heads;
  c.g = c.f + heads;
  c.width = c.g + heads * vdim;
  return c;
}

template <typename TI, int NC>
__global__ void __launch_bounds__(kThreads)
mlstm_walk_kernel(const TI* __restrict__ proj, int nsplit, size_t split_stride,
                  const float* __restrict__ i_bias, const float* __restrict__ f_bias,
                  float* __restrict__ state, size_t state_stride,
                  const int32_t* __restrict__ seq_in, const int32_t* __restrict__ seq_out,
                  const int32_t* __restrict__ seq_count, const int32_t* __restrict__ seq_row0,
                  float* __restrict__ o_raw, int heads, int dim, int vdim, int L, float cap,
                  float q_scale, float bottom_eps, int tile_rows) {
  // (tile_rows: tokens in LDS at a time, kTile, or 1 where every sequence brings one token: a
  // decode step then needs a sixteenth of the LDS, and many more waves fit a compute unit)
  extern __shared__ float lds[];
  constexpr int OWN = kOwn;
  const int dimP = L * OWN;
  const int CB = kThreads / L * NC;            // columns of S this block owns
  float* qs = lds;                             // [tile_rows][dimP]
  float* ks = qs + tile_rows * dimP;           // [tile_rows][dimP]
  float* vs = ks + tile_rows * dimP;           // [tile_rows][CB]
  float* keep_s = vs + tile_rows * CB;         // [tile_rows] e^(f + m' - m)
  float* take_s = keep_s + tile_rows;          // [tile_rows] e^(i - m)
  float* floor_s = take_s + tile_rows;         // [tile_rows] e^(-m)

  const int seq = blockIdx.x / heads, a = blockIdx.x % heads;
  const int count = seq_count[seq];
  if (count <= 0) return;                      // padding of a fixed-size batch
  const int row0 = seq_row0[seq];
  const Columns col_of = columns_of(heads, dim, vdim);
  const int P = col_of.width;
  const int t = threadIdx.x;
  const int part = t % L, group = t / L;
  const int col0 = blockIdx.y * CB + group * NC;      // the thread's first column
  const int r0 = part * OWN;
  const size_t head_floats = head_state_floats(dim, vdim);
  const float* in = state + static_cast<size_t>(seq_in[seq]) * state_stride + a * head_floats;
  float* out = state + static_cast<size_t>(seq_out[seq]) * state_stride + a * head_floats;
  // 16-byte loads of q and k: a bfloat16 projection whose head parts start at multiples of 8
  const bool octets = sizeof(TI) == 2 && nsplit == 1 && dim % 8 == 0 && P % 8 == 0;

  float S[NC][OWN], nn[OWN];
  const bool quads = dim % 4 == 0;             // 16-byte accesses to the state
  if (quads) {
#pragma unroll
    for (int r = 0; r < OWN; r += 4) {
      const bool live = r0 + r < dim;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        float x[4] = {0.f, 0.f, 0.f, 0.f};
        if (live && col0 + c < vdim) ei::Vec4<float>::load(in + static_cast<size_t>(col0 + c) * dim + r0 + r, x);
#pragma unroll
        for (int e = 0; e < 4; ++e) S[c][r + e] = x[e];
      }
      float x[4] = {0.f, 0.f, 0.f, 0.f};
      if (live) ei::Vec4<float>::load(in + static_cast<size_t>(vdim) * dim + r0 + r, x);
#pragma unroll
      for (int e = 0; e < 4; ++e) nn[r + e] = x[e];
    }
  } else {
#pragma unroll
    for (int r = 0; r < OWN; ++r) {
      const bool live = r0 + r < dim;
#pragma unroll
      for (int c = 0; c < NC; ++c)
        S[c][r] = (live && col0 + c < vdim) ? in[static_cast<size_t>(col0 + c) * dim + r0 + r] : 0.f;
      nn[r] = live ? in[static_cast<size_t>(vdim) * dim + r0 + r] : 0.f;
    }
  }
  float m_run = in[static_cast<size_t>(vdim) * dim + dim];

  // A long walk over a bfloat16 projection asks for a whole tile at once, from clamped places
  // so that no load waits for a branch, and for the next tile while it walks this one.
  constexpr int kAhead = 8;                    // most loads of a kind that a lane has in flight
  const int per_row = dimP / 8;
  const int qk_loads = (kTile * per_row + kThreads - 1) / kThreads;
  const int v_loads = (kTile * CB + kThreads - 1) / kThreads;
  const bool ahead = octets && tile_rows == kTile && qk_loads <= kAhead && v_loads <= kAhead;
  const bf16_t* rows16 = reinterpret_cast<const bf16_t*>(proj);
  uint4 q_pre[kAhead], k_pre[kAhead];
  bf16_t v_pre[kAhead], xi_pre = 0, xf_pre = 0;
  auto ask = [&](int t0) {
    const int tn = min(kTile, count - t0);
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      if (i < qk_loads) {
        const int idx = t + i * kThreads;
        const int tt = min(idx / per_row, tn - 1), d = min((idx % per_row) * 8, dim - 8);
        const bf16_t* src = rows16 + static_cast<size_t>(row0 + t0 + tt) * P + a * dim + d;
        q_pre[i] = *reinterpret_cast<const uint4*>(src + col_of.q);
        k_pre[i] = *reinterpret_cast<const uint4*>(src + col_of.k);
      }
    }
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      if (i < v_loads) {
        const int idx = t + i * kThreads;
        const int tt = min(idx / CB, tn - 1), c = min(blockIdx.y * CB + idx % CB, vdim - 1);
        v_pre[i] = rows16[static_cast<size_t>(row0 + t0 + tt) * P + col_of.v + a * vdim + c];
      }
    }
    const bf16_t* gates = rows16 + static_cast<size_t>(row0 + t0 + min(t, tn - 1)) * P;
    xi_pre = gates[col_of.i + a];
    xf_pre = gates[col_of.f + a];
  };
  if (ahead) ask(0);

  for (int t0 = 0; t0 < count; t0 += tile_rows) {
    const int tn = min(tile_rows, count - t0);
    __syncthreads();
    if (ahead) {
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        const int idx = t + i * kThreads;
        if (i < qk_loads && idx < tn * per_row) {   // (rows beyond the tile's tokens are never read)
          const int tt = idx / per_row, d = (idx % per_row) * 8;
          const bool live = tt < tn && d < dim;
          const uint32_t qw[4] = {q_pre[i].x, q_pre[i].y, q_pre[i].z, q_pre[i].w};
          const uint32_t kw[4] = {k_pre[i].x, k_pre[i].y, k_pre[i].z, k_pre[i].w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            qs[tt * dimP + d + 2 * e] = live ? __uint_as_float(qw[e] << 16) * q_scale : 0.f;
            qs[tt * dimP + d + 2 * e + 1] = live ? __uint_as_float(qw[e] & 0xffff0000u) * q_scale : 0.f;
            ks[tt * dimP + d + 2 * e] = live ? __uint_as_float(kw[e] << 16) : 0.f;
            ks[tt * dimP + d + 2 * e + 1] = live ? __uint_as_float(kw[e] & 0xffff0000u) : 0.f;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        const int idx = t + i * kThreads;
        if (i < v_loads && idx < tn * CB) {
          const bool live = idx / CB < tn && blockIdx.y * CB + idx % CB < vdim;
          vs[idx] = live ? ei::bf16_to_f32(v_pre[i]) : 0.f;
        }
      }
    } else if (octets) {
      for (int idx = t; idx < tn * per_row; idx += kThreads) {
        const int tt = idx / per_row, d = (idx % per_row) * 8;
        float qv[8], kv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) qv[e] = kv[e] = 0.f;
        if (tt < tn && d < dim) {
          const bf16_t* src = rows16 + static_cast<size_t>(row0 + t0 + tt) * P + a * dim + d;
          ei::VecN<bf16_t, 8>::load(src + col_of.q, qv);
          ei::VecN<bf16_t, 8>::load(src + col_of.k, kv);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          qs[tt * dimP + d + e] = qv[e] * q_scale;
          ks[tt * dimP + d + e] = kv[e];
        }
      }
    } else {
      for (int idx = t; idx < tn * dimP; idx += kThreads) {
        const int tt = idx / dimP, d = idx % dimP;
        float qv = 0.f, kv = 0.f;
        if (tt < tn && d < dim) {
          const TI* src = proj + static_cast<size_t>(row0 + t0 + tt) * P + a * dim + d;
          qv = sliced<TI>(src + col_of.q, nsplit, split_stride) * q_scale;
          kv = sliced<TI>(src + col_of.k, nsplit, split_stride);
        }
        qs[idx] = qv;
        ks[idx] = kv;
      }
    }
    if (!ahead) {
      for (int idx = t; idx < tn * CB; idx += kThreads) {
        const int tt = idx / CB, c = blockIdx.y * CB + idx % CB;
        float v = 0.f;
        if (tt < tn && c < vdim)
          v = sliced<TI>(proj + static_cast<size_t>(row0 + t0 + tt) * P + col_of.v + a * vdim + c,
                         nsplit, split_stride);
        vs[idx] = v;
      }
    }
    {
      // lane t: token t of the tile (lanes beyond the tile's tokens carry neutral gates)
      float li = -INFINITY, lf = 0.f;
      if (t < tn) {
        float xi, xf;
        if (ahead) {
          xi = ei::bf16_to_f32(xi_pre);
          xf = ei::bf16_to_f32(xf_pre);
        } else {
          const TI* src = proj + static_cast<size_t>(row0 + t0 + t) * P;
          xi = sliced<TI>(src + col_of.i + a, nsplit, split_stride);
          xf = sliced<TI>(src + col_of.f + a, nsplit, split_stride);
        }
        xi += i_bias[a];
        xf += f_bias[a];
        li = cap * tanhf(xi / cap);
        lf = log_sigmoid(cap * tanhf(xf / cap));
      }
      // the next tile's loads travel while this one is walked
      if (ahead && t0 + kTile < count) ask(t0 + kTile);      // (ahead: tile_rows is kTile)
      float F = lf;                              // sum of the log forget gates up to this token
#pragma unroll
      for (int step = 1; step < kTile; step *= 2) {
        const float other = __shfl_up(F, step, EI_WAVE);
        if (t >= step) F += other;
      }
      float u = li - F;                          // largest i_s - F_s up to this token
#pragma unroll
      for (int step = 1; step < kTile; step *= 2) {
        const float other = __shfl_up(u, step, EI_WAVE);
        if (t >= step) u = fmaxf(u, other);
      }
      const float m_here = F + fmaxf(m_run, u);
      float m_before = __shfl_up(m_here, 1, EI_WAVE);
      if (t == 0) m_before = m_run;
      if (t < tn) {
        keep_s[t] = expf(lf + m_before - m_here);
        take_s[t] = expf(li - m_here);
        floor_s[t] = expf(-m_here);
      }
      m_run = __shfl(m_here, tn - 1, EI_WAVE);   // every lane carries the tile's last m
    }
    __syncthreads();
#pragma unroll 4
    for (int tt = 0; tt < tn; ++tt) {
      const float keep = keep_s[tt], take = take_s[tt];
      float tv[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) tv[c] = take * vs[tt * CB + group * NC + c];
      const float* kr = ks + tt * dimP + r0;
      const float* qr = qs + tt * dimP + r0;
      float kk[OWN], qq[OWN];
#pragma unroll
      for (int r = 0; r < OWN; r += 4) {
        ei::Vec4<float>::load(kr + r, *reinterpret_cast<float(*)[4]>(&kk[r]));
        ei::Vec4<float>::load(qr + r, *reinterpret_cast<float(*)[4]>(&qq[r]));
      }
      float dot_s[NC], dot_n = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) dot_s[c] = 0.f;
#pragma unroll
      for (int r = 0; r < OWN; ++r) {
        nn[r] = keep * nn[r] + take * kk[r];
        dot_n += nn[r] * qq[r];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          S[c][r] = keep * S[c][r] + kk[r] * tv[c];
          dot_s[c] += S[c][r] * qq[r];
        }
      }
      dot_n = group_sum(dot_n, L);
#pragma unroll
      for (int c = 0; c < NC; ++c) dot_s[c] = group_sum(dot_s[c], L);
      if (part == 0) {
        // (one division a token: the columns share the denominator)
        const float over = 1.0f / (fmaxf(fabsf(dot_n), floor_s[tt]) + bottom_eps);
        float* dst = o_raw + static_cast<size_t>(row0 + t0 + tt) * heads * vdim + a * vdim + col0;
#pragma unroll
        for (int c = 0; c < NC; ++c)
          if (col0 + c < vdim) dst[c] = dot_s[c] * over;
      }
    }
  }

  if (quads) {
#pragma unroll
    for (int r = 0; r < OWN; r += 4) {
      if (r0 + r < dim) {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const float x[4] = {S[c][r], S[c][r + 1], S[c][r + 2], S[c][r + 3]};
          if (col0 + c < vdim) ei::Vec4<float>::store(out + static_cast<size_t>(col0 + c) * dim + r0 + r, x);
        }
        const float x[4] = {nn[r], nn[r + 1], nn[r + 2], nn[r + 3]};
        if (blockIdx.y == 0 && group == 0)
          ei::Vec4<float>::store(out + static_cast<size_t>(vdim) * dim + r0 + r, x);
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < OWN; ++r) {
      if (r0 + r < dim) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
          if (col0 + c < vdim) out[static_cast<size_t>(col0 + c) * dim + r0 + r] = S[c][r];
        if (blockIdx.y == 0 && group == 0) out[static_cast<size_t>(vdim) * dim + r0 + r] = nn[r];
      }
    }
  }
  if (blockIdx.y == 0 && t == 0) out[static_cast<size_t>(vdim) * dim + dim] = m_run;
}

// One wave per (row, head).
template <typename TI, typename TO>
__global__ void mlstm_out_kernel(const float* __restrict__ o_raw, const TI* __restrict__ proj,
                                 int nsplit, size_t split_stride,
                                 const float* __restrict__ norm_w, float eps,
                                 const int32_t* __restrict__ row_seq, TO* __restrict__ out,
                                 int heads, int dim, int vdim, int total) {
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= total) return;
  const int row = wave / heads, a = wave % heads;
  if (row_seq[row] < 0) return;
  const Columns col_of = columns_of(heads, dim, vdim);
  const float* o = o_raw + (static_cast<size_t>(row) * heads + a) * vdim;
  float sum = 0.f;
  for (int j = lane; j < vdim; j += EI_WAVE) sum += o[j] * o[j];
  sum = ei::wave_sum(sum);
  const float inv = 1.0f / sqrtf(sum / static_cast<float>(vdim) + eps);
  const TI* g = proj + static_cast<size_t>(row) * col_of.width + col_of.g + a * vdim;
  for (int j = lane; j < vdim; j += EI_WAVE) {
    const float gate = 1.0f / (1.0f + expf(-sliced<TI>(g + j, nsplit, split_stride)));
    out[(static_cast<size_t>(row) * heads + a) * vdim + j] =
        ei::from_f32<TO>((o[j] * inv) * norm_w[a * vdim + j] * gate);
  }
}

int lanes_for(int dim) {
  int L = 1;
  while (L * kOwn < dim) L *= 2;
  return L;
}

}  // namespace

// Floats of one sequence's state: per head S^T [vdim, dim], n [dim], m and padding to a
// multiple of 4.
extern "C" int ei_mlstm_state_floats(int heads, int dim, int vdim) {
  return heads * static_cast<int>(head_state_floats(dim, vdim));
}

// Width of the fused projection [q | k | v | i | f | g].
extern "C" int ei_mlstm_proj_width(int heads, int dim, int vdim) {
  return columns_of(heads, dim, vdim).width;
}

// proj: [nsplit][N, width]; state: rows of `state_stride` floats; seq_in / seq_out: the row
// each sequence's state is read from and written to; o_raw: float32 [N, heads * vdim].
extern "C" int ei_mlstm_walk(const void* proj, int dtype, int nsplit, long long split_stride,
                             const float* i_bias, const float* f_bias, float* state,
                             long long state_stride, const int32_t* seq_in, const int32_t* seq_out,
                             const int32_t* seq_count, const int32_t* seq_row0, float* o_raw,
                             int n_seqs, int heads, int dim, int vdim, float cap, float q_scale,
                             float bottom_eps, int rows, hipStream_t stream) {
  EI_REQUIRE(n_seqs > 0 && heads > 0 && vdim > 0 && nsplit >= 1 && rows >= 1, "mlstm_walk: bad sizes");
  EI_REQUIRE(dim >= 1 && dim <= 256, "mlstm_walk: the key size must lie in 1..256");
  EI_REQUIRE(cap > 0.f, "mlstm_walk: the cap of the gates must be positive");
  EI_REQUIRE(proj && i_bias && f_bias && state && seq_in && seq_out && seq_count && seq_row0 &&
                 o_raw,
             "mlstm_walk: null pointer");
  EI_REQUIRE(state_stride >= ei_mlstm_state_floats(heads, dim, vdim) && state_stride % 4 == 0,
             "mlstm_walk: state rows too short, or no multiple of 4 floats");
  const int L = lanes_for(dim);
  // columns a thread: as many (4, 2, 1) as still give every SIMD of the chip two waves
  const long long wanted = 2LL * 4 * ei_compute_units();
  int nc = kMostCols;
  while (nc > 1 && static_cast<long long>(n_seqs) * heads *
                           ((vdim + kThreads / L * nc - 1) / (kThreads / L * nc)) < wanted)
    nc /= 2;
  const int CB = kThreads / L * nc;
  // no more rows than sequences: every sequence brings one token at most (a decode step)
  const int tile_rows = rows <= n_seqs ? 1 : kTile;
  const size_t lds = sizeof(float) * (2 * static_cast<size_t>(tile_rows) * L * kOwn +
                                      static_cast<size_t>(tile_rows) * CB + 3 * tile_rows);
  EI_REQUIRE(static_cast<long long>(n_seqs) * heads <= 0x7fffffffLL, "mlstm_walk: too many blocks");
  EI_REQUIRE((vdim + CB - 1) / CB <= 65535, "mlstm_walk: too many blocks of columns");
  dim3 grid(n_seqs * heads, (vdim + CB - 1) / CB);
  const size_t ss = static_cast<size_t>(split_stride);
#define EI_WALK(TI, NC)                                                                        \
  mlstm_walk_kernel<TI, NC><<<grid, kThreads, lds, stream>>>(                                  \
      static_cast<const TI*>(proj), nsplit, ss, i_bias, f_bias, state,                         \
      static_cast<size_t>(state_stride), seq_in, seq_out, seq_count, seq_row0, o_raw, heads,   \
      dim, vdim, L, cap, q_scale, bottom_eps, tile_rows)
#define EI_WALK_COLS(TI)              \
  do {                                \
    if (nc == 4) EI_WALK(TI, 4);      \
    else if (nc == 2) EI_WALK(TI, 2); \
    else EI_WALK(TI, 1);              \
  } while (0)
  if (dtype == EI_F32) EI_WALK_COLS(float);
  else if (dtype == EI_BF16) EI_WALK_COLS(bf16_t);
  else EI_REQUIRE(false, "mlstm_walk: unknown dtype");
#undef EI_WALK_COLS
#undef EI_WALK
  EI_LAUNCH_CHECK();
}

extern "C" int ei_mlstm_out(const float* o_raw, const void* proj, int in_dtype, int nsplit,
                            long long split_stride, const float* norm_w, float eps,
                            const int32_t* row_seq, void* out, int out_dtype, int N, int heads,
                            int dim, int vdim, hipStream_t stream) {
  EI_REQUIRE(N > 0 && heads > 0 && dim > 0 && vdim > 0 && nsplit >= 1, "mlstm_out: bad sizes");
  EI_REQUIRE(o_raw && proj && norm_w && row_seq && out, "mlstm_out: null pointer");
  const int total = N * heads;
  const int threads = 256;
  const int blocks = (total * EI_WAVE + threads - 1) / threads;
  const size_t ss = static_cast<size_t>(split_stride);
#define EI_MO_CASE(TI, TO)                                                                   \
  mlstm_out_kernel<TI, TO><<<blocks, threads, 0, stream>>>(                                  \
      o_raw, static_cast<const TI*>(proj), nsplit, ss, norm_w, eps, row_seq,                 \
      static_cast<TO*>(out), heads, dim, vdim, total)
  if (in_dtype == EI_F32 && out_dtype == EI_F32) EI_MO_CASE(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16) EI_MO_CASE(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16) EI_MO_CASE(bf16_t, bf16_t);
  else EI_REQUIRE(false, "mlstm_out: unsupported dtype combination");
#undef EI_MO_CASE
  EI_LAUNCH_CHECK();
}

// Gated delta rule: a recurrent mixer whose state is one matrix S [D, DV] per head and
// sequence, fed through short causal convolutions.  Per token t and head h (query/key head
// h / (H / G)), everything in float32:
//
//   x      = silu(conv(projection))          for the q, k and v channels (J taps a channel,
//                                            the last one on the current token, zeros before
//                                            the sequence starts)
//   q, k   = x / sqrt(sum(x^2) + unit_eps)   per head; q also times q_scale
//   beta   = sigmoid(b),  g = exp(-exp(A_log) * softplus(a + dt_bias))
//   S     <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//   out    = o / sqrt(mean(o^2) + eps) * w * silu(gate)
//
// Per sequence the cache keeps S (stored transposed, [H, DV, D], so that the D values a
// thread owns are contiguous) and the last J - 1 inputs of every convolved channel.  One
// set of kernels serves prompts (rows of a sequence are walked in order) and decoding (one
// row a sequence):
//
//   delta_conv   convolution + silu of all q, k, v channels of every row
//   delta_tail   the new last J - 1 inputs of every sequence (after delta_conv has read the
//                old ones)
//   delta_rule   the recurrence; a thread owns 8 or 16 rows of one column of S, L lanes share a
//                column; tokens come in tiles through LDS
//   delta_out    the read-out's norm and gate
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kTile = 32;        // most tokens of a sequence that delta_rule stages in LDS at a time
constexpr int kMaxTaps = 32;
constexpr int kFewTaps = 8;      // up to so many taps a thread keeps a channel's inputs in registers

template <typename TI>
__device__ __forceinline__ float slice_sum(const TI* p, int nsplit, size_t stride) {
  float x = 0.f;
  for (int s0 = 0; s0 < nsplit; s0 += 8) {        // eight slices per trip to memory, added in order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + u < nsplit) v[u] = ei::to_f32<TI>(p[(s0 + u) * stride]);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + u < nsplit) x += v[u];
  }
  return x;
}

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

__device__ __forceinline__ float softplus_f32(float x) {
  return x > 30.f ? x : log1pf(expf(x));
}

// proj: [nsplit][N, WP]; the convolved channels are its first C columns.  conv_w: [C, J].
// new_tail_state (the state again, or null): a step in which every sequence brings one row
// may have the tails renewed here (up to kFewTaps taps), which saves the launch of delta_tail.
// The tail of a sequence (its last J - 1 inputs before this step, oldest first) lies at
// state + row * state_stride + tail_offset as [J - 1, C]; a sequence's state is read from row
// seq_in[seq] and written to row seq_out[seq] (the same row, or the other of two versions).
template <typename TI>
__global__ void delta_conv_kernel(const TI* __restrict__ proj, int nsplit, size_t split_stride,
                                  int WP, const float* __restrict__ conv_w, int J,
                                  const float* __restrict__ state, size_t state_stride,
                                  size_t tail_offset, const int32_t* __restrict__ row_pos,
                                  const int32_t* __restrict__ row_seq,
                                  const int32_t* __restrict__ seq_in,
                                  const int32_t* __restrict__ seq_out,
                                  const int32_t* __restrict__ seq_start, float* __restrict__ out,
                                  int C, float* __restrict__ new_tail_state) {
  const size_t row = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int seq = row_seq[row];
  if (seq < 0 || c >= C) return;
  const int pos = row_pos[row], start = seq_start[seq];
  const float* tail = state + static_cast<size_t>(seq_in[seq]) * state_stride + tail_offset;
  auto input = [&](int j) {                  // the input that tap j multiplies
    const int back = J - 1 - j;
    const int p = pos - back;
    if (p >= start) return slice_sum(proj + (row - back) * WP + c, nsplit, split_stride);
    if (p >= 0) return tail[static_cast<size_t>(p - start + J - 1) * C + c];
    return 0.f;
  };
  float acc = 0.f;
  if (J <= kFewTaps) {                       // every input is asked for before the first is used
    float x[kFewTaps];
#pragma unroll
    for (int j = 0; j < kFewTaps; ++j) x[j] = j < J ? input(j) : 0.f;
#pragma unroll
    for (int j = 0; j < kFewTaps; ++j)
      if (j < J) acc += conv_w[static_cast<size_t>(c) * J + j] * x[j];
    if (new_tail_state) {
      // every sequence brings this one row (the caller says so): the thread is the only
      // reader of its channel's tail, and the new tail is the inputs it holds, moved by one
      float* to = new_tail_state + static_cast<size_t>(seq_out[seq]) * state_stride + tail_offset;
#pragma unroll
      for (int j = 1; j < kFewTaps; ++j)
        if (j < J) to[static_cast<size_t>(j - 1) * C + c] = x[j];
    }
  } else {
    for (int j = 0; j < J; ++j) acc += conv_w[static_cast<size_t>(c) * J + j] * input(j);
  }
  out[row * C + c] = silu_f32(acc);
}

// The same for four neighbouring channels a thread (channel counts, row widths and slice
// strides that are multiples of 4, up to kFewTaps taps): 8- or 16-byte loads of the inputs, the
// filters of four channels as J consecutive 16-byte pieces, one 16-byte store.
template <typename TI>
__global__ void delta_conv_vec_kernel(const TI* __restrict__ proj, int nsplit, size_t split_stride,
                                      int WP, const float* __restrict__ conv_w, int J,
                                      const float* __restrict__ state, size_t state_stride,
                                      size_t tail_offset, const int32_t* __restrict__ row_pos,
                                      const int32_t* __restrict__ row_seq,
                                      const int32_t* __restrict__ seq_in,
                                      const int32_t* __restrict__ seq_out,
                                      const int32_t* __restrict__ seq_start,
                                      float* __restrict__ out, int C,
                                      float* __restrict__ new_tail_state) {
  const size_t row = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
  const int seq = row_seq[row];
  if (seq < 0 || c >= C) return;
  const int pos = row_pos[row], start = seq_start[seq];
  const float* tail = state + static_cast<size_t>(seq_in[seq]) * state_stride + tail_offset;
  float x[kFewTaps][4];
#pragma unroll
  for (int j = 0; j < kFewTaps; ++j) {
    x[j][0] = x[j][1] = x[j][2] = x[j][3] = 0.f;
    if (j < J) {
      const int back = J - 1 - j;
      const int p = pos - back;
      if (p >= start) {
        const TI* src = proj + (row - back) * WP + c;
        for (int s0 = 0; s0 < nsplit; s0 += 4) {
          float v[4][4];
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (s0 + u < nsplit) ei::Vec4<TI>::load(src + (s0 + u) * split_stride, v[u]);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (s0 + u < nsplit) {
#pragma unroll
              for (int e = 0; e < 4; ++e) x[j][e] += v[u][e];
            }
        }
      } else if (p >= 0) {
        ei::Vec4<float>::load(tail + static_cast<size_t>(p - start + J - 1) * C + c, x[j]);
      }
    }
  }
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < kFewTaps; ++j)
    if (j < J) {
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += conv_w[static_cast<size_t>(c + e) * J + j] * x[j][e];
    }
#pragma unroll
  for (int e = 0; e < 4; ++e) acc[e] = silu_f32(acc[e]);
  ei::Vec4<float>::store(out + row * C + c, acc);
  if (new_tail_state) {
    float* to = new_tail_state + static_cast<size_t>(seq_out[seq]) * state_stride + tail_offset;
#pragma unroll
    for (int j = 1; j < kFewTaps; ++j)
      if (j < J) ei::Vec4<float>::store(to + static_cast<size_t>(j - 1) * C + c, x[j]);
  }
}

// A thread writes a sequence's new tail for its channel: the inputs of the last J - 1
// positions, from this step's rows or, where the step brought fewer, from the old tail (read
// before anything is written).
template <typename TI>
__global__ void delta_tail_kernel(const TI* __restrict__ proj, int nsplit, size_t split_stride,
                                  int WP, int J, float* __restrict__ state, size_t state_stride,
                                  size_t tail_offset, const int32_t* __restrict__ seq_in,
                                  const int32_t* __restrict__ seq_out,
                                  const int32_t* __restrict__ seq_count,
                                  const int32_t* __restrict__ seq_row0, int C) {
  const int seq = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int count = seq_count[seq];
  if (count <= 0 || c >= C) return;          // padding of a fixed-size batch
  const size_t row = static_cast<size_t>(seq_row0[seq]) + count - 1;     // the last row
  const float* tail = state + static_cast<size_t>(seq_in[seq]) * state_stride + tail_offset;
  float* to = state + static_cast<size_t>(seq_out[seq]) * state_stride + tail_offset;
  auto kept = [&](int i) {                    // what place i of the new tail holds
    const int back = J - 2 - i;               // the input `back` positions before the last row
    return back < count ? slice_sum(proj + (row - back) * WP + c, nsplit, split_stride)
                        : tail[static_cast<size_t>(i + count) * C + c];
  };
  if (J - 1 <= kFewTaps) {
    float keep[kFewTaps];
#pragma unroll
    for (int i = 0; i < kFewTaps; ++i) keep[i] = i < J - 1 ? kept(i) : 0.f;
#pragma unroll
    for (int i = 0; i < kFewTaps; ++i)
      if (i < J - 1) to[static_cast<size_t>(i) * C + c] = keep[i];
  } else {
    float keep[kMaxTaps - 1];
    for (int i = 0; i < J - 1; ++i) keep[i] = kept(i);
    for (int i = 0; i < J - 1; ++i) to[static_cast<size_t>(i) * C + c] = keep[i];
  }
}

// Sum over the L neighbouring lanes that share a column (L a power of two up to 32), every
// one of them getting it.  Steps inside a row of 16 lanes are DPP modifiers of the add.
template <int L>
__device__ __forceinline__ float group_sum(float v) {
  if (L >= 2)
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xb1, 0xf, 0xf, false));
  if (L >= 4)
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4e, 0xf, 0xf, false));
  if (L >= 8)
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));
  if (L >= 16)
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));
  if (L >= 32) {
    const ei::ei_u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r.x) + __uint_as_float(r.y);
  }
  return v;
}

// conv: [N, C] = q [G * D] | k [G * D] | v [H * DV] after convolution and silu.  The block
// (sequence, head, column block) walks the sequence's rows of this step in order.  A thread owns
// OWN (8 or 16) rows of one column of S, L neighbouring lanes share the column.  Per token, with S the
// state before the token, g its decay, k, q the unit key and the scaled unit query:
//   seen = g (S^T k)[col];  u = beta (v[col] - seen);  o[col] = g (S^T q)[col] + u (k . q);
//   S[., col] <- g S[., col] + k u
// (o = (g S + k u^T)^T q written out: both dot products are taken from the old S, so their
// sums over the lanes run side by side and the update is off the read-out's path).
template <typename TI, int L, int OWN>
__global__ void __launch_bounds__(kThreads)
delta_rule_kernel(const float* __restrict__ conv, int C, const TI* __restrict__ proj, int nsplit,
                  size_t split_stride, int WP, int beta_col, int decay_col,
                  const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                  float* __restrict__ state, size_t state_stride,
                  const int32_t* __restrict__ seq_in, const int32_t* __restrict__ seq_out,
                  const int32_t* __restrict__ seq_count,
                  const int32_t* __restrict__ seq_row0, float* __restrict__ o_raw, int H, int G,
                  int D, int DV, float q_scale, float unit_eps) {
  constexpr int DP = L * OWN;             // D rounded up to what the lanes of a column hold
  constexpr int CB = kThreads / L;        // columns of S a block holds
  constexpr int TILE = DP >= 256 ? kTile / 2 : kTile;   // (the widest keys: half, to fit 64 KB)
  constexpr int PIECES = OWN / 4;         // 16-byte pieces of a thread's rows
  __shared__ __attribute__((aligned(16))) float q_s[TILE][DP];
  __shared__ __attribute__((aligned(16))) float k_s[TILE][DP];
  __shared__ float v_s[TILE][CB];
  // per token: decay g, the factor kf that makes k a unit vector, beta kf, the factor qf of q
  // (unit vector times q_scale); and qf (k . q) of the raw vectors
  __shared__ __attribute__((aligned(16))) float4 coef_s[TILE];
  __shared__ float kq_s[TILE];
  __shared__ float beta_s[TILE], decay_s[TILE];

  const int seq = blockIdx.x;
  const int count = seq_count[seq];
  if (count <= 0) return;                 // padding of a fixed-size batch
  const int row0 = seq_row0[seq];
  const int head = blockIdx.y, shared_head = head / (H / G);
  const int tid = threadIdx.x;
  const int col_in_block = tid / L, part = tid % L;
  const int col = blockIdx.z * CB + col_in_block;
  const bool col_ok = col < DV;
  const int i0 = part * OWN;
  const int QK = G * D, VW = H * DV;

  const size_t in_row = (static_cast<size_t>(head) * DV + (col_ok ? col : 0)) * D + i0;
  const float* mine = state + static_cast<size_t>(seq_in[seq]) * state_stride + in_row;
  float* mine_out = state + static_cast<size_t>(seq_out[seq]) * state_stride + in_row;
  // (D a multiple of 4: the rows a thread owns are whole 16-byte pieces, inside S or outside)
  const bool wide = D % 4 == 0;
  float s[OWN];
#pragma unroll
  for (int m = 0; m < OWN; ++m) s[m] = 0.f;
  if (col_ok) {
    if (wide) {
#pragma unroll
      for (int pc = 0; pc < PIECES; ++pc)
        if (i0 + 4 * pc < D) {
          const float4 a = *reinterpret_cast<const float4*>(mine + 4 * pc);
          s[4 * pc] = a.x; s[4 * pc + 1] = a.y; s[4 * pc + 2] = a.z; s[4 * pc + 3] = a.w;
        }
    } else {
#pragma unroll
      for (int m = 0; m < OWN; ++m)
        if (i0 + m < D) s[m] = mine[m];
    }
  }
  const float rate = expf(a_log[head]), shift = dt_bias[head];

  // A tile's operands travel global memory -> registers -> LDS, and the registers are filled
  // for tile t + 1 while tile t is walked, so the walk does not wait for memory.  Rows of q, k
  // come as 16-byte pieces where the sizes allow (FAST), else element by element.
  constexpr int QUADS = DP / 4;                          // 16-byte pieces of a padded q or k row
  constexpr int NQ = (TILE * QUADS + kThreads - 1) / kThreads;   // pieces a thread moves per tile
  constexpr int NV = (TILE * CB + kThreads - 1) / kThreads;      // values a thread moves per tile
  const bool fast = D % 4 == 0 && C % 4 == 0;
  float4 fq[NQ], fk[NQ];
  float fv[NV], fb = 0.f, fa = 0.f;
  auto fetch = [&](int t0, int nt) __attribute__((always_inline)) {
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
      const int idx = tid + n * kThreads, tt = idx / QUADS, i = (idx % QUADS) * 4;
      fq[n] = fk[n] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (tt < nt && i < D) {
        const float* src = conv + static_cast<size_t>(row0 + t0 + tt) * C + shared_head * D + i;
        if (fast) {
          fq[n] = *reinterpret_cast<const float4*>(src);
          fk[n] = *reinterpret_cast<const float4*>(src + QK);
        } else {
          float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (i + e < D) {
              a[e] = src[e];
              b[e] = src[QK + e];
            }
          fq[n] = make_float4(a[0], a[1], a[2], a[3]);
          fk[n] = make_float4(b[0], b[1], b[2], b[3]);
        }
      }
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int idx = tid + n * kThreads, tt = idx / CB, cg = blockIdx.z * CB + idx % CB;
      fv[n] = (tt < nt && cg < DV)
                  ? conv[static_cast<size_t>(row0 + t0 + tt) * C + 2 * QK + head * DV + cg] : 0.f;
    }
    if (tid < nt) {
      const TI* src = proj + static_cast<size_t>(row0 + t0 + tid) * WP;
      fb = slice_sum(src + beta_col + head, nsplit, split_stride);
      fa = slice_sum(src + decay_col + head, nsplit, split_stride);
    }
  };
  auto commit = [&](int nt) __attribute__((always_inline)) {
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
      const int idx = tid + n * kThreads, tt = idx / QUADS, i = (idx % QUADS) * 4;
      if (tt < TILE) {
        *reinterpret_cast<float4*>(&q_s[tt][i]) = fq[n];
        *reinterpret_cast<float4*>(&k_s[tt][i]) = fk[n];
      }
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int idx = tid + n * kThreads;
      if (idx / CB < TILE) v_s[idx / CB][idx % CB] = fv[n];
    }
    if (tid < nt) {
      beta_s[tid] = 1.0f / (1.0f + expf(-fb));
      decay_s[tid] = expf(-rate * softplus_f32(fa + shift));
    }
  };

  fetch(0, min(TILE, count));
  for (int t0 = 0; t0 < count; t0 += TILE) {
    const int nt = min(TILE, count - t0);
    __syncthreads();                      // the last tile has been walked
    commit(nt);
    if (t0 + TILE < count) fetch(t0 + TILE, min(TILE, count - t0 - TILE));
    __syncthreads();
    {   // the factors that make q and k unit vectors, and k . q: 8 threads a token
      const int tt = tid / 8, sub = tid % 8;
      float q_sq = 0.f, k_sq = 0.f, kq = 0.f;
      if (tt < nt)
        for (int i = sub; i < D; i += 8) {
          q_sq += q_s[tt][i] * q_s[tt][i];
          k_sq += k_s[tt][i] * k_s[tt][i];
          kq += k_s[tt][i] * q_s[tt][i];
        }
      q_sq = group_sum<8>(q_sq);
      k_sq = group_sum<8>(k_sq);
      kq = group_sum<8>(kq);
      if (tt < nt && sub == 0) {
        const float kf = 1.0f / sqrtf(k_sq + unit_eps), qf = q_scale / sqrtf(q_sq + unit_eps);
        coef_s[tt] = make_float4(decay_s[tt], kf, beta_s[tt] * kf, qf);
        kq_s[tt] = kq * qf;
      }
    }
    __syncthreads();
    // the walk: what token tt + 1 needs is read from LDS while token tt is computed
    float4 kn[PIECES], qn[PIECES];
#pragma unroll
    for (int pc = 0; pc < PIECES; ++pc) {
      kn[pc] = *reinterpret_cast<const float4*>(&k_s[0][i0 + 4 * pc]);
      qn[pc] = *reinterpret_cast<const float4*>(&q_s[0][i0 + 4 * pc]);
    }
    float4 cf = coef_s[0];
    float vv = v_s[0][col_in_block], kqv = kq_s[0];
    for (int tt = 0; tt < nt; ++tt) {
      float kv[OWN], qv[OWN];
#pragma unroll
      for (int pc = 0; pc < PIECES; ++pc) {
        kv[4 * pc] = kn[pc].x; kv[4 * pc + 1] = kn[pc].y; kv[4 * pc + 2] = kn[pc].z; kv[4 * pc + 3] = kn[pc].w;
        qv[4 * pc] = qn[pc].x; qv[4 * pc + 1] = qn[pc].y; qv[4 * pc + 2] = qn[pc].z; qv[4 * pc + 3] = qn[pc].w;
      }
      const float g = cf.x, kf = cf.y, bk = cf.z, qf = cf.w, v_now = vv, kq_now = kqv;
      const int nx = tt + 1 < nt ? tt + 1 : tt;
#pragma unroll
      for (int pc = 0; pc < PIECES; ++pc) {
        kn[pc] = *reinterpret_cast<const float4*>(&k_s[nx][i0 + 4 * pc]);
        qn[pc] = *reinterpret_cast<const float4*>(&q_s[nx][i0 + 4 * pc]);
      }
      cf = coef_s[nx];
      vv = v_s[nx][col_in_block];
      kqv = kq_s[nx];
      float seen0 = 0.f, seen1 = 0.f, read0 = 0.f, read1 = 0.f;
#pragma unroll
      for (int m = 0; m < OWN; m += 2) {
        seen0 = fmaf(s[m], kv[m], seen0);
        seen1 = fmaf(s[m + 1], kv[m + 1], seen1);
        read0 = fmaf(s[m], qv[m], read0);
        read1 = fmaf(s[m + 1], qv[m + 1], read1);
      }
      const float seen = group_sum<L>(seen0 + seen1) * (g * kf);    // g (S^T k)[col], k a unit vector
      const float read = group_sum<L>(read0 + read1) * (g * qf);    // g (S^T q)[col]
      const float u = bk * (v_now - seen);                          // beta (v - seen), times k's factor
#pragma unroll
      for (int m = 0; m < OWN; ++m) s[m] = fmaf(s[m], g, kv[m] * u);
      if (part == 0 && col_ok)
        o_raw[static_cast<size_t>(row0 + t0 + tt) * VW + head * DV + col] = fmaf(u, kq_now, read);
    }
  }
  if (col_ok) {
    if (wide) {
#pragma unroll
      for (int pc = 0; pc < PIECES; ++pc)
        if (i0 + 4 * pc < D)
          *reinterpret_cast<float4*>(mine_out + 4 * pc) =
              make_float4(s[4 * pc], s[4 * pc + 1], s[4 * pc + 2], s[4 * pc + 3]);
    } else {
#pragma unroll
      for (int m = 0; m < OWN; ++m)
        if (i0 + m < D) mine_out[m] = s[m];
    }
  }
}

// A wave a (row, head), four heads a block: out = o / sqrt(mean(o^2) + eps) * w * silu(gate).
template <typename TI, typename TO>
__global__ void delta_out_kernel(const float* __restrict__ o_raw, const TI* __restrict__ proj,
                                 int nsplit, size_t split_stride, int WP, int gate_col,
                                 const float* __restrict__ norm_w, float eps,
                                 const int32_t* __restrict__ row_seq, TO* __restrict__ out,
                                 int H, int DV) {
  const size_t row = blockIdx.x;
  const int wave = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  const bool padding = row_seq[row] < 0;      // a defined input for the next product
  const int head = blockIdx.y * (kThreads / EI_WAVE) + wave;
  if (head < H) {
    const size_t base = (row * H + head) * DV;
    if (padding) {
      for (int j = lane; j < DV; j += EI_WAVE) out[base + j] = ei::from_f32<TO>(0.f);
      return;
    }
    const TI* gate = proj + row * WP + gate_col + static_cast<size_t>(head) * DV;
    float sq = 0.f;
    for (int j = lane; j < DV; j += EI_WAVE) sq += o_raw[base + j] * o_raw[base + j];
    sq = ei::wave_sum(sq);
    const float inv = 1.0f / sqrtf(sq / static_cast<float>(DV) + eps);
    for (int j = lane; j < DV; j += EI_WAVE) {
      const float gt = slice_sum(gate + j, nsplit, split_stride);
      out[base + j] = ei::from_f32<TO>((o_raw[base + j] * inv) * norm_w[j] * silu_f32(gt));
    }
  }
}

int lanes_a_column(int D, int own) {
  int lanes = 1;
  while (lanes * own < D) lanes *= 2;
  return lanes;
}

}  // namespace

extern "C" int ei_delta_conv(const void* proj, int in_dtype, int nsplit, long long split_stride,
                             int WP, const float* conv_w, int J, const float* state,
                             long long state_stride, long long tail_offset, const int32_t* row_pos,
                             const int32_t* row_seq, const int32_t* seq_in,
                             const int32_t* seq_out, const int32_t* seq_start, float* out, int N,
                             int C, int renew_tail, hipStream_t stream) {
  EI_REQUIRE(proj && conv_w && state && row_pos && row_seq && seq_in && seq_out && seq_start && out,
             "delta_conv: null pointer");
  EI_REQUIRE(!renew_tail || J <= kFewTaps, "delta_conv: the tails are renewed here for up to 8 taps");
  float* renewed = renew_tail ? const_cast<float*>(state) : nullptr;
  EI_REQUIRE(N > 0 && C > 0 && C <= WP && nsplit >= 1, "delta_conv: sizes must be positive");
  EI_REQUIRE(J >= 1 && J <= kMaxTaps, "delta_conv: taps must lie between 1 and 32");
  EI_REQUIRE((C + kThreads - 1) / kThreads <= 65535, "delta_conv: too many channels");
  const dim3 grid(N, (C + kThreads - 1) / kThreads);
  const size_t ss = static_cast<size_t>(split_stride);
  const bool vec = J <= kFewTaps && C % 4 == 0 && WP % 4 == 0 && ss % 4 == 0 &&
                   state_stride % 4 == 0 && tail_offset % 4 == 0 &&
                   (reinterpret_cast<uintptr_t>(proj) | reinterpret_cast<uintptr_t>(out) |
                    reinterpret_cast<uintptr_t>(state)) % 16 == 0;
  if (vec) {
    const int threads = 64;         // four channels a thread: 256 channels a block
    const dim3 vgrid(N, (C / 4 + threads - 1) / threads);
    if (in_dtype == EI_F32)
      delta_conv_vec_kernel<float><<<vgrid, threads, 0, stream>>>(
          static_cast<const float*>(proj), nsplit, ss, WP, conv_w, J, state,
          static_cast<size_t>(state_stride), static_cast<size_t>(tail_offset), row_pos, row_seq,
          seq_in, seq_out, seq_start, out, C, renewed);
    else if (in_dtype == EI_BF16)
      delta_conv_vec_kernel<bf16_t><<<vgrid, threads, 0, stream>>>(
          static_cast<const bf16_t*>(proj), nsplit, ss, WP, conv_w, J, state,
          static_cast<size_t>(state_stride), static_cast<size_t>(tail_offset), row_pos, row_seq,
          seq_in, seq_out, seq_start, out, C, renewed);
    else
      EI_REQUIRE(false, "delta_conv: unknown dtype");
    EI_LAUNCH_CHECK();
  }
  if (in_dtype == EI_F32)
    delta_conv_kernel<float><<<grid, kThreads, 0, stream>>>(
        static_cast<const float*>(proj), nsplit, ss, WP, conv_w, J, state,
        static_cast<size_t>(state_stride), static_cast<size_t>(tail_offset), row_pos, row_seq,
        seq_in, seq_out, seq_start, out, C, renewed);
  else if (in_dtype == EI_BF16)
    delta_conv_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(
        static_cast<const bf16_t*>(proj), nsplit, ss, WP, conv_w, J, state,
        static_cast<size_t>(state_stride), static_cast<size_t>(tail_offset), row_pos, row_seq,
        seq_in, seq_out, seq_start, out, C, renewed);
  else
    EI_REQUIRE(false, "delta_conv: unknown dtype");
  EI_LAUNCH_CHECK();
}

extern "C" int ei_delta_tail(const void* proj, int in_dtype, int nsplit, long long split_stride,
                             int WP, int J, float* state, long long state_stride,
                             long long tail_offset, const int32_t* seq_in,
                             const int32_t* seq_out, const int32_t* seq_count,
                             const int32_t* seq_row0, int n_seqs, int C, hipStream_t stream) {
  EI_REQUIRE(proj && state && seq_in && seq_out && seq_count && seq_row0, "delta_tail: null pointer");
  EI_REQUIRE(n_seqs > 0 && C > 0 && C <= WP && nsplit >= 1, "delta_tail: sizes must be positive");
  EI_REQUIRE(J >= 2 && J <= kMaxTaps, "delta_tail: taps must lie between 2 and 32");
  EI_REQUIRE((C + kThreads - 1) / kThreads <= 65535, "delta_tail: too many channels");
  const dim3 grid(n_seqs, (C + kThreads - 1) / kThreads);
  const size_t ss = static_cast<size_t>(split_stride);
  if (in_dtype == EI_F32)
    delta_tail_kernel<float><<<grid, kThreads, 0, stream>>>(
        static_cast<const float*>(proj), nsplit, ss, WP, J, state,
        static_cast<size_t>(state_stride), static_cast<size_t>(tail_offset), seq_in, seq_out,
        seq_count, seq_row0, C);
  else if (in_dtype == EI_BF16)
    delta_tail_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(
        static_cast<const bf16_t*>(proj), nsplit, ss, WP, J, state,
        static_cast<size_t>(state_stride), static_cast<size_t>(tail_offset), seq_in, seq_out,
        seq_count, seq_row0, C);
  else
    EI_REQUIRE(false, "delta_tail: unknown dtype");
  EI_LAUNCH_CHECK();
}

// conv [N, 2 G D + H DV] float32; proj as above with the beta and decay projections (H
// columns each) at beta_col and decay_col; o_raw [N, H DV] float32.  n_seqs blocks walk
// seq_count rows each from seq_row0.
extern "C" int ei_delta_rule(const float* conv, const void* proj, int in_dtype, int nsplit,
                             long long split_stride, int WP, int beta_col, int decay_col,
                             const float* a_log, const float* dt_bias, float* state,
                             long long state_stride, const int32_t* seq_in,
                             const int32_t* seq_out, const int32_t* seq_count,
                             const int32_t* seq_row0, float* o_raw,
                             int n_seqs, int H, int G, int D, int DV, float q_scale,
                             float unit_eps, hipStream_t stream) {
  EI_REQUIRE(conv && proj && a_log && dt_bias && state && seq_in && seq_out && seq_count && seq_row0 && o_raw,
             "delta_rule: null pointer");
  EI_REQUIRE(n_seqs > 0 && H > 0 && G > 0 && H % G == 0 && DV > 0, "delta_rule: bad head counts");
  EI_REQUIRE(D >= 1 && D <= 256, "delta_rule: the key size must lie between 1 and 256");
  EI_REQUIRE(beta_col >= 0 && decay_col >= 0 && beta_col + H <= WP && decay_col + H <= WP,
             "delta_rule: projection columns outside the row");
  // Rows of a column that a thread owns: 8 or 16.  What a token costs a wave beside its FMAs
  // (two sums over the lanes, operand reads, the read-out's store) does not grow with them, so
  // more rows mean fewer instructions in all; but a sequence and head then has fewer waves, so
  // 16 are taken only where that still leaves every SIMD of the chip two waves.  (32 rows, 256
  // registers and one wave a SIMD, measured slower: 2.9 against 2.5 ms for 64 prompts of 512
  // tokens, 67 against 60 us for a decode step of 64.)
  int own = 8;
  {
    const long long simds = 4ll * ei_compute_units();
    for (int wanted = 16; wanted > 8; wanted /= 2) {
      const int lanes = lanes_a_column(D, wanted);
      const long long waves = static_cast<long long>(n_seqs) * H *
                              ((static_cast<long long>(DV) * lanes + EI_WAVE - 1) / EI_WAVE);
      if (waves >= 2 * simds) {
        own = wanted;
        break;
      }
    }
  }
  const int L = lanes_a_column(D, own);
  const int CB = kThreads / L;
  const int C = 2 * G * D + H * DV;
  EI_REQUIRE(H <= 65535 && (DV + CB - 1) / CB <= 65535, "delta_rule: too many heads or columns");
  dim3 grid(n_seqs, H, (DV + CB - 1) / CB);
  const size_t ss = static_cast<size_t>(split_stride);
#define EI_DELTA(TI, LL, OO)                                                                    \
  delta_rule_kernel<TI, LL, OO><<<grid, kThreads, 0, stream>>>(                                 \
      conv, C, static_cast<const TI*>(proj), nsplit, ss, WP, beta_col, decay_col, a_log, dt_bias, \
      state, static_cast<size_t>(state_stride), seq_in, seq_out, seq_count, seq_row0, o_raw, H, \
      G, D,                                                                                     \
      DV, q_scale, unit_eps)
#define EI_DELTA_O(TI, LL)                         \
  do {                                             \
    if (own == 8) EI_DELTA(TI, LL, 8);             \
    else EI_DELTA(TI, LL, 16);                     \
  } while (0)
#define EI_DELTA_L(TI)                                                  \
  do {                                                                  \
    if (L == 1) EI_DELTA_O(TI, 1);                                      \
    else if (L == 2) EI_DELTA_O(TI, 2);                                 \
    else if (L == 4) EI_DELTA_O(TI, 4);                                 \
    else if (L == 8) EI_DELTA_O(TI, 8);                                 \
    else if (L == 16) EI_DELTA_O(TI, 16);                               \
    else EI_DELTA(TI, 32, 8);                                           \
  } while (0)
  if (in_dtype == EI_F32) EI_DELTA_L(float);
  else if (in_dtype == EI_BF16) EI_DELTA_L(bf16_t);
  else EI_REQUIRE(false, "delta_rule: unknown dtype");
#undef EI_DELTA_O
#undef EI_DELTA_L
#undef EI_DELTA
  EI_LAUNCH_CHECK();
}

extern "C" int ei_delta_out(const float* o_raw, const void* proj, int in_dtype, int nsplit,
                            long long split_stride, int WP, int gate_col, const float* norm_w,
                            float eps, const int32_t* row_seq, void* out, int out_dtype, int N,
                            int H, int DV, hipStream_t stream) {
  EI_REQUIRE(o_raw && proj && norm_w && row_seq && out, "delta_out: null pointer");
  EI_REQUIRE(N > 0 && H > 0 && DV > 0 && nsplit >= 1, "delta_out: sizes must be positive");
  EI_REQUIRE(gate_col >= 0 && gate_col + H * DV <= WP, "delta_out: gate columns outside the row");
  EI_REQUIRE(eps > 0.f, "delta_out: eps must be positive");
  EI_REQUIRE((H + 3) / 4 <= 65535, "delta_out: too many heads");
  const size_t ss = static_cast<size_t>(split_stride);
#define EI_DOUT(TI, TO)                                                                      \
  delta_out_kernel<TI, TO><<<dim3(N, (H + 3) / 4), kThreads, 0, stream>>>(                   \
      o_raw, static_cast<const TI*>(proj), nsplit, ss, WP, gate_col, norm_w, eps, row_seq,   \
      static_cast<TO*>(out), H, DV)
  if (in_dtype == EI_F32 && out_dtype == EI_F32) EI_DOUT(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16) EI_DOUT(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16) EI_DOUT(bf16_t, bf16_t);
  else EI_REQUIRE(false, "delta_out: unsupported dtype combination");
#undef EI_DOUT
  EI_LAUNCH_CHECK();
}

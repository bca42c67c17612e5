// Sequence mixers beside the softmax paged attention: a sliding-window attention whose weights are
// sigmoid(score + bias) (not normalised over keys), and the gated delta rule, a linear recurrence
// with a matrix state per head, with its short causal convolution.  All of them run over a packed
// batch of chunks (whole prompts, portions of prompts, single decoded tokens side by side):
//   tok_seq[t]     which chunk packed row t belongs to
//   positions[t]   its position in its sequence
//   cu_seqlens[s]  first packed row of chunk s (cu_seqlens[S] = number of rows)
// K/V live in the engine's 16-token pages (block tables); recurrent and convolution state live in
// per-sequence slots.  Scores, weights, decays and state are fp32; K/V pages and activations are
// stored in the dtype argument's type.
//
//   rope_partial_kv_write   rotate the first rot_dims coordinates of q and k (pairs i, i + rot_dims/2)
//                           by fp32 table angles, store k and v into their pages
//   sigmoid_window_attn     out[t,h] = gate * sum_{j : 0 <= p - j < window} sigmoid(q.k_j * scale * temp[h] + bias[h]) v_j
//   causal_conv_silu        y[t,c] = silu(sum_j w[c,j] x[t - (taps-1-j), c]), inputs before the chunk from the state
//   conv_state_update       state <- the last taps-1 inputs of each sequence
//   gated_delta_rule        S <- a S; u = b (v - S^T k); S <- S + k u^T; o = S^T q   per token and head
//   general_delta_rule      S <- diag(w) S - (a * u) (u^T S) + k v^T; o = S^T r      per token and head
//   mingru_scan             S <- (1 - z) S + z c per channel, z = sigmoid(zp + bz), c = u + 1/2 (u >= 0) or sigmoid(u),
//                           u = xp + bx; out = S * silu(gp)
#include "common.h"

namespace mi355 {

constexpr int kPage = MI355_BLOCK_SIZE;

// one workgroup per packed row; threads walk the (head, pair / coordinate) space
template <typename T>
__global__ __launch_bounds__(256) void rope_partial_kv_write_kernel(
    typename Elem<T>::S* __restrict__ q, int64_t q_stride, const typename Elem<T>::S* __restrict__ k, int64_t k_stride,
    const typename Elem<T>::S* __restrict__ v, int64_t v_stride, const float* __restrict__ cos_sin, int max_pos,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ slot_mapping,
    typename Elem<T>::S* __restrict__ k_cache, typename Elem<T>::S* __restrict__ v_cache, int H, int G, int d, int dv,
    int rot) {
  const int64_t t = blockIdx.x;
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
  const int64_t slot = MI355_LD(int64_t, slot_mapping, slot_mapping + t);
  const int half = rot >> 1;
  const float* cs = cos_sin + p * rot;                 // cos[0..half) | sin[0..half)
  // queries: rotate in place (pairs only; the coordinates past rot stay as they are)
  for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
    const int h = i / half, j = i % half;
    typename Elem<T>::S* row = q + t * q_stride + static_cast<int64_t>(h) * d;
    const float c = MI355_LD(float, cos_sin, cs + j), s = MI355_LD(float, cos_sin, cs + half + j);
    const float a = MI355_LDF(T, q, row + j), b = MI355_LDF(T, q, row + half + j);
    MI355_STF(T, q, row + j, a * c - b * s);
    MI355_STF(T, q, row + half + j, b * c + a * s);
  }
  if (slot < 0 || k == nullptr) return;                 // k null: a layer that reads another layer's pages
  const int64_t page = slot / kPage, off = slot % kPage;
  for (int i = threadIdx.x; i < G * d; i += blockDim.x) {
    const int g = i / d, j = i % d;
    const typename Elem<T>::S* row = k + t * k_stride + static_cast<int64_t>(g) * d;
    float val;
    if (j < half) {
      const float c = MI355_LD(float, cos_sin, cs + j), s = MI355_LD(float, cos_sin, cs + half + j);
      val = MI355_LDF(T, k, row + j) * c - MI355_LDF(T, k, row + half + j) * s;
    } else if (j < rot) {
      const int jj = j - half;
      const float c = MI355_LD(float, cos_sin, cs + jj), s = MI355_LD(float, cos_sin, cs + half + jj);
      val = MI355_LDF(T, k, row + j) * c + MI355_LDF(T, k, row + jj) * s;
    } else {
      val = MI355_LDF(T, k, row + j);
    }
    MI355_STF(T, k_cache, k_cache + ((page * G + g) * kPage + off) * d + j, val);
  }
  for (int i = threadIdx.x; i < G * dv; i += blockDim.x) {
    const int g = i / dv, j = i % dv;
    MI355_ST(typename Elem<T>::S, v_cache, v_cache + ((page * G + g) * dv + j) * kPage + off,
             MI355_LD(typename Elem<T>::S, v, v + t * v_stride + static_cast<int64_t>(g) * dv + j));
  }
}

// One wave per (packed row, query head).  Keys are taken 64 at a time: every lane scores one key
// (a dot product over its page row), the 64 weights go through LDS, then every lane accumulates
// its value channels over the 64 keys.  Serves portions of prompts and decoded tokens alike.
template <typename T, int DV_PER_LANE>
__global__ __launch_bounds__(64) void sigmoid_window_attn_kernel(
    typename Elem<T>::S* __restrict__ out, const typename Elem<T>::S* __restrict__ q, int64_t q_stride,
    const typename Elem<T>::S* __restrict__ k_cache, const typename Elem<T>::S* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ tok_seq,
    const int64_t* __restrict__ positions, const float* __restrict__ temp, const float* __restrict__ bias,
    const typename Elem<T>::S* __restrict__ gate, int64_t gate_stride, int H, int G, int d, int dv, int window,
    float scale) {
  extern __shared__ float lds[];                        // q [d] | w [64]
  float* qs = lds;
  float* ws = lds + d;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, g = h / (H / G), lane = threadIdx.x;
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  if (p >= static_cast<int64_t>(max_blocks) * kPage) p = static_cast<int64_t>(max_blocks) * kPage - 1;   // never past the table
  const int32_t* bt = block_tables + static_cast<int64_t>(MI355_LD(int32_t, tok_seq, tok_seq + t)) * max_blocks;
  for (int i = lane; i < d; i += 64) qs[i] = MI355_LDF(T, q, q + t * q_stride + static_cast<int64_t>(h) * d + i);
  const float mul = scale * MI355_LD(float, temp, temp + h), add = MI355_LD(float, bias, bias + h);
  float acc[DV_PER_LANE];
#pragma unroll
  for (int i = 0; i < DV_PER_LANE; ++i) acc[i] = 0.f;
  int64_t lo = p - window + 1;
  if (lo < 0) lo = 0;
  __syncthreads();
  for (int64_t base = lo; base <= p; base += 64) {
    const int64_t j = base + lane;
    float w = 0.f;
    if (j <= p) {
      const int64_t page = MI355_LD(int32_t, block_tables, bt + j / kPage);
      const typename Elem<T>::S* kr = k_cache + ((page * G + g) * kPage + j % kPage) * d;
      float s = 0.f;
      for (int i = 0; i < d; ++i) s += qs[i] * MI355_LDF(T, k_cache, kr + i);
      w = 1.0f / (1.0f + expf(-(s * mul + add)));
    }
    ws[lane] = w;
    __syncthreads();
    const int n = static_cast<int>((p - base + 1) < 64 ? (p - base + 1) : 64);
    for (int jj = 0; jj < n; ++jj) {
      const int64_t key = base + jj;
      const int64_t page = MI355_LD(int32_t, block_tables, bt + key / kPage);
      const typename Elem<T>::S* vr = v_cache + (page * G + g) * dv * kPage + key % kPage;
      const float wj = ws[jj];
#pragma unroll
      for (int i = 0; i < DV_PER_LANE; ++i) {
        const int c = lane + 64 * i;
        if (c < dv) acc[i] += wj * MI355_LDF(T, v_cache, vr + c * kPage);
      }
    }
    __syncthreads();
  }
  float gt = 1.0f;
  if (gate != nullptr) gt = 1.0f / (1.0f + expf(-MI355_LDF(T, gate, gate + t * gate_stride + h)));
#pragma unroll
  for (int i = 0; i < DV_PER_LANE; ++i) {
    const int c = lane + 64 * i;
    if (c < dv) MI355_STF(T, out, out + (t * H + h) * dv + c, acc[i] * gt);
  }
}

// The matrix-core form for 16-bit activations, d a multiple of 32, dv a multiple of 16.  One wave
// per (tile of up to 16 consecutive rows of one chunk, block of HB query heads of one kv head): the
// K and V fragments it loads serve all HB heads, whose query fragments and accumulators stay in
// registers (a wave per head would pull the same pages through the cache HB times).  Keys are
// taken 32 at a time (two pages).  Scores are computed transposed, S^T = K Q^T, so that a lane ends
// up holding, for its query (lane % 16), eight weights -- keys 4 (lane / 16) + r of either page --
// which is exactly an A-operand fragment of the P V product once V's fragment lists the same
// eight keys: with V pages stored [dv, 16 tokens] that is two 8-byte loads.  Scores, the sigmoid
// and the accumulators are fp32; the weights are rounded to the storage type for the second product.
// gridDim.z > 1: the key tiles are dealt out to the z blocks in turn and each writes its fp32 sums
// (no gate) to its slab of `partial`; the weights are not normalised, so the slabs simply add up.
template <typename T, int HB, int DS, int CB>
__global__ __launch_bounds__(256) void sigmoid_window_attn_mfma_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q, int64_t q_stride, const uint16_t* __restrict__ k_cache,
    const uint16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tiles, int num_tiles, const int64_t* __restrict__ positions,
    const float* __restrict__ temp, const float* __restrict__ bias, const uint16_t* __restrict__ gate,
    int64_t gate_stride, int H, int G, int d, int dv, int window, float scale, float* __restrict__ partial,
    int64_t partial_stride) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tile = blockIdx.x * (blockDim.x >> 6) + wave;
  if (tile >= num_tiles) return;                        // (no workgroup barrier below)
  const int rep = H / G, hbs = rep / HB;
  const int g = blockIdx.y / hbs, h0 = g * rep + (blockIdx.y % hbs) * HB;
  const int nz = gridDim.z, z = blockIdx.z;
  const int li = lane & 15, kk = lane >> 4;
  const int seq = MI355_LD(int32_t, tiles, tiles + 3 * tile);
  const int64_t row0 = MI355_LD(int32_t, tiles, tiles + 3 * tile + 1);
  const int nrows = MI355_LD(int32_t, tiles, tiles + 3 * tile + 2);
  const int64_t p0 = MI355_LD(int64_t, positions, positions + row0);
  const int32_t* bt = block_tables + static_cast<int64_t>(seq) * max_blocks;
  const int ds = d >> 5, cbs = dv >> 4;
  const int64_t p_last = p0 + nrows - 1;
  int64_t lo = p0 - window + 1;
  if (lo < 0) lo = 0;
  const int64_t my_p = p0 + li;                         // position of this lane's query (rows past nrows: masked out)
  uint4 qf[HB][DS];
  float mul[HB], add[HB];
  f32x4 acc[HB][CB];
#pragma unroll
  for (int i = 0; i < HB; ++i) {
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      qf[i][s] = make_uint4(0, 0, 0, 0);
      if (s < ds && li < nrows)
        qf[i][s] = MI355_LD(uint4, q, q + (row0 + li) * q_stride + static_cast<int64_t>(h0 + i) * d + 32 * s + 8 * kk);
    }
    mul[i] = -1.4426950408889634f * scale * MI355_LD(float, temp, temp + h0 + i);
    add[i] = -1.4426950408889634f * MI355_LD(float, bias, bias + h0 + i);
#pragma unroll
    for (int c = 0; c < CB; ++c) acc[i][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  for (int64_t base = ((lo >> 5) << 5) + 32 * z; base <= p_last; base += 32 * nz) {
    // every load of the tile is issued before the first product: one trip to memory per tile, not
    // one per fragment
    uint4 kf[2][DS];
    uint2 vf[2][CB];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int64_t kb = base + 16 * half;
      const bool have = kb <= p_last;
      const int64_t page = have ? MI355_LD(int32_t, block_tables, bt + kb / kPage) : 0;
      const uint16_t* kr = k_cache + ((page * G + g) * kPage + li) * d + 8 * kk;
      const uint16_t* vr = v_cache + ((page * G + g) * dv + li) * kPage + 4 * kk;
#pragma unroll
      for (int s = 0; s < DS; ++s)
        kf[half][s] = (have && s < ds) ? MI355_LD(uint4, k_cache, kr + 32 * s) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int c = 0; c < CB; ++c)
        vf[half][c] = (have && c < cbs) ? MI355_LD(uint2, v_cache, vr + 16 * c * kPage) : make_uint2(0, 0);
    }
    uint32_t pw[HB][4];                                 // 8 weights of this lane's query per head, packed
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int64_t kb = base + 16 * half;
      bool vis[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int64_t key = kb + 4 * kk + r;
        vis[r] = li < nrows && key <= my_p && my_p - key < window;
      }
#pragma unroll
      for (int i = 0; i < HB; ++i) {
        f32x4 sacc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < DS; ++s)
          if (s < ds) sacc = T::mfma(kf[half][s], qf[i][s], sacc);
        float w[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)                       // sigmoid(x) = 1 / (1 + 2^(-x log2 e))
          w[r] = vis[r] ? __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sacc[r] * mul[i] + add[i])) : 0.f;
        pw[i][2 * half] = T::pack2(w[0], w[1]);
        pw[i][2 * half + 1] = T::pack2(w[2], w[3]);
      }
    }
    if (base + 31 > p_last) {
      // slots past the newest key may hold anything (0 * NaN is NaN): clear them in the last tile
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int64_t k0 = base + 16 * half + 4 * kk;
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          if (k0 > p_last) vf[half][c].x &= 0xFFFF0000u;
          if (k0 + 1 > p_last) vf[half][c].x &= 0x0000FFFFu;
          if (k0 + 2 > p_last) vf[half][c].y &= 0xFFFF0000u;
          if (k0 + 3 > p_last) vf[half][c].y &= 0x0000FFFFu;
        }
      }
    }
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      if (c < cbs) {
        const uint4 v4 = make_uint4(vf[0][c].x, vf[0][c].y, vf[1][c].x, vf[1][c].y);
#pragma unroll
        for (int i = 0; i < HB; ++i)
          acc[i][c] = T::mfma(make_uint4(pw[i][0], pw[i][1], pw[i][2], pw[i][3]), v4, acc[i][c]);
      }
    }
  }
  // C layout: this lane holds rows 4 kk + r of column li of every 16-column block
#pragma unroll
  for (int i = 0; i < HB; ++i) {
    const int h = h0 + i;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int rr = 4 * kk + r;
      if (rr >= nrows) continue;
      if (partial != nullptr) {
#pragma unroll
        for (int c = 0; c < CB; ++c)
          if (c < cbs) MI355_ST(float, partial, partial + z * partial_stride + ((row0 + rr) * H + h) * dv + 16 * c + li, acc[i][c][r]);
        continue;
      }
      float gt = 1.0f;
      if (gate != nullptr) gt = 1.0f / (1.0f + expf(-T::to_f(MI355_LD(uint16_t, gate, gate + (row0 + rr) * gate_stride + h))));
#pragma unroll
      for (int c = 0; c < CB; ++c)
        if (c < cbs) MI355_ST(uint16_t, out, out + ((row0 + rr) * H + h) * dv + 16 * c + li, T::from_f(acc[i][c][r] * gt));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    typename Elem<T>::S* __restrict__ y, const typename Elem<T>::S* __restrict__ x, int64_t x_stride,
    const typename Elem<T>::S* __restrict__ w, const float* __restrict__ state, const int32_t* __restrict__ tok_seq,
    const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_seqlens,
    const int32_t* __restrict__ state_slots, int C, int taps) {
  const int64_t t = blockIdx.x;
  const int s = MI355_LD(int32_t, tok_seq, tok_seq + t);
  const int64_t cs = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s);
  const int64_t p = MI355_LD(int64_t, positions, positions + t);
  const int64_t slot = MI355_LD(int32_t, state_slots, state_slots + s);
  const float* st = state + slot * (taps - 1) * C;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      if (p - back < 0) continue;                       // zeros before the start of the sequence
      const int64_t src = t - back;
      float xv;
      if (src >= cs) xv = MI355_LDF(T, x, x + src * x_stride + c);
      else xv = MI355_LD(float, state, st + (src - cs + taps - 1) * C + c);
      acc += MI355_LDF(T, w, w + static_cast<int64_t>(c) * taps + j) * xv;
    }
    MI355_STF(T, y, y + t * C + c, acc / (1.0f + expf(-acc)));
  }
}

// 16-bit rows, 8 channels per thread, the taps a template constant
template <typename T, int TAPS>
__global__ __launch_bounds__(256) void causal_conv_silu_vec_kernel(
    uint16_t* __restrict__ y, const uint16_t* __restrict__ x, int64_t x_stride, const uint16_t* __restrict__ w,
    const float* __restrict__ state, const int32_t* __restrict__ tok_seq, const int64_t* __restrict__ positions,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, int64_t num_tokens, int C) {
  const int vec_per_row = C >> 3;
  const int64_t total = num_tokens * vec_per_row;
  for (int64_t idx = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; idx < total;
       idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = idx / vec_per_row;
    const int c8 = static_cast<int>(idx % vec_per_row) * 8;
    const int s = MI355_LD(int32_t, tok_seq, tok_seq + t);
    const int64_t cs = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s);
    const int64_t p = MI355_LD(int64_t, positions, positions + t);
    const float* st = state + static_cast<int64_t>(MI355_LD(int32_t, state_slots, state_slots + s)) * (TAPS - 1) * C;
    float wv[TAPS][8];                                  // weights of the 8 channels: 8 * TAPS contiguous values
#pragma unroll
    for (int j = 0; j < TAPS; ++j) unpack8<T>(MI355_LD(uint4, w, w + static_cast<int64_t>(c8) * TAPS + 8 * j), wv[j]);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
      const int back = TAPS - 1 - j;
      if (p - back < 0) continue;
      const int64_t src = t - back;
      float xv[8];
      if (src >= cs) {
        unpack8<T>(MI355_LD(uint4, x, x + src * x_stride + c8), xv);
      } else {
        const float* sr = st + (src - cs + TAPS - 1) * C + c8;
        const float4 a = MI355_LD(float4, state, sr), b = MI355_LD(float4, state, sr + 4);
        xv[0] = a.x, xv[1] = a.y, xv[2] = a.z, xv[3] = a.w, xv[4] = b.x, xv[5] = b.y, xv[6] = b.z, xv[7] = b.w;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += (&wv[0][0])[i * TAPS + j] * xv[i];
    }
    float o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = acc[i] / (1.0f + expf(-acc[i]));
    MI355_ST(uint4, y, y + t * C + c8, pack8<T>(o));
  }
}

constexpr int kMaxTaps = 16;

template <typename T>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    float* __restrict__ state, const typename Elem<T>::S* __restrict__ x, int64_t x_stride,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, int C, int taps) {
  const int s = blockIdx.x;
  const int64_t cs = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s);
  const int64_t n = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s + 1) - cs;
  if (n <= 0) return;
  const int64_t slot = MI355_LD(int32_t, state_slots, state_slots + s);
  float* st = state + slot * (taps - 1) * C;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float nv[kMaxTaps];
#pragma unroll
    for (int m = 0; m < kMaxTaps; ++m) {
      if (m < taps - 1) {
        const int64_t idx = n - (taps - 1) + m;         // row of the chunk, or (negative) before it
        nv[m] = idx >= 0 ? MI355_LDF(T, x, x + (cs + idx) * x_stride + c)
                         : MI355_LD(float, state, st + (idx + taps - 1) * C + c);
      }
    }
#pragma unroll
    for (int m = 0; m < kMaxTaps; ++m)
      if (m < taps - 1) MI355_ST(float, state, st + static_cast<int64_t>(m) * C + c, nv[m]);
  }
}

// One wave per (chunk, head, 64 value channels).  Lane j owns column j of the head's state matrix
// S [d, dv] in registers (D >= d rows, the rest zero) and walks the chunk's tokens in order.  Per
// token the wave first prepares, in LDS, the unit-length key, the unit-length scaled query and the
// decay (per head, or per key channel), all fp32; then every lane runs the recurrence on its column.
template <typename T, int D>
__global__ __launch_bounds__(64) void gated_delta_rule_kernel(
    float* __restrict__ o, const typename Elem<T>::S* __restrict__ qkv, int64_t stride, int q_off, int k_off, int v_off,
    const typename Elem<T>::S* __restrict__ beta, int64_t beta_stride, const typename Elem<T>::S* __restrict__ decay,
    int64_t decay_stride, const float* __restrict__ a_log, const float* __restrict__ dt_bias, int per_channel,
    float* __restrict__ state, const int32_t* __restrict__ cu_seqlens, const int64_t* __restrict__ positions,
    const int32_t* __restrict__ state_slots, int H, int G, int d, int dv) {
  __shared__ float ks[D], qs[D], as[D];
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int col = blockIdx.z * 64 + lane;
  const int g = h / (H / G);
  const int64_t cs = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s);
  const int64_t n = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s + 1) - cs;
  if (n <= 0) return;
  const int64_t slot = MI355_LD(int32_t, state_slots, state_slots + s);
  float* sp = state + ((slot * H + h) * d) * dv;
  const bool live = col < dv;
  const bool fresh = MI355_LD(int64_t, positions, positions + cs) == 0;
  float S[D];
#pragma unroll
  for (int i = 0; i < D; ++i) S[i] = (live && !fresh && i < d) ? MI355_LD(float, state, sp + static_cast<int64_t>(i) * dv + col) : 0.f;
  const float na = -expf(MI355_LD(float, a_log, a_log + h));
  const float qscale = 1.0f / sqrtf(static_cast<float>(d));
  for (int64_t r = 0; r < n; ++r) {
    const int64_t t = cs + r;
    const typename Elem<T>::S* row = qkv + t * stride;
    // ---- per-token vectors, fp32 (the lanes share the work; D <= 4 * 64)
    float kv[(D + 63) / 64], qv[(D + 63) / 64], kk = 0.f, qq = 0.f;
#pragma unroll
    for (int i = 0; i < (D + 63) / 64; ++i) {
      const int c = lane + 64 * i;
      kv[i] = c < d ? MI355_LDF(T, qkv, row + k_off + g * d + c) : 0.f;
      qv[i] = c < d ? MI355_LDF(T, qkv, row + q_off + g * d + c) : 0.f;
      kk += kv[i] * kv[i];
      qq += qv[i] * qv[i];
    }
    kk = 1.0f / sqrtf(wave_sum(kk) + 1e-6f);
    qq = qscale / sqrtf(wave_sum(qq) + 1e-6f);
    __syncthreads();                                  // the previous token's reads of ks / qs / as are done
#pragma unroll
    for (int i = 0; i < (D + 63) / 64; ++i) {
      const int c = lane + 64 * i;
      if (c < D) {
        ks[c] = kv[i] * kk;
        qs[c] = qv[i] * qq;
        float a = 1.0f;
        if (c < d) {
          const float z = per_channel
                              ? MI355_LDF(T, decay, decay + t * decay_stride + h * d + c) + MI355_LD(float, dt_bias, dt_bias + h * d + c)
                              : MI355_LDF(T, decay, decay + t * decay_stride + h) + MI355_LD(float, dt_bias, dt_bias + h);
          const float sp_ = z > 20.0f ? z : log1pf(expf(z));
          a = expf(na * sp_);
        }
        as[c] = a;
      }
    }
    const float b = 1.0f / (1.0f + expf(-MI355_LDF(T, beta, beta + t * beta_stride + h)));
    const float vj = live ? MI355_LDF(T, qkv, row + v_off + h * dv + col) : 0.f;
    __syncthreads();
    // ---- the recurrence on this lane's column
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < D; ++i) {
      S[i] *= as[i];
      dot += S[i] * ks[i];
    }
    const float u = b * (vj - dot);
    float out = 0.f;
#pragma unroll
    for (int i = 0; i < D; ++i) {
      S[i] += ks[i] * u;
      out += S[i] * qs[i];
    }
    if (live) MI355_ST(float, o, o + (t * H + h) * dv + col, out);
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < D; ++i)
      if (i < d) MI355_ST(float, state, sp + static_cast<int64_t>(i) * dv + col, S[i]);
  }
}

// ---- the gated delta rule for chunks of many tokens -------------------------------------------------
// With one state column per lane a token costs 4 * d dependent vector operations per wave and a
// prompt keeps only heads * dv / 64 waves busy.  Here the d rows of a column are split over R = 16
// (or 8) adjacent lanes (a wave holds 64 / R columns, DR = ceil(d / R) rows each), the two dot products
// of a token are finished with four (three) cross-lane steps each, and everything that does not depend on the
// state -- unit-length key and query, decay, beta -- is computed for all tokens at once by
// delta_prep_kernel, in fp32, into rows padded to R * DR (key / query 0, decay 1 in the padding).
// The loop then reads the next token's rows while it works on the current one.

// sum over the 8 adjacent lanes of a group, in every lane of it, by data-parallel-primitive moves
// (no trip through the LDS crossbar): swap within pairs, swap pairs within quads, mirror the half row
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int R>
__device__ __forceinline__ float sum_lanes(float v) {
  v += dpp_move<0xB1>(v);       // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);       // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x141>(v);      // row_half_mirror: lane i of 8 takes lane 7 - i
  if (R == 16) v += dpp_move<0x128>(v);   // row_ror 8: the other half of the 16-lane row
  return v;
}

template <typename T>
__global__ __launch_bounds__(64) void delta_prep_kernel(
    float* __restrict__ kq, float* __restrict__ dec, float* __restrict__ bet, const typename Elem<T>::S* __restrict__ qkv,
    int64_t stride, int q_off, int k_off, const typename Elem<T>::S* __restrict__ beta, int64_t beta_stride,
    const typename Elem<T>::S* __restrict__ decay, int64_t decay_stride, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, int per_channel, int H, int G, int d, int dp) {
  const int64_t t = blockIdx.x;
  const int y = blockIdx.y, lane = threadIdx.x;
  if (y < G) {                                          // unit-length key and scaled unit-length query of kv head y
    const typename Elem<T>::S* row = qkv + t * stride;
    float kk = 0.f, qq = 0.f;
    for (int c = lane; c < d; c += 64) {
      const float kv = MI355_LDF(T, qkv, row + k_off + y * d + c), qv = MI355_LDF(T, qkv, row + q_off + y * d + c);
      kk += kv * kv;
      qq += qv * qv;
    }
    kk = 1.0f / sqrtf(wave_sum(kk) + 1e-6f);
    qq = (1.0f / sqrtf(static_cast<float>(d))) / sqrtf(wave_sum(qq) + 1e-6f);
    float* o = kq + (t * G + y) * 2 * dp;
    for (int c = lane; c < dp; c += 64) {
      MI355_ST(float, kq, o + c, c < d ? MI355_LDF(T, qkv, row + k_off + y * d + c) * kk : 0.f);
      MI355_ST(float, kq, o + dp + c, c < d ? MI355_LDF(T, qkv, row + q_off + y * d + c) * qq : 0.f);
    }
    return;
  }
  const int h = y - G;
  const float na = -expf(MI355_LD(float, a_log, a_log + h));
  float* o = dec + (t * H + h) * dp;
  for (int c = lane; c < dp; c += 64) {
    float a = 1.0f;
    if (c < d) {
      const float z = per_channel
                          ? MI355_LDF(T, decay, decay + t * decay_stride + h * d + c) + MI355_LD(float, dt_bias, dt_bias + h * d + c)
                          : MI355_LDF(T, decay, decay + t * decay_stride + h) + MI355_LD(float, dt_bias, dt_bias + h);
      a = expf(na * (z > 20.0f ? z : log1pf(expf(z))));
    }
    MI355_ST(float, dec, o + c, a);
  }
  if (lane == 0)
    MI355_ST(float, bet, bet + t * H + h, 1.0f / (1.0f + expf(-MI355_LDF(T, beta, beta + t * beta_stride + h))));
}

template <typename T, int R, int DR, int PF>
__global__ __launch_bounds__(64) void gated_delta_rule_split_kernel(
    float* __restrict__ o, const typename Elem<T>::S* __restrict__ qkv, int64_t stride, int v_off,
    const float* __restrict__ kq, const float* __restrict__ dec, const float* __restrict__ bet, float* __restrict__ state,
    const int32_t* __restrict__ cu_seqlens, const int64_t* __restrict__ positions,
    const int32_t* __restrict__ state_slots, int H, int G, int d, int dv) {
  constexpr int dp = R * DR;
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = lane & (R - 1), col = blockIdx.z * (64 / R) + lane / R;
  const int g = h / (H / G);
  const int64_t cs = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s);
  const int64_t n = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s + 1) - cs;
  if (n <= 0) return;
  const int64_t slot = MI355_LD(int32_t, state_slots, state_slots + s);
  float* sp = state + ((slot * H + h) * d) * dv;
  const bool live = col < dv;
  const bool fresh = MI355_LD(int64_t, positions, positions + cs) == 0;
  float S[DR];
#pragma unroll
  for (int j = 0; j < DR; ++j) {
    const int i = r * DR + j;
    S[j] = (live && !fresh && i < d) ? MI355_LD(float, state, sp + static_cast<int64_t>(i) * dv + col) : 0.f;
  }
  // Two register sets of PF tokens each: while one is worked on, the rows of the PF tokens after
  // it travel into the other (a token's arithmetic is far shorter than a trip to memory).
  struct Rows {
    float k[PF][DR], q[PF][DR], a[PF][DR], b[PF], v[PF];
  };
  Rows A, B;
  auto fetch = [&](Rows& w, int64_t first) {
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      int64_t t = first + u;
      if (t > cs + n - 1) t = cs + n - 1;               // past the chunk: a row that is loaded and not used
      const float* kp = kq + (t * G + g) * 2 * dp + r * DR;
      const float* ap = dec + (t * H + h) * dp + r * DR;
#pragma unroll
      for (int j = 0; j < DR; j += 4) {
        const float4 a4 = MI355_LD(float4, kq, kp + j), b4 = MI355_LD(float4, kq, kp + dp + j), c4 = MI355_LD(float4, dec, ap + j);
        w.k[u][j] = a4.x, w.k[u][j + 1] = a4.y, w.k[u][j + 2] = a4.z, w.k[u][j + 3] = a4.w;
        w.q[u][j] = b4.x, w.q[u][j + 1] = b4.y, w.q[u][j + 2] = b4.z, w.q[u][j + 3] = b4.w;
        w.a[u][j] = c4.x, w.a[u][j + 1] = c4.y, w.a[u][j + 2] = c4.z, w.a[u][j + 3] = c4.w;
      }
      w.b[u] = MI355_LD(float, bet, bet + t * H + h);
      w.v[u] = live ? MI355_LDF(T, qkv, qkv + t * stride + v_off + h * dv + col) : 0.f;
    }
  };
  auto work = [&](const Rows& w, int64_t i0) {
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      if (i0 + u >= n) break;
      float d0 = 0.f, d1 = 0.f;
#pragma unroll
      for (int j = 0; j < DR; j += 2) {
        S[j] *= w.a[u][j];
        S[j + 1] *= w.a[u][j + 1];
        d0 += S[j] * w.k[u][j];
        d1 += S[j + 1] * w.k[u][j + 1];
      }
      const float dot = sum_lanes<R>(d0 + d1);
      const float uu = w.b[u] * (w.v[u] - dot);
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int j = 0; j < DR; j += 2) {
        S[j] += w.k[u][j] * uu;
        S[j + 1] += w.k[u][j + 1] * uu;
        o0 += S[j] * w.q[u][j];
        o1 += S[j + 1] * w.q[u][j + 1];
      }
      const float out = sum_lanes<R>(o0 + o1);
      if (live && r == 0) MI355_ST(float, o, o + ((cs + i0 + u) * H + h) * dv + col, out);
    }
  };
  fetch(A, cs);
  for (int64_t i0 = 0; i0 < n; i0 += 2 * PF) {
    if (i0 + PF < n) fetch(B, cs + i0 + PF);
    work(A, i0);
    if (i0 + PF >= n) break;
    if (i0 + 2 * PF < n) fetch(A, cs + i0 + 2 * PF);
    work(B, i0 + PF);
  }
  if (live) {
#pragma unroll
    for (int j = 0; j < DR; ++j) {
      const int i = r * DR + j;
      if (i < d) MI355_ST(float, state, sp + static_cast<int64_t>(i) * dv + col, S[j]);
    }
  }
}

// ---- the general delta rule ------------------------------------------------------------------------
// State S [d, d] per head (key channel i, value channel j), a decay per key channel and a removal
// along the unit key, both terms on the OLD state:
//     S <- diag(w) S - (a * u) (u^T S) + k v^T,   o = S^T r
//     w = exp(-e^(-1/2) sigmoid(wl + w0)),  a = sigmoid(al + ab),  u = k / sqrt(|k|^2 + 1e-6)
// wl / al are projection outputs; everything after them is fp32.  general_delta_prep_kernel computes
// w, u, a * u (and fp32 copies of k and r) for every token and head into rows padded to dp; the
// recurrence kernel splits the d rows of a state column over R adjacent lanes as above.
template <typename T>
__global__ __launch_bounds__(64) void general_delta_prep_kernel(
    float* __restrict__ ws, const typename Elem<T>::S* __restrict__ r, int64_t r_stride,
    const typename Elem<T>::S* __restrict__ k, int64_t k_stride, const typename Elem<T>::S* __restrict__ wl,
    int64_t wl_stride, const float* __restrict__ w0, const typename Elem<T>::S* __restrict__ al, int64_t al_stride,
    const float* __restrict__ ab, int H, int d, int dp) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const typename Elem<T>::S* kr = k + t * k_stride + static_cast<int64_t>(h) * d;
  float kk = 0.f;
  for (int c = lane; c < d; c += 64) {
    const float kv = MI355_LDF(T, k, kr + c);
    kk += kv * kv;
  }
  kk = 1.0f / sqrtf(wave_sum(kk) + 1e-6f);
  float* o = ws + (t * H + h) * 5 * dp;                  // w | u | a u | k | r
  for (int c = lane; c < dp; c += 64) {
    float w = 1.f, u = 0.f, au = 0.f, kv = 0.f, rv = 0.f;
    if (c < d) {
      const int64_t hc = static_cast<int64_t>(h) * d + c;
      kv = MI355_LDF(T, k, kr + c);
      rv = MI355_LDF(T, r, r + t * r_stride + hc);
      u = kv * kk;
      const float zw = MI355_LDF(T, wl, wl + t * wl_stride + hc) + MI355_LD(float, w0, w0 + hc);
      w = expf(-0.6065306597126334f / (1.0f + expf(-zw)));
      const float za = MI355_LDF(T, al, al + t * al_stride + hc) + MI355_LD(float, ab, ab + hc);
      au = u / (1.0f + expf(-za));
    }
    MI355_ST(float, ws, o + c, w);
    MI355_ST(float, ws, o + dp + c, u);
    MI355_ST(float, ws, o + 2 * dp + c, au);
    MI355_ST(float, ws, o + 3 * dp + c, kv);
    MI355_ST(float, ws, o + 4 * dp + c, rv);
  }
}

template <typename T, int R, int DR, int PF>
__global__ __launch_bounds__(64) void general_delta_rule_kernel(
    float* __restrict__ o, const typename Elem<T>::S* __restrict__ v, int64_t v_stride, const float* __restrict__ ws,
    float* __restrict__ state, const int32_t* __restrict__ cu_seqlens, const int64_t* __restrict__ positions,
    const int32_t* __restrict__ state_slots, int H, int d) {
  constexpr int dp = R * DR;
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = lane & (R - 1), col = blockIdx.z * (64 / R) + lane / R;
  const int64_t cs = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s);
  const int64_t n = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s + 1) - cs;
  if (n <= 0) return;
  const int64_t slot = MI355_LD(int32_t, state_slots, state_slots + s);
  float* sp = state + ((slot * H + h) * d) * d;
  const bool live = col < d;
  const bool fresh = MI355_LD(int64_t, positions, positions + cs) == 0;
  float S[DR];
#pragma unroll
  for (int j = 0; j < DR; ++j) {
    const int i = r * DR + j;
    S[j] = (live && !fresh && i < d) ? MI355_LD(float, state, sp + static_cast<int64_t>(i) * d + col) : 0.f;
  }
  struct Rows {
    float w[PF][DR], u[PF][DR], au[PF][DR], k[PF][DR], r[PF][DR], v[PF];
  };
  Rows A, B;
  auto fetch = [&](Rows& x, int64_t first) {
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      int64_t t = first + q;
      if (t > cs + n - 1) t = cs + n - 1;               // past the chunk: a row that is loaded and not used
      const float* p = ws + (t * H + h) * 5 * dp + r * DR;
#pragma unroll
      for (int j = 0; j < DR; j += 4) {
        const float4 a4 = MI355_LD(float4, ws, p + j), b4 = MI355_LD(float4, ws, p + dp + j),
                     c4 = MI355_LD(float4, ws, p + 2 * dp + j), d4 = MI355_LD(float4, ws, p + 3 * dp + j),
                     e4 = MI355_LD(float4, ws, p + 4 * dp + j);
        x.w[q][j] = a4.x, x.w[q][j + 1] = a4.y, x.w[q][j + 2] = a4.z, x.w[q][j + 3] = a4.w;
        x.u[q][j] = b4.x, x.u[q][j + 1] = b4.y, x.u[q][j + 2] = b4.z, x.u[q][j + 3] = b4.w;
        x.au[q][j] = c4.x, x.au[q][j + 1] = c4.y, x.au[q][j + 2] = c4.z, x.au[q][j + 3] = c4.w;
        x.k[q][j] = d4.x, x.k[q][j + 1] = d4.y, x.k[q][j + 2] = d4.z, x.k[q][j + 3] = d4.w;
        x.r[q][j] = e4.x, x.r[q][j + 1] = e4.y, x.r[q][j + 2] = e4.z, x.r[q][j + 3] = e4.w;
      }
      x.v[q] = live ? MI355_LDF(T, v, v + t * v_stride + static_cast<int64_t>(h) * d + col) : 0.f;
    }
  };
  auto work = [&](const Rows& x, int64_t i0) {
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      if (i0 + q >= n) break;
      float d0 = 0.f, d1 = 0.f;
#pragma unroll
      for (int j = 0; j < DR; j += 2) {
        d0 += S[j] * x.u[q][j];
        d1 += S[j + 1] * x.u[q][j + 1];
      }
      const float dot = sum_lanes<R>(d0 + d1);          // u^T S of this column, from the old state
      const float vj = x.v[q];
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int j = 0; j < DR; j += 2) {
        S[j] = x.w[q][j] * S[j] - x.au[q][j] * dot + x.k[q][j] * vj;
        S[j + 1] = x.w[q][j + 1] * S[j + 1] - x.au[q][j + 1] * dot + x.k[q][j + 1] * vj;
        o0 += S[j] * x.r[q][j];
        o1 += S[j + 1] * x.r[q][j + 1];
      }
      const float out = sum_lanes<R>(o0 + o1);
      if (live && r == 0) MI355_ST(float, o, o + ((cs + i0 + q) * H + h) * d + col, out);
    }
  };
  fetch(A, cs);
  for (int64_t i0 = 0; i0 < n; i0 += 2 * PF) {
    if (i0 + PF < n) fetch(B, cs + i0 + PF);
    work(A, i0);
    if (i0 + PF >= n) break;
    if (i0 + 2 * PF < n) fetch(A, cs + i0 + 2 * PF);
    work(B, i0 + PF);
  }
  if (live) {
#pragma unroll
    for (int j = 0; j < DR; ++j) {
      const int i = r * DR + j;
      if (i < d) MI355_ST(float, state, sp + static_cast<int64_t>(i) * d + col, S[j]);
    }
  }
}

// The same recurrence for chunks of one or two tokens (decode): one wave per (chunk, head, 64 value
// channels), lane j owns column j of S in registers, so a state row is one coalesced load.  The wave
// prepares the token's vectors itself, in LDS (no workspace, one launch); with heads wider than 64
// the waves of a head each do so.
template <typename T, int D>
__global__ __launch_bounds__(64) void general_delta_rule_cols_kernel(
    float* __restrict__ o, const typename Elem<T>::S* __restrict__ r, int64_t r_stride,
    const typename Elem<T>::S* __restrict__ k, int64_t k_stride, const typename Elem<T>::S* __restrict__ v, int64_t v_stride,
    const typename Elem<T>::S* __restrict__ wl, int64_t wl_stride, const float* __restrict__ w0,
    const typename Elem<T>::S* __restrict__ al, int64_t al_stride, const float* __restrict__ ab, float* __restrict__ state,
    const int32_t* __restrict__ cu_seqlens, const int64_t* __restrict__ positions, const int32_t* __restrict__ state_slots,
    int H, int d) {
  __shared__ float ws[D], us[D], aus[D], ks[D], rs[D];
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, col = blockIdx.z * 64 + lane;
  const int64_t cs = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s);
  const int64_t n = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s + 1) - cs;
  if (n <= 0) return;
  const int64_t slot = MI355_LD(int32_t, state_slots, state_slots + s);
  float* sp = state + ((slot * H + h) * d) * d;
  const bool live = col < d;
  const bool fresh = MI355_LD(int64_t, positions, positions + cs) == 0;
  float S[D];
#pragma unroll
  for (int i = 0; i < D; ++i) S[i] = (live && !fresh && i < d) ? MI355_LD(float, state, sp + static_cast<int64_t>(i) * d + col) : 0.f;
  for (int64_t t = cs; t < cs + n; ++t) {
    const int64_t hd = static_cast<int64_t>(h) * d;
    float kv[(D + 63) / 64], kk = 0.f;
#pragma unroll
    for (int i = 0; i < (D + 63) / 64; ++i) {
      const int c = lane + 64 * i;
      kv[i] = c < d ? MI355_LDF(T, k, k + t * k_stride + hd + c) : 0.f;
      kk += kv[i] * kv[i];
    }
    kk = 1.0f / sqrtf(wave_sum(kk) + 1e-6f);
    __syncthreads();                                    // the previous token's reads of the vectors are done
#pragma unroll
    for (int i = 0; i < (D + 63) / 64; ++i) {
      const int c = lane + 64 * i;
      if (c < D) {
        float w = 1.f, u = 0.f, au = 0.f, rv = 0.f;
        if (c < d) {
          u = kv[i] * kk;
          rv = MI355_LDF(T, r, r + t * r_stride + hd + c);
          const float zw = MI355_LDF(T, wl, wl + t * wl_stride + hd + c) + MI355_LD(float, w0, w0 + hd + c);
          w = expf(-0.6065306597126334f / (1.0f + expf(-zw)));
          const float za = MI355_LDF(T, al, al + t * al_stride + hd + c) + MI355_LD(float, ab, ab + hd + c);
          au = u / (1.0f + expf(-za));
        }
        ws[c] = w, us[c] = u, aus[c] = au, ks[c] = kv[i], rs[c] = rv;
      }
    }
    const float vj = live ? MI355_LDF(T, v, v + t * v_stride + hd + col) : 0.f;
    __syncthreads();
    float d0 = 0.f, d1 = 0.f;
#pragma unroll
    for (int i = 0; i < D; i += 2) {
      d0 += S[i] * us[i];
      d1 += S[i + 1] * us[i + 1];
    }
    const float dot = d0 + d1;
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int i = 0; i < D; i += 2) {
      S[i] = ws[i] * S[i] - aus[i] * dot + ks[i] * vj;
      S[i + 1] = ws[i + 1] * S[i + 1] - aus[i + 1] * dot + ks[i + 1] * vj;
      o0 += S[i] * rs[i];
      o1 += S[i + 1] * rs[i + 1];
    }
    if (live) MI355_ST(float, o, o + (t * H + h) * d + col, o0 + o1);
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < D; ++i)
      if (i < d) MI355_ST(float, state, sp + static_cast<int64_t>(i) * d + col, S[i]);
  }
}

// A gated recurrence per channel whose gates read only the current token (zp, xp, gp: three column
// ranges of the projection rows).  One workgroup per (64 channels, chunk, part of the chunk); its
// waves take consecutive segments of the part's rows.  The recurrence is linear in S, so a run of
// rows is summarised by (A, B) with S_end = A S_start + B: every wave scans its segment from zero for
// (A, B), the summaries of the earlier segments give its true start, and a second scan writes the
// outputs.  A single wave (decoded tokens) scans once.  With several parts per chunk (gridDim.z > 1:
// long prompts, few chunks) a first launch (PASS 1) leaves every part's summary in `parts`
// [chunks, parts, channels, 2], and the second (PASS 2) starts every part from the summaries of
// the parts before it.  State, gates and candidates are fp32.
template <typename T, int PASS>
__global__ __launch_bounds__(1024) void mingru_scan_kernel(
    typename Elem<T>::S* __restrict__ out, const typename Elem<T>::S* __restrict__ proj, int64_t stride, int z_off, int x_off,
    int g_off, const float* __restrict__ bz, const float* __restrict__ bx, float* __restrict__ state,
    const int32_t* __restrict__ cu_seqlens, const int64_t* __restrict__ positions, const int32_t* __restrict__ state_slots,
    int C, float* __restrict__ parts) {
  __shared__ float sa[16][64], sb[16][64];
  const int s = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const bool live = c < C;
  const int q0 = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s), q1 = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s + 1);
  if (q1 <= q0) return;                                 // (the whole workgroup)
  // this workgroup's part of the chunk
  const int nz = gridDim.z, zi = blockIdx.z;
  const int per_z = (q1 - q0 + nz - 1) / nz;
  const int r0 = q0 + zi * per_z < q1 ? q0 + zi * per_z : q1;
  const int r1 = r0 + per_z < q1 ? r0 + per_z : q1;
  const int per = (r1 - r0 + nw - 1) / nw;
  const int a = r0 + wave * per < r1 ? r0 + wave * per : r1;
  const int b = a + per < r1 ? a + per : r1;
  const float zb = (live && bz != nullptr) ? MI355_LD(float, bz, bz + c) : 0.f;
  const float xb = (live && bx != nullptr) ? MI355_LD(float, bx, bx + c) : 0.f;
  auto gates = [&](int t, float& z, float& cand) {
    const typename Elem<T>::S* row = proj + static_cast<int64_t>(t) * stride;
    z = 1.0f / (1.0f + expf(-(MI355_LDF(T, proj, row + z_off + c) + zb)));
    const float u = MI355_LDF(T, proj, row + x_off + c) + xb;
    cand = u >= 0.f ? u + 0.5f : 1.0f / (1.0f + expf(-u));
  };
  if (nw > 1 || PASS == 1) {
    float A = 1.0f, B = 0.f;
    if (live) {
      for (int t = a; t < b; ++t) {
        float z, cand;
        gates(t, z, cand);
        A *= 1.0f - z;
        B = (1.0f - z) * B + z * cand;
      }
    }
    sa[wave][lane] = A;
    sb[wave][lane] = B;
    __syncthreads();
  }
  if (PASS == 1) {                                      // the part's summary: its waves' summaries in turn
    if (wave == 0 && live) {
      float A = 1.0f, B = 0.f;
      for (int i = 0; i < nw; ++i) {
        B = sa[i][lane] * B + sb[i][lane];
        A *= sa[i][lane];
      }
      float* dst = parts + ((static_cast<int64_t>(s) * nz + zi) * C + c) * 2;
      MI355_ST(float, parts, dst, A);
      MI355_ST(float, parts, dst + 1, B);
    }
    return;
  }
  if (!live || a >= b) return;
  const int64_t slot = MI355_LD(int32_t, state_slots, state_slots + s);
  float S = MI355_LD(int64_t, positions, positions + q0) > 0 ? MI355_LD(float, state, state + slot * C + c) : 0.f;
  if (PASS == 2) {
    for (int i = 0; i < zi; ++i) {
      const float* src = parts + ((static_cast<int64_t>(s) * nz + i) * C + c) * 2;
      S = MI355_LD(float, parts, src) * S + MI355_LD(float, parts, src + 1);
    }
  }
  for (int i = 0; i < wave; ++i) S = sa[i][lane] * S + sb[i][lane];
  for (int t = a; t < b; ++t) {
    float z, cand;
    gates(t, z, cand);
    S = (1.0f - z) * S + z * cand;
    const float g = MI355_LDF(T, proj, proj + static_cast<int64_t>(t) * stride + g_off + c);
    MI355_STF(T, out, out + static_cast<int64_t>(t) * C + c, S * (g / (1.0f + expf(-g))));
  }
  if (b == q1) MI355_ST(float, state, state + slot * C + c, S);
}

// out = sigmoid(gate) * sum of the key-range partial sums of sigmoid_window_attn_mfma_kernel
template <typename T>
__global__ __launch_bounds__(256) void window_attn_reduce_kernel(uint16_t* __restrict__ out, const float* __restrict__ partial,
                                                                 const uint16_t* __restrict__ gate, int64_t gate_stride,
                                                                 int64_t rows, int H, int dv, int splits) {
  const int64_t total = rows * H * dv;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    float v = 0.f;
    for (int z = 0; z < splits; ++z) v += MI355_LD(float, partial, partial + z * total + i);
    const int64_t th = i / dv;
    float gt = 1.0f;
    if (gate != nullptr)
      gt = 1.0f / (1.0f + expf(-T::to_f(MI355_LD(uint16_t, gate, gate + (th / H) * gate_stride + th % H))));
    MI355_ST(uint16_t, out, out + i, T::from_f(v * gt));
  }
}

}  // namespace mi355

using namespace mi355;

#define REQ_DTYPE(dtype) MI355_REQUIRE((dtype) >= MI355_BF16 && (dtype) <= MI355_F32, MI355_ERR_UNSUPPORTED, "dtype code %d", (dtype))

extern "C" int32_t mi355_rope_partial_kv_write(void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                               int64_t v_stride, const float* cos_sin, int32_t max_pos,
                                               const int64_t* positions, const int64_t* slot_mapping, void* k_cache,
                                               void* v_cache, int64_t num_tokens, int32_t num_heads,
                                               int32_t num_kv_heads, int32_t head_dim, int32_t v_dim, int32_t rot_dims,
                                               int32_t dtype, void* stream) {
  MI355_REQUIRE(q && cos_sin && positions && slot_mapping, MI355_ERR_INVALID, "rope_partial_kv_write: null pointer");
  MI355_REQUIRE((k && v && k_cache && v_cache) || (!k && !v && !k_cache && !v_cache), MI355_ERR_INVALID,
                "rope_partial_kv_write: k, v and both caches go together (all null: queries only)");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && num_kv_heads > 0 && head_dim > 0 && v_dim > 0 && max_pos > 0,
                MI355_ERR_INVALID, "rope_partial_kv_write: sizes");
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= head_dim && rot_dims % 2 == 0, MI355_ERR_INVALID,
                "rope_partial_kv_write: rot_dims %d must be even and at most head_dim %d", rot_dims, head_dim);
  MI355_REQUIRE(q_stride >= static_cast<int64_t>(num_heads) * head_dim &&
                    (k == nullptr || (k_stride >= static_cast<int64_t>(num_kv_heads) * head_dim &&
                                      v_stride >= static_cast<int64_t>(num_kv_heads) * v_dim)),
                MI355_ERR_INVALID, "rope_partial_kv_write: row strides shorter than the rows");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((rope_partial_kv_write_kernel<TT>), dim3(num_tokens), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(q), q_stride,
                                                  static_cast<const Elem<TT>::S*>(k), k_stride,
                                                  static_cast<const Elem<TT>::S*>(v), v_stride, cos_sin, max_pos,
                                                  positions, slot_mapping, static_cast<Elem<TT>::S*>(k_cache),
                                                  static_cast<Elem<TT>::S*>(v_cache), num_heads, num_kv_heads, head_dim,
                                                  v_dim, rot_dims));
  return check_launch("rope_partial_kv_write");
}

template <typename TT>
static void launch_window_attn(hipStream_t s, void* out, const void* q, int64_t q_stride, const void* k_cache,
                               const void* v_cache, const int32_t* block_tables, int32_t max_blocks,
                               const int32_t* tok_seq, const int64_t* positions, const float* temp, const float* bias,
                               const void* gate, int64_t gate_stride, int64_t T, int H, int G, int d, int dv, int window,
                               float scale) {
  typedef typename Elem<TT>::S E;
  const dim3 grid(static_cast<unsigned>(T), static_cast<unsigned>(H));
  const size_t lds = (static_cast<size_t>(d) + 64) * sizeof(float);
#define MI355_WATTN(N)                                                                                             \
  hipLaunchKernelGGL((sigmoid_window_attn_kernel<TT, N>), grid, dim3(64), lds, s, static_cast<E*>(out),            \
                     static_cast<const E*>(q), q_stride, static_cast<const E*>(k_cache),                           \
                     static_cast<const E*>(v_cache), block_tables, max_blocks, tok_seq, positions, temp, bias,     \
                     static_cast<const E*>(gate), gate_stride, H, G, d, dv, window, scale)
  if (dv <= 64) MI355_WATTN(1);
  else if (dv <= 128) MI355_WATTN(2);
  else MI355_WATTN(4);
#undef MI355_WATTN
}

extern "C" int32_t mi355_sigmoid_window_attn(void* out, const void* q, int64_t q_stride, const void* k_cache,
                                             const void* v_cache, const int32_t* block_tables, int32_t max_blocks,
                                             const int32_t* tok_seq, const int64_t* positions, const float* temp,
                                             const float* bias, const void* gate, int64_t gate_stride,
                                             int64_t num_tokens, int32_t num_heads, int32_t num_kv_heads,
                                             int32_t head_dim, int32_t v_dim, int32_t window, float scale,
                                             const int32_t* tiles, int32_t num_tiles, float* partial,
                                             int32_t num_splits, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && q && k_cache && v_cache && block_tables && tok_seq && positions && temp && bias,
                MI355_ERR_INVALID, "sigmoid_window_attn: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0 &&
                    head_dim > 0 && v_dim > 0 && max_blocks > 0 && window > 0,
                MI355_ERR_INVALID, "sigmoid_window_attn: sizes");
  MI355_REQUIRE(v_dim <= 256 && head_dim <= 8192 && num_heads <= 65535, MI355_ERR_UNSUPPORTED,
                "sigmoid_window_attn: v_dim %d (at most 256), head_dim %d", v_dim, head_dim);
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (tiles != nullptr && num_tiles > 0 && dtype != MI355_F32 && head_dim % 32 == 0 && head_dim <= 256 &&
      v_dim % 16 == 0 && q_stride % 8 == 0 && aligned16(q) && aligned16(k_cache) && aligned16(v_cache)) {
    // the matrix-core form: `tiles` lists (chunk, first row, rows <= 16) for every 16-row tile of the batch
    const int rep = num_heads / num_kv_heads;
    const bool split = partial != nullptr && num_splits > 1;
    MI355_REQUIRE(num_splits >= 0 && num_splits <= 64, MI355_ERR_INVALID, "sigmoid_window_attn: %d key splits", num_splits);
    const bool small = head_dim <= 128 && v_dim <= 128;
    // query heads per wave: four measured faster than two with twice the waves per SIMD (99 vs 131 us
    // for a 2048-token prompt of 16 heads)
    const int hb = !small ? 1 : (rep % 4 == 0 ? 4 : rep % 2 == 0 ? 2 : 1);
    const int waves = num_tiles < 4 ? num_tiles : 4;                              // a tile per wave
    const dim3 grid(static_cast<unsigned>((num_tiles + waves - 1) / waves), static_cast<unsigned>(num_kv_heads * (rep / hb)),
                    split ? num_splits : 1);
    const dim3 block(64u * static_cast<unsigned>(waves));
    const int64_t slab = num_tokens * num_heads * v_dim;
#define MI355_WMFMA(TT, HB, DS, CB)                                                                                 \
  hipLaunchKernelGGL((sigmoid_window_attn_mfma_kernel<TT, HB, DS, CB>), grid, block, 0, s,                          \
                     static_cast<uint16_t*>(out), static_cast<const uint16_t*>(q), q_stride,                        \
                     static_cast<const uint16_t*>(k_cache), static_cast<const uint16_t*>(v_cache), block_tables,    \
                     max_blocks, tiles, num_tiles, positions, temp, bias, static_cast<const uint16_t*>(gate),       \
                     gate_stride, num_heads, num_kv_heads, head_dim, v_dim, window, scale,                          \
                     split ? partial : nullptr, slab)
#define MI355_WMFMA_HB(TT)                                                                                          \
  do {                                                                                                              \
    if (!small) MI355_WMFMA(TT, 1, 8, 16);                                                                          \
    else if (hb == 4) MI355_WMFMA(TT, 4, 4, 8);                                                                     \
    else if (hb == 2) MI355_WMFMA(TT, 2, 4, 8);                                                                     \
    else MI355_WMFMA(TT, 1, 4, 8);                                                                                  \
    if (split)                                                                                                      \
      hipLaunchKernelGGL((window_attn_reduce_kernel<TT>),                                                           \
                         dim3(static_cast<unsigned>((slab + 255) / 256 > 4096 ? 4096 : (slab + 255) / 256)),        \
                         dim3(256), 0, s, static_cast<uint16_t*>(out), partial, static_cast<const uint16_t*>(gate), \
                         gate_stride, num_tokens, num_heads, v_dim, num_splits);                                    \
  } while (0)
    if (dtype == MI355_BF16) MI355_WMFMA_HB(BF16); else MI355_WMFMA_HB(F16);
#undef MI355_WMFMA_HB
#undef MI355_WMFMA
    return check_launch("sigmoid_window_attn (matrix cores)");
  }
  MI355_DISPATCH_DTYPE3(dtype, launch_window_attn<TT>(s, out, q, q_stride, k_cache, v_cache, block_tables, max_blocks,
                                                     tok_seq, positions, temp, bias, gate, gate_stride, num_tokens,
                                                     num_heads, num_kv_heads, head_dim, v_dim, window, scale));
  return check_launch("sigmoid_window_attn");
}

extern "C" int32_t mi355_causal_conv_silu(void* y, const void* x, int64_t x_stride, const void* weight,
                                          const float* state, const int32_t* tok_seq, const int64_t* positions,
                                          const int32_t* cu_seqlens, const int32_t* state_slots, int64_t num_tokens,
                                          int32_t channels, int32_t taps, int32_t dtype, void* stream) {
  MI355_REQUIRE(y && x && weight && state && tok_seq && positions && cu_seqlens && state_slots, MI355_ERR_INVALID,
                "causal_conv_silu: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && channels > 0 && x_stride >= channels, MI355_ERR_INVALID, "causal_conv_silu: sizes");
  MI355_REQUIRE(taps >= 1 && taps <= kMaxTaps, MI355_ERR_UNSUPPORTED, "causal_conv_silu: %d taps (1..%d)", taps, kMaxTaps);
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype != MI355_F32 && taps >= 2 && taps <= 4 && channels % 8 == 0 && x_stride % 8 == 0 && aligned16(x) &&
      aligned16(y) && aligned16(weight) && aligned16(state)) {
    const int64_t vecs = num_tokens * (channels / 8);
    const dim3 vgrid(static_cast<unsigned>((vecs + 255) / 256 > 65536 ? 65536 : (vecs + 255) / 256));
#define MI355_CONV(TT, TAPS)                                                                                      \
  hipLaunchKernelGGL((causal_conv_silu_vec_kernel<TT, TAPS>), vgrid, dim3(256), 0, s, static_cast<uint16_t*>(y),  \
                     static_cast<const uint16_t*>(x), x_stride, static_cast<const uint16_t*>(weight), state,     \
                     tok_seq, positions, cu_seqlens, state_slots, num_tokens, channels)
    if (dtype == MI355_BF16) {
      if (taps == 2) MI355_CONV(BF16, 2); else if (taps == 3) MI355_CONV(BF16, 3); else MI355_CONV(BF16, 4);
    } else {
      if (taps == 2) MI355_CONV(F16, 2); else if (taps == 3) MI355_CONV(F16, 3); else MI355_CONV(F16, 4);
    }
#undef MI355_CONV
    return check_launch("causal_conv_silu");
  }
  const dim3 grid(static_cast<unsigned>(num_tokens), static_cast<unsigned>((channels + 255) / 256 > 64 ? 64 : (channels + 255) / 256));
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((causal_conv_silu_kernel<TT>), grid, dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(y), static_cast<const Elem<TT>::S*>(x),
                                                  x_stride, static_cast<const Elem<TT>::S*>(weight), state, tok_seq,
                                                  positions, cu_seqlens, state_slots, channels, taps));
  return check_launch("causal_conv_silu");
}

extern "C" int32_t mi355_conv_state_update(float* state, const void* x, int64_t x_stride, const int32_t* cu_seqlens,
                                           const int32_t* state_slots, int32_t num_seqs, int32_t channels, int32_t taps,
                                           int32_t dtype, void* stream) {
  MI355_REQUIRE(state && x && cu_seqlens && state_slots, MI355_ERR_INVALID, "conv_state_update: null pointer");
  MI355_REQUIRE(num_seqs >= 0 && channels > 0 && x_stride >= channels, MI355_ERR_INVALID, "conv_state_update: sizes");
  MI355_REQUIRE(taps >= 1 && taps <= kMaxTaps, MI355_ERR_UNSUPPORTED, "conv_state_update: %d taps (1..%d)", taps, kMaxTaps);
  REQ_DTYPE(dtype);
  if (num_seqs == 0 || taps == 1) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(num_seqs), static_cast<unsigned>((channels + 255) / 256 > 64 ? 64 : (channels + 255) / 256));
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((conv_state_update_kernel<TT>), grid, dim3(256), 0, s, state,
                                                  static_cast<const Elem<TT>::S*>(x), x_stride, cu_seqlens, state_slots,
                                                  channels, taps));
  return check_launch("conv_state_update");
}

template <typename TT>
static void launch_delta(hipStream_t s, float* o, const void* qkv, int64_t stride, int q_off, int k_off, int v_off,
                         const void* beta, int64_t beta_stride, const void* decay, int64_t decay_stride,
                         const float* a_log, const float* dt_bias, int per_channel, float* state,
                         const int32_t* cu_seqlens, const int64_t* positions, const int32_t* state_slots, int S, int H,
                         int G, int d, int dv) {
  typedef typename Elem<TT>::S E;
  const dim3 grid(static_cast<unsigned>(S), static_cast<unsigned>(H), static_cast<unsigned>((dv + 63) / 64));
#define MI355_DELTA(D)                                                                                              \
  hipLaunchKernelGGL((gated_delta_rule_kernel<TT, D>), grid, dim3(64), 0, s, o, static_cast<const E*>(qkv), stride, \
                     q_off, k_off, v_off, static_cast<const E*>(beta), beta_stride, static_cast<const E*>(decay),   \
                     decay_stride, a_log, dt_bias, per_channel, state, cu_seqlens, positions, state_slots, H, G, d, dv)
  if (d <= 32) MI355_DELTA(32);
  else if (d <= 64) MI355_DELTA(64);
  else if (d <= 128) MI355_DELTA(128);
  else MI355_DELTA(256);
#undef MI355_DELTA
}

extern "C" int64_t mi355_gated_delta_rule_workspace(int64_t num_tokens, int32_t num_heads, int32_t num_kv_heads,
                                                    int32_t head_dim) {
  const int64_t dp = 8 * (head_dim <= 32 ? 4 : head_dim <= 64 ? 8 : head_dim <= 128 ? 16 : 32);
  return num_tokens * (static_cast<int64_t>(num_kv_heads) * 2 * dp + static_cast<int64_t>(num_heads) * dp + num_heads + 4) / 4 * 4;
}

extern "C" int32_t mi355_gated_delta_rule(float* o, const void* qkv, int64_t stride, int32_t q_off, int32_t k_off,
                                          int32_t v_off, const void* beta, int64_t beta_stride, const void* decay,
                                          int64_t decay_stride, const float* a_log, const float* dt_bias,
                                          int32_t per_channel, float* state, const int32_t* cu_seqlens,
                                          const int64_t* positions, const int32_t* state_slots, int32_t num_seqs,
                                          int32_t num_heads, int32_t num_kv_heads, int32_t head_dim, int32_t v_dim,
                                          int64_t num_tokens, float* workspace, int64_t workspace_floats,
                                          int32_t dtype, void* stream) {
  MI355_REQUIRE(o && qkv && beta && decay && a_log && dt_bias && state && cu_seqlens && positions && state_slots,
                MI355_ERR_INVALID, "gated_delta_rule: null pointer");
  MI355_REQUIRE(num_seqs >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0 && head_dim > 0 &&
                    v_dim > 0 && q_off >= 0 && k_off >= 0 && v_off >= 0,
                MI355_ERR_INVALID, "gated_delta_rule: sizes");
  MI355_REQUIRE(head_dim <= 256 && num_heads <= 65535, MI355_ERR_UNSUPPORTED,
                "gated_delta_rule: head_dim %d (at most 256)", head_dim);
  REQ_DTYPE(dtype);
  if (num_seqs == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (workspace != nullptr && num_tokens > 0) {
    // the form for chunks of many tokens: rows split over 8 lanes, per-token vectors prepared up front
    // state rows of a column over 16 adjacent lanes (8 for heads of up to 32 rows); rows padded to dp
    const int64_t dp = head_dim <= 32 ? 32 : head_dim <= 64 ? 64 : head_dim <= 128 ? 128 : 256;
    const int lanes = head_dim <= 32 ? 8 : 16;
    const int64_t need = mi355_gated_delta_rule_workspace(num_tokens, num_heads, num_kv_heads, head_dim);
    MI355_REQUIRE(workspace_floats >= need && aligned16(workspace), MI355_ERR_INVALID,
                  "gated_delta_rule: workspace of %lld floats, %lld needed, 16-byte aligned",
                  static_cast<long long>(workspace_floats), static_cast<long long>(need));
    float* kq = workspace;
    float* dec = kq + num_tokens * num_kv_heads * 2 * dp;
    float* bet = dec + num_tokens * num_heads * dp;
    const dim3 pgrid(static_cast<unsigned>(num_tokens), static_cast<unsigned>(num_kv_heads + num_heads));
    const int cols = 64 / lanes;
    const dim3 grid(static_cast<unsigned>(num_seqs), static_cast<unsigned>(num_heads), static_cast<unsigned>((v_dim + cols - 1) / cols));
#define MI355_DSPLIT(TT, R, DR, PF)                                                                                   \
  hipLaunchKernelGGL((gated_delta_rule_split_kernel<TT, R, DR, PF>), grid, dim3(64), 0, s, o,                         \
                     static_cast<const Elem<TT>::S*>(qkv), stride, v_off, kq, dec, bet, state, cu_seqlens, positions, \
                     state_slots, num_heads, num_kv_heads, head_dim, v_dim)
    MI355_DISPATCH_DTYPE3(dtype, {
      hipLaunchKernelGGL((delta_prep_kernel<TT>), pgrid, dim3(64), 0, s, kq, dec, bet, static_cast<const Elem<TT>::S*>(qkv),
                         stride, q_off, k_off, static_cast<const Elem<TT>::S*>(beta), beta_stride,
                         static_cast<const Elem<TT>::S*>(decay), decay_stride, a_log, dt_bias, per_channel, num_heads,
                         num_kv_heads, head_dim, static_cast<int>(dp));
      if (dp == 32) MI355_DSPLIT(TT, 8, 4, 4);
      else if (dp == 64) MI355_DSPLIT(TT, 16, 4, 4);
      else if (dp == 128) MI355_DSPLIT(TT, 16, 8, 4);
      else MI355_DSPLIT(TT, 16, 16, 2);
    });
#undef MI355_DSPLIT
    return check_launch("gated_delta_rule (split rows)");
  }
  MI355_DISPATCH_DTYPE3(dtype, launch_delta<TT>(s, o, qkv, stride, q_off, k_off, v_off, beta, beta_stride, decay,
                                               decay_stride, a_log, dt_bias, per_channel, state, cu_seqlens, positions,
                                               state_slots, num_seqs, num_heads, num_kv_heads, head_dim, v_dim));
  return check_launch("gated_delta_rule");
}

static inline int64_t general_delta_dp(int head_dim) { return head_dim <= 32 ? 32 : head_dim <= 64 ? 64 : head_dim <= 128 ? 128 : 256; }

extern "C" int64_t mi355_general_delta_rule_workspace(int64_t num_tokens, int32_t num_heads, int32_t head_dim) {
  return num_tokens * num_heads * 5 * general_delta_dp(head_dim);
}

extern "C" int32_t mi355_general_delta_rule(float* o, const void* r, int64_t r_stride, const void* k, int64_t k_stride,
                                            const void* v, int64_t v_stride, const void* decay, int64_t decay_stride,
                                            const float* decay_bias, const void* rate, int64_t rate_stride,
                                            const float* rate_bias, float* state, const int32_t* cu_seqlens,
                                            const int64_t* positions, const int32_t* state_slots, int32_t num_seqs,
                                            int32_t num_heads, int32_t head_dim, int64_t num_tokens, int32_t long_chunks,
                                            float* workspace, int64_t workspace_floats, int32_t dtype, void* stream) {
  MI355_REQUIRE(o && r && k && v && decay && decay_bias && rate && rate_bias && state && cu_seqlens && positions &&
                    state_slots && (workspace || !long_chunks),
                MI355_ERR_INVALID, "general_delta_rule: null pointer");
  MI355_REQUIRE(num_seqs >= 0 && num_tokens >= 0 && num_heads > 0 && head_dim > 0, MI355_ERR_INVALID,
                "general_delta_rule: sizes");
  MI355_REQUIRE(head_dim <= 256 && num_heads <= 65535, MI355_ERR_UNSUPPORTED,
                "general_delta_rule: head_dim %d (at most 256)", head_dim);
  const int64_t width = static_cast<int64_t>(num_heads) * head_dim;
  MI355_REQUIRE(r_stride >= width && k_stride >= width && v_stride >= width && decay_stride >= width && rate_stride >= width,
                MI355_ERR_INVALID, "general_delta_rule: row strides shorter than the rows");
  REQ_DTYPE(dtype);
  if (num_seqs == 0 || num_tokens == 0) return MI355_OK;
  const int64_t dp = general_delta_dp(head_dim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!long_chunks) {
    // the form for chunks of a token or two: one state column per lane, no workspace
    const dim3 cgrid(static_cast<unsigned>(num_seqs), static_cast<unsigned>(num_heads), static_cast<unsigned>((head_dim + 63) / 64));
#define MI355_GCOLS(D)                                                                                                 \
  hipLaunchKernelGGL((general_delta_rule_cols_kernel<TT, D>), cgrid, dim3(64), 0, s, o, static_cast<const E*>(r),     \
                     r_stride, static_cast<const E*>(k), k_stride, static_cast<const E*>(v), v_stride,                 \
                     static_cast<const E*>(decay), decay_stride, decay_bias, static_cast<const E*>(rate), rate_stride, \
                     rate_bias, state, cu_seqlens, positions, state_slots, num_heads, head_dim)
    MI355_DISPATCH_DTYPE3(dtype, {
      typedef Elem<TT>::S E;
      if (dp == 32) MI355_GCOLS(32);
      else if (dp == 64) MI355_GCOLS(64);
      else if (dp == 128) MI355_GCOLS(128);
      else MI355_GCOLS(256);
    });
#undef MI355_GCOLS
    return check_launch("general_delta_rule (one column per lane)");
  }
  const int64_t need = mi355_general_delta_rule_workspace(num_tokens, num_heads, head_dim);
  MI355_REQUIRE(workspace_floats >= need && aligned16(workspace), MI355_ERR_INVALID,
                "general_delta_rule: workspace of %lld floats, %lld needed, 16-byte aligned",
                static_cast<long long>(workspace_floats), static_cast<long long>(need));
  const int lanes = head_dim <= 32 ? 8 : 16;
  const int cols = 64 / lanes;
  const dim3 pgrid(static_cast<unsigned>(num_tokens), static_cast<unsigned>(num_heads));
  const dim3 grid(static_cast<unsigned>(num_seqs), static_cast<unsigned>(num_heads),
                  static_cast<unsigned>((head_dim + cols - 1) / cols));
#define MI355_GDELTA(TT, R, DR, PF)                                                                                  \
  hipLaunchKernelGGL((general_delta_rule_kernel<TT, R, DR, PF>), grid, dim3(64), 0, s, o,                            \
                     static_cast<const Elem<TT>::S*>(v), v_stride, workspace, state, cu_seqlens, positions,          \
                     state_slots, num_heads, head_dim)
  MI355_DISPATCH_DTYPE3(dtype, {
    typedef Elem<TT>::S E;
    hipLaunchKernelGGL((general_delta_prep_kernel<TT>), pgrid, dim3(64), 0, s, workspace, static_cast<const E*>(r),
                       r_stride, static_cast<const E*>(k), k_stride, static_cast<const E*>(decay), decay_stride,
                       decay_bias, static_cast<const E*>(rate), rate_stride, rate_bias, num_heads, head_dim,
                       static_cast<int>(dp));
    if (dp == 32) MI355_GDELTA(TT, 8, 4, 4);
    else if (dp == 64) MI355_GDELTA(TT, 16, 4, 4);
    else if (dp == 128) MI355_GDELTA(TT, 16, 8, 2);
    else MI355_GDELTA(TT, 16, 16, 1);
  });
#undef MI355_GDELTA
  return check_launch("general_delta_rule");
}

extern "C" int64_t mi355_mingru_scan_workspace(int32_t num_seqs, int32_t channels, int32_t num_parts) {
  return num_parts > 1 ? static_cast<int64_t>(num_seqs) * num_parts * channels * 2 : 0;          // floats
}

extern "C" int32_t mi355_mingru_scan(void* out, const void* proj, int64_t stride, int32_t z_off, int32_t x_off, int32_t g_off,
                                     const float* z_bias, const float* x_bias, float* state, const int32_t* cu_seqlens,
                                     const int64_t* positions, const int32_t* state_slots, int32_t num_seqs,
                                     int64_t num_tokens, int32_t channels, int32_t long_chunks, float* workspace,
                                     int32_t num_parts, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && proj && state && cu_seqlens && positions && state_slots, MI355_ERR_INVALID, "mingru_scan: null pointer");
  MI355_REQUIRE(num_seqs >= 0 && num_seqs <= 65535 && num_tokens >= 0 && channels > 0 && z_off >= 0 && x_off >= 0 && g_off >= 0,
                MI355_ERR_INVALID, "mingru_scan: sizes");
  MI355_REQUIRE(stride >= static_cast<int64_t>(z_off) + channels && stride >= static_cast<int64_t>(x_off) + channels &&
                    stride >= static_cast<int64_t>(g_off) + channels,
                MI355_ERR_INVALID, "mingru_scan: rows shorter than the column ranges");
  MI355_REQUIRE(num_parts >= 0 && num_parts <= 64 && (num_parts <= 1 || workspace != nullptr), MI355_ERR_INVALID,
                "mingru_scan: %d parts per chunk need a workspace", num_parts);
  REQ_DTYPE(dtype);
  if (num_tokens == 0 || num_seqs == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned nz = (long_chunks && num_parts > 1) ? static_cast<unsigned>(num_parts) : 1u;
  const dim3 grid(static_cast<unsigned>((channels + 63) / 64), static_cast<unsigned>(num_seqs), nz);
  const dim3 block(long_chunks ? 1024 : 64);
#define MI355_GRU(PASS)                                                                                                  \
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((mingru_scan_kernel<TT, PASS>), grid, block, 0, s,                     \
                                                  static_cast<Elem<TT>::S*>(out), static_cast<const Elem<TT>::S*>(proj), \
                                                  stride, z_off, x_off, g_off, z_bias, x_bias, state, cu_seqlens,        \
                                                  positions, state_slots, channels, workspace))
  if (nz > 1) {
    MI355_GRU(1);
    MI355_GRU(2);
  } else {
    MI355_GRU(0);
  }
#undef MI355_GRU
  return check_launch("mingru_scan");
}

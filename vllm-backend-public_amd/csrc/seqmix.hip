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
  if (slot < 0) return;
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
    MI355_ST(typename Elem<T>::S, v_cache, v_cache + ((page * G + g) * kPage + off) * dv + j,
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
      const typename Elem<T>::S* vr = v_cache + ((page * G + g) * kPage + key % kPage) * dv;
      const float wj = ws[jj];
#pragma unroll
      for (int i = 0; i < DV_PER_LANE; ++i) {
        const int c = lane + 64 * i;
        if (c < dv) acc[i] += wj * MI355_LDF(T, v_cache, vr + c);
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

}  // namespace mi355

using namespace mi355;

#define REQ_DTYPE(dtype) MI355_REQUIRE((dtype) >= MI355_BF16 && (dtype) <= MI355_F32, MI355_ERR_UNSUPPORTED, "dtype code %d", (dtype))

extern "C" int32_t mi355_rope_partial_kv_write(void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                               int64_t v_stride, const float* cos_sin, int32_t max_pos,
                                               const int64_t* positions, const int64_t* slot_mapping, void* k_cache,
                                               void* v_cache, int64_t num_tokens, int32_t num_heads,
                                               int32_t num_kv_heads, int32_t head_dim, int32_t v_dim, int32_t rot_dims,
                                               int32_t dtype, void* stream) {
  MI355_REQUIRE(q && k && v && cos_sin && positions && slot_mapping && k_cache && v_cache, MI355_ERR_INVALID,
                "rope_partial_kv_write: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && num_kv_heads > 0 && head_dim > 0 && v_dim > 0 && max_pos > 0,
                MI355_ERR_INVALID, "rope_partial_kv_write: sizes");
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= head_dim && rot_dims % 2 == 0, MI355_ERR_INVALID,
                "rope_partial_kv_write: rot_dims %d must be even and at most head_dim %d", rot_dims, head_dim);
  MI355_REQUIRE(q_stride >= static_cast<int64_t>(num_heads) * head_dim &&
                    k_stride >= static_cast<int64_t>(num_kv_heads) * head_dim &&
                    v_stride >= static_cast<int64_t>(num_kv_heads) * v_dim,
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
                                             int32_t dtype, void* stream) {
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

extern "C" int32_t mi355_gated_delta_rule(float* o, const void* qkv, int64_t stride, int32_t q_off, int32_t k_off,
                                          int32_t v_off, const void* beta, int64_t beta_stride, const void* decay,
                                          int64_t decay_stride, const float* a_log, const float* dt_bias,
                                          int32_t per_channel, float* state, const int32_t* cu_seqlens,
                                          const int64_t* positions, const int32_t* state_slots, int32_t num_seqs,
                                          int32_t num_heads, int32_t num_kv_heads, int32_t head_dim, int32_t v_dim,
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
  MI355_DISPATCH_DTYPE3(dtype, launch_delta<TT>(s, o, qkv, stride, q_off, k_off, v_off, beta, beta_stride, decay,
                                               decay_stride, a_log, dt_bias, per_channel, state, cu_seqlens, positions,
                                               state_slots, num_seqs, num_heads, num_kv_heads, head_dim, v_dim));
  return check_launch("gated_delta_rule");
}

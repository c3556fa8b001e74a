// Attention through a low-rank latent with a sliding window and a sink in the softmax.
// What is cached per token is the normed latent c [rank] and ONE rotated key part kr [rot] shared by
// all heads, side by side in the engine's 16-token pages: cache [blocks, 16, rank + rot].  Every
// head's unrotated key is Wuk_h c and its value Wuv_h c; the products with Wuk and Wuv are moved out
// of the loop over keys:
//     score(i, j, h) = ((Wuk_h^T qn_i,h) . c_j + qr_i,h . kr_j) * scale
//     out(i, h)      = Wuv_h (sum_j p_ij c_j)
// so the kernel below sees one key / value head of width rank + rot / rank serving all query heads,
// takes the absorbed query ql = Wuk_h^T qn and returns the weighted latent; the caller applies Wuv.
//   latent_kv_write      c = x[:rank] / rms * w (fp32), kr = rotate(x[rank:]), into the page slot
//   latent_window_attn   p_ij = exp(s_ij) / (exp(sink_h) + sum_{j' in window} exp(s_ij')), keys j with
//                        0 <= i - j < window; the query's rotated part is rotated on the way in; the
//                        result is multiplied by sigmoid(gate[i, h])
// Scores, weights, the softmax and its running sums, norms and angles are fp32.
#include "common.h"

namespace mi355 {

constexpr int kPageL = MI355_BLOCK_SIZE;

// rotate coordinate j of a vector of `rot` coordinates whose first `dims` are rotated (pairs j, j + dims/2)
template <typename T>
__device__ __forceinline__ float rotated_at(const typename Elem<T>::S* base, const typename Elem<T>::S* v, int j, int dims,
                                            const float* table, const float* cs) {
  const int half = dims >> 1;
  if (j >= dims) return MI355_LDF(T, base, v + j);
  if (j < half) {
    const float c = MI355_LD(float, table, cs + j), s = MI355_LD(float, table, cs + half + j);
    return MI355_LDF(T, base, v + j) * c - MI355_LDF(T, base, v + j + half) * s;
  }
  const int jj = j - half;
  const float c = MI355_LD(float, table, cs + jj), s = MI355_LD(float, table, cs + half + jj);
  return MI355_LDF(T, base, v + j) * c + MI355_LDF(T, base, v + jj) * s;
}

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(typename Elem<T>::S* __restrict__ cache,
                                                              const typename Elem<T>::S* __restrict__ x, int64_t x_stride,
                                                              const float* __restrict__ norm_w,
                                                              const float* __restrict__ cos_sin, int max_pos,
                                                              const int64_t* __restrict__ positions,
                                                              const int64_t* __restrict__ slot_mapping, int rank, int rot,
                                                              int dims, float eps) {
  __shared__ float scratch[32];
  const int64_t t = blockIdx.x;
  const int64_t slot = MI355_LD(int64_t, slot_mapping, slot_mapping + t);
  if (slot < 0) return;                                 // (uniform over the workgroup)
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
  const typename Elem<T>::S* row = x + t * x_stride;
  typename Elem<T>::S* dst = cache + slot * (rank + rot);
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = MI355_LDF(T, x, row + i);
    ss += v * v;
  }
  ss = block_sum32(ss, scratch);
  const float r = 1.0f / sqrtf(ss / static_cast<float>(rank) + eps);
  for (int i = threadIdx.x; i < rank; i += blockDim.x)
    MI355_STF(T, cache, dst + i, MI355_LDF(T, x, row + i) * r * MI355_LD(float, norm_w, norm_w + i));
  const float* cs = cos_sin + p * dims;
  for (int j = threadIdx.x; j < rot; j += blockDim.x)
    MI355_STF(T, cache, dst + rank + j, rotated_at<T>(x, row + rank, j, dims, cos_sin, cs));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// One wave per (packed row, query head).  Keys are taken 64 at a time: every lane scores one key,
// the running maximum and sum are updated, the 64 weights go through LDS, then every lane
// accumulates its channels of the latent over the 64 keys.
template <typename T, int CPL>
__global__ __launch_bounds__(64) void latent_window_attn_kernel(
    typename Elem<T>::S* __restrict__ out, int64_t out_stride, int64_t out_head_stride,
    const typename Elem<T>::S* __restrict__ ql, int64_t ql_stride, int64_t ql_head_stride,
    const typename Elem<T>::S* __restrict__ q, int64_t q_stride, int q_head, int q_rot_off,
    const typename Elem<T>::S* __restrict__ cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int64_t* __restrict__ positions, const float* __restrict__ sink,
    const typename Elem<T>::S* __restrict__ gate, int64_t gate_stride, const float* __restrict__ cos_sin, int max_pos,
    int H, int rank, int rot, int dims, int window, float scale) {
  extern __shared__ float lds[];                        // query [rank + rot] | weights [64]
  float* qs = lds;
  float* ws = lds + rank + rot;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int row_w = rank + rot;
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  if (p >= static_cast<int64_t>(max_blocks) * kPageL) p = static_cast<int64_t>(max_blocks) * kPageL - 1;
  const int32_t* bt = block_tables + static_cast<int64_t>(MI355_LD(int32_t, tok_seq, tok_seq + t)) * max_blocks;
  for (int i = lane; i < rank; i += 64) qs[i] = MI355_LDF(T, ql, ql + t * ql_stride + h * ql_head_stride + i);
  {
    const int64_t pc = p >= max_pos ? max_pos - 1 : p;
    const float* cs = cos_sin + pc * dims;
    const typename Elem<T>::S* qr = q + t * q_stride + static_cast<int64_t>(h) * q_head + q_rot_off;
    for (int j = lane; j < rot; j += 64) qs[rank + j] = rotated_at<T>(q, qr, j, dims, cos_sin, cs);
  }
  float m = MI355_LD(float, sink, sink + h), l = 1.0f;  // the sink: one term exp(sink - m), no key, no value
  float acc[CPL];
#pragma unroll
  for (int i = 0; i < CPL; ++i) acc[i] = 0.f;
  int64_t lo = p - window + 1;
  if (lo < 0) lo = 0;
  __syncthreads();
  for (int64_t base = lo; base <= p; base += 64) {
    const int64_t j = base + lane;
    float s = -__builtin_inff();
    if (j <= p) {
      const int64_t page = MI355_LD(int32_t, block_tables, bt + j / kPageL);
      const typename Elem<T>::S* kr = cache + (page * kPageL + j % kPageL) * row_w;
      float d = 0.f;
      for (int i = 0; i < row_w; ++i) d += qs[i] * MI355_LDF(T, cache, kr + i);
      s = d * scale;
    }
    const float mn = fmaxf(m, wave_max(s));
    const float corr = expf(m - mn);
    const float w = j <= p ? expf(s - mn) : 0.f;
    l = l * corr + wave_sum(w);
    m = mn;
#pragma unroll
    for (int i = 0; i < CPL; ++i) acc[i] *= corr;
    ws[lane] = w;
    __syncthreads();
    const int n = static_cast<int>((p - base + 1) < 64 ? (p - base + 1) : 64);
    for (int jj = 0; jj < n; ++jj) {
      const int64_t key = base + jj;
      const int64_t page = MI355_LD(int32_t, block_tables, bt + key / kPageL);
      const typename Elem<T>::S* vr = cache + (page * kPageL + key % kPageL) * row_w;
      const float wj = ws[jj];
#pragma unroll
      for (int i = 0; i < CPL; ++i) {
        const int c = lane + 64 * i;
        if (c < rank) acc[i] += wj * MI355_LDF(T, cache, vr + c);
      }
    }
    __syncthreads();
  }
  float gt = 1.0f / l;
  if (gate != nullptr) gt /= 1.0f + expf(-MI355_LDF(T, gate, gate + t * gate_stride + h));
#pragma unroll
  for (int i = 0; i < CPL; ++i) {
    const int c = lane + 64 * i;
    if (c < rank) MI355_STF(T, out, out + t * out_stride + h * out_head_stride + c, acc[i] * gt);
  }
}

}  // namespace mi355

using namespace mi355;

#define REQ_DTYPE(dtype) MI355_REQUIRE((dtype) >= MI355_BF16 && (dtype) <= MI355_F32, MI355_ERR_UNSUPPORTED, "dtype code %d", (dtype))

extern "C" int32_t mi355_latent_kv_write(void* cache, const void* x, int64_t x_stride, const float* norm_weight,
                                         const float* cos_sin, int32_t max_pos, const int64_t* positions,
                                         const int64_t* slot_mapping, int64_t num_tokens, int32_t rank, int32_t rot,
                                         int32_t rot_dims, float eps, int32_t dtype, void* stream) {
  MI355_REQUIRE(cache && x && norm_weight && cos_sin && positions && slot_mapping, MI355_ERR_INVALID,
                "latent_kv_write: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && rank > 0 && rot >= 0 && max_pos > 0 && x_stride >= rank + rot, MI355_ERR_INVALID,
                "latent_kv_write: sizes");
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, MI355_ERR_INVALID,
                "latent_kv_write: rot_dims %d must be even and at most %d", rot_dims, rot);
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((latent_kv_write_kernel<TT>), dim3(num_tokens), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(cache), static_cast<const Elem<TT>::S*>(x),
                                                  x_stride, norm_weight, cos_sin, max_pos, positions, slot_mapping, rank,
                                                  rot, rot_dims, eps));
  return check_launch("latent_kv_write");
}

template <typename TT>
static void launch_latent_attn(hipStream_t s, void* out, int64_t out_stride, int64_t out_head_stride, const void* ql,
                               int64_t ql_stride, int64_t ql_head_stride, const void* q, int64_t q_stride,
                               int q_head, int q_rot_off, const void* cache, const int32_t* block_tables, int max_blocks,
                               const int32_t* tok_seq, const int64_t* positions, const float* sink, const void* gate,
                               int64_t gate_stride, const float* cos_sin, int max_pos, int64_t T, int H, int rank, int rot,
                               int dims, int window, float scale) {
  typedef typename Elem<TT>::S E;
  const dim3 grid(static_cast<unsigned>(T), static_cast<unsigned>(H));
  const size_t lds = (static_cast<size_t>(rank) + rot + 64) * sizeof(float);
#define MI355_LATTN(N)                                                                                              \
  hipLaunchKernelGGL((latent_window_attn_kernel<TT, N>), grid, dim3(64), lds, s, static_cast<E*>(out), out_stride,  \
                     out_head_stride, static_cast<const E*>(ql), ql_stride, ql_head_stride,                         \
                     static_cast<const E*>(q), q_stride, q_head, q_rot_off,                                         \
                     static_cast<const E*>(cache), block_tables, max_blocks, tok_seq, positions, sink,              \
                     static_cast<const E*>(gate), gate_stride, cos_sin, max_pos, H, rank, rot, dims, window, scale)
  if (rank <= 64) MI355_LATTN(1);
  else if (rank <= 128) MI355_LATTN(2);
  else if (rank <= 256) MI355_LATTN(4);
  else MI355_LATTN(8);
#undef MI355_LATTN
}

extern "C" int32_t mi355_latent_window_attn(void* out, int64_t out_stride, int64_t out_head_stride, const void* q_latent,
                                            int64_t q_latent_stride, int64_t q_latent_head_stride, const void* q,
                                            int64_t q_stride, int32_t q_head_width, int32_t q_rot_offset,
                                            const void* cache, const int32_t* block_tables, int32_t max_blocks,
                                            const int32_t* tok_seq, const int64_t* positions, const float* sink,
                                            const void* gate, int64_t gate_stride, const float* cos_sin, int32_t max_pos,
                                            int64_t num_tokens, int32_t num_heads, int32_t rank, int32_t rot,
                                            int32_t rot_dims, int32_t window, float scale, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && q_latent && q && cache && block_tables && tok_seq && positions && sink && cos_sin,
                MI355_ERR_INVALID, "latent_window_attn: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && num_heads <= 65535 && rank > 0 && rot >= 0 && max_blocks > 0 &&
                    window > 0 && max_pos > 0 && q_rot_offset >= 0 && q_head_width >= q_rot_offset + rot,
                MI355_ERR_INVALID, "latent_window_attn: sizes");
  MI355_REQUIRE(rank <= 512 && rot <= 4096, MI355_ERR_UNSUPPORTED, "latent_window_attn: rank %d (at most 512)", rank);
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, MI355_ERR_INVALID,
                "latent_window_attn: rot_dims %d must be even and at most %d", rot_dims, rot);
  MI355_REQUIRE(q_latent_stride >= rank && q_latent_head_stride >= rank && out_stride >= rank && out_head_stride >= rank &&
                    q_stride >= static_cast<int64_t>(num_heads) * q_head_width,
                MI355_ERR_INVALID, "latent_window_attn: strides shorter than the rows");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, launch_latent_attn<TT>(s, out, out_stride, out_head_stride, q_latent, q_latent_stride,
                                                     q_latent_head_stride, q, q_stride, q_head_width,
                                                     q_rot_offset, cache, block_tables, max_blocks, tok_seq, positions,
                                                     sink, gate, gate_stride, cos_sin, max_pos, num_tokens, num_heads,
                                                     rank, rot, rot_dims, window, scale));
  return check_launch("latent_window_attn");
}

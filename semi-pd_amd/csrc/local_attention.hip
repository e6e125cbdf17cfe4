// Block-local attention with a sink term, and the step in front of it (gfx950, wave64).
//
//  * unit_norm_kv_store_kernel: per head, q <- q / rms(q) in place, k <- k / rms(k) into the key pool,
//    v <- (1 - a) v + a v0 (optional) into the value pool.  Everything between the projection GEMM and the attention
//    in one launch; sums of squares, the division and the blend in fp32.
//  * local_attention_rows_kernel: one wave per (query row, head) for every element type, any head sizes up to 512 / 256.
//    Keys come from the paged pools through the request's row of req_to_token, so a prompt portion, a whole prompt and
//    a decode step are the same walk: query at position p sees keys lo(p) .. p, lo(p) = floor(p / chunk) * chunk
//    (chunk 0: lo = 0).  score = cap * tanh(scale * q.k / cap) (cap 0: none); the softmax denominator holds one more
//    term exp(sink[head]) that has no value row.  Optional epilogue: out *= sigmoid(gate).
//  * local_attention_mfma_kernel (bf16 / f16, head sizes in steps of 32 / 16): 64 query rows of one request and head
//    per workgroup, S^T = K Q^T and O^T += V^T P^T on v_mfma_f32_16x16x32, P^T taken from the accumulators in place.
//  * local_attention_decode_kernel (bf16 / f16): one workgroup per (request, kv head); the waves split the visible keys,
//    the q heads of the group are the MFMA's columns, partials meet in LDS.
#include "common.h"
#include "mfma_frag.h"

namespace semipd {

// ------------------------------------------------------------------------------------------------ norm + store
template <typename T>
__global__ void __launch_bounds__(256) unit_norm_kv_store_kernel(
    T* __restrict__ qkv, int64_t ld, int64_t num_tokens, int H, int G, int D, int E, int64_t k_off, int64_t v_off, float eps,
    const T* __restrict__ v_first, int64_t v_first_ld, const T* __restrict__ mix, T* __restrict__ k_pool,
    T* __restrict__ v_pool, const int64_t* __restrict__ loc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int items = H + 2 * G;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= num_tokens * items) return;
  const int64_t t = item / items;
  const int h = (int)(item % items);
  T* row = qkv + t * ld;
  if (h < H + G) {
    const bool is_q = h < H;
    T* src = is_q ? row + (int64_t)h * D : row + k_off + (int64_t)(h - H) * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float x = Elem<T>::to_f(src[d]);
      ss += x * x;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)D + eps);
    T* dst = is_q ? src : k_pool + (loc[t] * G + (h - H)) * D;
    for (int d = lane; d < D; d += 64) dst[d] = Elem<T>::from_f(Elem<T>::to_f(src[d]) * r);
  } else {
    const int g = h - H - G;
    const T* src = row + v_off + (int64_t)g * E;
    T* dst = v_pool + (loc[t] * G + g) * E;
    if (v_first != nullptr) {
      const float a = Elem<T>::to_f(mix[0]);
      const T* v0 = v_first + t * v_first_ld + (int64_t)g * E;
      for (int e = lane; e < E; e += 64)
        dst[e] = Elem<T>::from_f((1.0f - a) * Elem<T>::to_f(src[e]) + a * Elem<T>::to_f(v0[e]));
    } else {
      for (int e = lane; e < E; e += 64) dst[e] = src[e];
    }
  }
}

// ------------------------------------------------------------------------------------------------ shared pieces
struct LocalAttnArgs {
  const void* q; int64_t q_ld;
  const void* gate; int64_t gate_ld;
  void* out; int64_t out_ld;
  const void* k_pool; const void* v_pool;
  const int32_t* req_to_token; int64_t r2t_stride;
  const int64_t* req_pool_indices; const int64_t* seq_lens;
  const int32_t* q_start; const int32_t* q_len;
  int64_t batch, num_tokens;
  int H, G, D, E;
  const float* sink;
  float scale, cap;
  int chunk;
};

__device__ __forceinline__ float capped(float s, float scale, float cap) {
  s *= scale;
  return cap > 0.f ? cap * tanhf(s / cap) : s;
}

// the request that owns query row t, its position and its table row (q_start == NULL: row t is request t's newest token)
__device__ __forceinline__ bool locate_row(const LocalAttnArgs& a, int64_t t, int& b, int64_t& pos) {
  if (a.q_start == nullptr) {
    b = (int)t;
    pos = a.seq_lens[b] - 1;
    return pos >= 0;
  }
  for (int r = 0; r < (int)a.batch; ++r) {
    const int64_t s = a.q_start[r], n = a.q_len[r];
    if (t >= s && t < s + n) {
      b = r;
      pos = a.seq_lens[r] - n + (t - s);
      return true;
    }
  }
  return false;
}

// ------------------------------------------------------------------------------------------------ one wave per row
template <typename T>
__global__ void __launch_bounds__(256) local_attention_rows_kernel(LocalAttnArgs a) {
  __shared__ float q_lds[4][512];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * 4 + wave;
  const int h = blockIdx.y;
  if (t >= a.num_tokens) return;
  int b;
  int64_t pos;
  if (!locate_row(a, t, b, pos)) return;
  const int D = a.D, E = a.E, G = a.G;
  const int g = h / (a.H / G);
  const T* q = (const T*)a.q + t * a.q_ld + (int64_t)h * D;
  for (int d = lane; d < D; d += 64) q_lds[wave][d] = Elem<T>::to_f(q[d]);
  __builtin_amdgcn_wave_barrier();
  const int32_t* row = a.req_to_token + a.req_pool_indices[b] * a.r2t_stride;
  const int64_t lo = a.chunk > 0 ? (pos / a.chunk) * a.chunk : 0;
  const T* kp = (const T*)a.k_pool;
  const T* vp = (const T*)a.v_pool;
  float m = -INFINITY, l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
  constexpr int V = Elem<T>::kVec;
  for (int64_t j0 = lo; j0 <= pos; j0 += 64) {
    const int64_t j = j0 + lane;
    const bool valid = j <= pos;
    const int slot = valid ? row[j] : 0;
    float s = -INFINITY;
    if (valid) {
      const T* k = kp + ((int64_t)slot * G + g) * D;
      float dot = 0.f;
      if ((D % V) == 0) {
        for (int d = 0; d < D; d += V) {
          const Vec16<T> kv = load16(k + d);
#pragma unroll
          for (int u = 0; u < V; ++u) dot += q_lds[wave][d + u] * Elem<T>::to_f(kv.e[u]);
        }
      } else {
        for (int d = 0; d < D; ++d) dot += q_lds[wave][d] * Elem<T>::to_f(k[d]);
      }
      s = capped(dot, a.scale, a.cap);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);      // first tile: exp(-inf) = 0
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int u = 0; u < 4; ++u) acc[u] *= alpha;
    m = m_new;
    const int n = (int)((pos - j0 + 1) < 64 ? (pos - j0 + 1) : 64);
    for (int jj = 0; jj < n; ++jj) {
      const float pj = __shfl(p, jj, 64);
      const int sj = __shfl(slot, jj, 64);
      const T* v = vp + ((int64_t)sj * G + g) * E;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int e = lane + 64 * u;
        if (e < E) acc[u] += pj * Elem<T>::to_f(v[e]);
      }
    }
  }
  if (a.sink != nullptr) l += expf(a.sink[h] - m);
  const float inv = 1.0f / l;
  T* o = (T*)a.out + t * a.out_ld + (int64_t)h * E;
  const T* gt = a.gate ? (const T*)a.gate + t * a.gate_ld + (int64_t)h * E : nullptr;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int e = lane + 64 * u;
    if (e < E) {
      float y = acc[u] * inv;
      if (gt) y *= 1.0f / (1.0f + expf(-Elem<T>::to_f(gt[e])));
      o[e] = Elem<T>::from_f(y);
    }
  }
}

}  // namespace semipd

using namespace semipd;

extern "C" int semipd_unit_norm_kv_store(void* qkv, int64_t ld, int64_t num_tokens, int num_q_heads, int num_kv_heads,
                                         int qk_dim, int v_dim, int64_t k_off, int64_t v_off, float eps, const void* v_first,
                                         int64_t v_first_ld, const void* mix, void* k_pool, void* v_pool, const int64_t* loc,
                                         int dtype, void* stream) {
  SEMIPD_CHECK_ARG(num_tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0 && qk_dim > 0 && v_dim > 0, SEMIPD_EINVAL,
                   "unit_norm_kv_store: bad sizes");
  if (num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(qkv && k_pool && v_pool && loc, SEMIPD_EINVAL, "unit_norm_kv_store: null pointer");
  SEMIPD_CHECK_ARG((v_first == nullptr) == (mix == nullptr), SEMIPD_EINVAL,
                   "unit_norm_kv_store: the first values and their weight come together");
  SEMIPD_CHECK_ARG(ld >= v_off + (int64_t)num_kv_heads * v_dim && k_off >= (int64_t)num_q_heads * qk_dim &&
                       v_off >= k_off + (int64_t)num_kv_heads * qk_dim,
                   SEMIPD_EINVAL, "unit_norm_kv_store: column ranges overlap or leave the row");
  const int64_t items = num_tokens * (num_q_heads + 2 * num_kv_heads);
  const unsigned blocks = (unsigned)((items + 3) / 4);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((unit_norm_kv_store_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream),
                                           (T*)qkv, ld, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_dim, k_off, v_off, eps,
                                           (const T*)v_first, v_first_ld, (const T*)mix, (T*)k_pool, (T*)v_pool, loc));
  return launch_status("unit_norm_kv_store");
}

extern "C" int semipd_local_attention(const void* q, int64_t q_ld, const void* gate, int64_t gate_ld, void* out, int64_t out_ld,
                                      const void* k_pool, const void* v_pool, const int32_t* req_to_token,
                                      int64_t req_to_token_stride, const int64_t* req_pool_indices, const int64_t* seq_lens,
                                      const int32_t* q_start, const int32_t* q_len, int64_t batch, int64_t num_tokens,
                                      int64_t max_q_len, int num_q_heads, int num_kv_heads, int qk_dim, int v_dim,
                                      const float* sink, float scale, float logit_cap, int chunk, int form, int dtype,
                                      void* stream) {
  SEMIPD_CHECK_ARG(batch >= 0 && num_tokens >= 0, SEMIPD_EINVAL, "local_attention: bad sizes");
  if (batch == 0 || num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0, SEMIPD_ESHAPE,
                   "local_attention: %d query heads over %d key/value heads", num_q_heads, num_kv_heads);
  SEMIPD_CHECK_ARG(qk_dim > 0 && qk_dim <= 512 && v_dim > 0 && v_dim <= 256, SEMIPD_ESHAPE,
                   "local_attention: head sizes %d / %d (at most 512 / 256)", qk_dim, v_dim);
  SEMIPD_CHECK_ARG(q && out && k_pool && v_pool && req_to_token && req_pool_indices && seq_lens, SEMIPD_EINVAL,
                   "local_attention: null pointer");
  SEMIPD_CHECK_ARG((q_start == nullptr) == (q_len == nullptr), SEMIPD_EINVAL, "local_attention: q_start and q_len come together");
  SEMIPD_CHECK_ARG(q_start != nullptr || num_tokens == batch, SEMIPD_EINVAL, "local_attention: one row per request without q_start");
  SEMIPD_CHECK_ARG(chunk >= 0 && logit_cap >= 0.f, SEMIPD_EINVAL, "local_attention: bad chunk or cap");
  LocalAttnArgs a{q, q_ld, gate, gate_ld, out, out_ld, k_pool, v_pool, req_to_token, req_to_token_stride, req_pool_indices,
                  seq_lens, q_start, q_len, batch, num_tokens, num_q_heads, num_kv_heads, qk_dim, v_dim, sink, scale, logit_cap,
                  chunk};
  (void)max_q_len;
  (void)form;
  const dim3 grid((unsigned)((num_tokens + 3) / 4), (unsigned)num_q_heads);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((local_attention_rows_kernel<T>), grid, dim3(256), 0, as_stream(stream), a));
  return launch_status("local_attention");
}

extern "C" int semipd_local_attention_mfma_supported(int num_q_heads, int num_kv_heads, int qk_dim, int v_dim, int dtype) {
  (void)num_q_heads; (void)num_kv_heads; (void)qk_dim; (void)v_dim; (void)dtype;
  return 0;
}

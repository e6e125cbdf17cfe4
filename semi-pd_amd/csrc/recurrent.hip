// Gated linear recurrences over a pool of per-request state rows (gfx950, wave64).
//
// minGRU: per channel c of a request's sequence
//     z_t = sigmoid(zlin_t + bz),   u_t = xlin_t + bx,   cand_t = u_t >= 0 ? u_t + 1/2 : sigmoid(u_t)
//     S_t = (1 - z_t) S_(t-1) + z_t cand_t,              y_t = out_scale * S_t * silu(glin_t)
// zlin | xlin | glin are column ranges of one projection GEMM's output rows (the gates read the current token only), S lives
// in fp32 in the request's slot of the state pool: read when the rows of this launch do not start the sequence, zero
// otherwise, written back after the last row -- so a prompt cut into portions, single decode tokens and a slot that
// another request held before all take the same path.  Gates, candidates and the recurrence are fp32 whatever the
// activation type.
//
//  * min_gru_rows_kernel: a thread per (request, channel) walks the request's rows in order: decode steps and short
//    portions.
//  * min_gru_chunk_*: long prompt portions in chunks of kChunk rows.  The recurrence is linear in S, so a chunk is the map
//    S -> A S + B with A = prod (1 - z_t) and B its result from S = 0: (1) every chunk computes (A, B) side by side, (2) a
//    thread per (request, channel) chains the chunks' maps and leaves every chunk's entry state (and the final state in the
//    pool), (3) every chunk walks its rows again from its entry state and writes y.
#include "common.h"

namespace semipd {

struct MinGruArgs {
  const void* p; int64_t ld;          // projection rows
  int64_t z_off, x_off, g_off;
  const void* bz; const void* bx;     // [R] of the activation type, may be NULL
  void* y; int64_t y_ld;              // [T, >= R] of the activation type
  float* state; int64_t state_ld;     // [slots, >= R] fp32
  const int64_t* state_indices;       // [B]
  const int64_t* seq_lens;            // [B]
  const int32_t* q_start; const int32_t* q_len;   // [B] or NULL (one row per request)
  int64_t batch, num_tokens;
  int R;
  float out_scale;
  float* work;                        // chunked form: [n_chunks][2][R] fp32
  int64_t n_chunks;                   // an upper bound (chunks past the last request's do nothing)
};

constexpr int kChunk = 32;

// 1 / (1 + exp(-x)) from one v_exp_f32 and one v_rcp_f32 (overflow of the exponential gives 0)
__device__ __forceinline__ float sigmoidf_(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

// V adjacent channels of one row as floats (V = 4: one 8- or 16-byte access)
template <typename T, int V> __device__ __forceinline__ void load_ch(const T* p, float (&f)[V]) {
  if constexpr (V == 4 && sizeof(T) == 2) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    T e[4];
    __builtin_memcpy(e, &w, 8);
#pragma unroll
    for (int k = 0; k < 4; ++k) f[k] = Elem<T>::to_f(e[k]);
  } else if constexpr (V == 4) {
    const float4 w = *reinterpret_cast<const float4*>(p);
    f[0] = w.x; f[1] = w.y; f[2] = w.z; f[3] = w.w;
  } else {
#pragma unroll
    for (int k = 0; k < V; ++k) f[k] = Elem<T>::to_f(p[k]);
  }
}
template <typename T, int V> __device__ __forceinline__ void store_ch(T* p, const float (&f)[V]) {
  if constexpr (V == 4 && sizeof(T) == 2) {
    T e[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) e[k] = Elem<T>::from_f(f[k]);
    uint2 w;
    __builtin_memcpy(&w, e, 8);
    *reinterpret_cast<uint2*>(p) = w;
  } else if constexpr (V == 4) {
    *reinterpret_cast<float4*>(p) = float4{f[0], f[1], f[2], f[3]};
  } else {
#pragma unroll
    for (int k = 0; k < V; ++k) p[k] = Elem<T>::from_f(f[k]);
  }
}

// one row of V channels: S <- (1 - z) S + z cand; keep = 1 - z
template <typename T, int V>
__device__ __forceinline__ void gru_step(const T* row, const MinGruArgs& a, int c, const float (&bz)[V], const float (&bx)[V],
                                         float (&S)[V], float (&keep)[V]) {
  float zl[V], xl[V];
  load_ch<T, V>(row + a.z_off + c, zl);
  load_ch<T, V>(row + a.x_off + c, xl);
#pragma unroll
  for (int k = 0; k < V; ++k) {
    const float z = sigmoidf_(zl[k] + bz[k]);
    const float u = xl[k] + bx[k];
    const float cand = u >= 0.f ? u + 0.5f : sigmoidf_(u);
    keep[k] = 1.0f - z;
    S[k] = keep[k] * S[k] + z * cand;
  }
}

template <typename T, int V>
__device__ __forceinline__ void gru_out(const T* row, const MinGruArgs& a, int c, const float (&S)[V], T* y) {
  float g[V], o[V];
  load_ch<T, V>(row + a.g_off + c, g);
#pragma unroll
  for (int k = 0; k < V; ++k) o[k] = a.out_scale * S[k] * (g[k] * sigmoidf_(g[k]));
  store_ch<T, V>(y + c, o);
}

template <typename T, int V>
__device__ __forceinline__ void load_biases(const MinGruArgs& a, int c, float (&bz)[V], float (&bx)[V]) {
#pragma unroll
  for (int k = 0; k < V; ++k) {
    bz[k] = a.bz ? Elem<T>::to_f(((const T*)a.bz)[c + k]) : 0.f;
    bx[k] = a.bx ? Elem<T>::to_f(((const T*)a.bx)[c + k]) : 0.f;
  }
}

template <typename T, int V>
__global__ void __launch_bounds__(256) min_gru_rows_kernel(MinGruArgs a) {
  const int c = (blockIdx.x * 256 + threadIdx.x) * V;
  const int b = blockIdx.y;
  if (c >= a.R) return;
  const int64_t n = a.q_len ? a.q_len[b] : 1, t0 = a.q_start ? a.q_start[b] : b;
  if (n <= 0) return;
  const int64_t first_pos = a.seq_lens[b] - n;
  float* sp = a.state + a.state_indices[b] * a.state_ld + c;
  float S[V], keep[V], bz[V], bx[V];
#pragma unroll
  for (int k = 0; k < V; ++k) S[k] = first_pos > 0 ? sp[k] : 0.f;
  load_biases<T, V>(a, c, bz, bx);
#pragma unroll 2
  for (int64_t i = 0; i < n; ++i) {
    const T* row = (const T*)a.p + (t0 + i) * a.ld;
    gru_step<T, V>(row, a, c, bz, bx, S, keep);
    gru_out<T, V>(row, a, c, S, (T*)a.y + (t0 + i) * a.y_ld);
  }
#pragma unroll
  for (int k = 0; k < V; ++k) sp[k] = S[k];
}

// which request and which of its chunks chunk id `id` is (chunks are counted request after request)
__device__ __forceinline__ bool locate_chunk(const MinGruArgs& a, int64_t id, int& b, int64_t& k) {
  int64_t left = id;
  for (int r = 0; r < (int)a.batch; ++r) {
    const int64_t chunks = ((int64_t)a.q_len[r] + kChunk - 1) / kChunk;
    if (left < chunks) {
      b = r;
      k = left;
      return true;
    }
    left -= chunks;
  }
  return false;
}

template <typename T, int V, bool WRITE>
__global__ void __launch_bounds__(256) min_gru_chunk_kernel(MinGruArgs a) {
  const int c = (blockIdx.x * 256 + threadIdx.x) * V;
  int b;
  int64_t k;
  if (c >= a.R || !locate_chunk(a, blockIdx.y, b, k)) return;
  const int64_t n = a.q_len[b], i0 = k * kChunk, i1 = i0 + kChunk < n ? i0 + kChunk : n, t0 = a.q_start[b];
  float S[V], A[V], keep[V], bz[V], bx[V];
  load_biases<T, V>(a, c, bz, bx);
  float* wk = a.work + (int64_t)blockIdx.y * 2 * a.R;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    S[j] = WRITE ? wk[a.R + c + j] : 0.f;
    A[j] = 1.0f;
  }
#pragma unroll 8
  for (int64_t i = i0; i < i1; ++i) {
    const T* row = (const T*)a.p + (t0 + i) * a.ld;
    gru_step<T, V>(row, a, c, bz, bx, S, keep);
    if constexpr (WRITE) {
      gru_out<T, V>(row, a, c, S, (T*)a.y + (t0 + i) * a.y_ld);
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) A[j] *= keep[j];
    }
  }
  if constexpr (!WRITE) {
#pragma unroll
    for (int j = 0; j < V; ++j) {
      wk[c + j] = A[j];
      wk[a.R + c + j] = S[j];
    }
  }
}

// chains the chunk maps of one request: work[k][1] <- the state the chunk starts from
__global__ void __launch_bounds__(256) min_gru_chain_kernel(MinGruArgs a) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int b = blockIdx.y;
  if (c >= a.R) return;
  const int64_t n = a.q_len[b];
  if (n <= 0) return;
  int64_t first = 0;
  for (int r = 0; r < b; ++r) first += ((int64_t)a.q_len[r] + kChunk - 1) / kChunk;
  const int64_t chunks = (n + kChunk - 1) / kChunk;
  float* sp = a.state + a.state_indices[b] * a.state_ld + c;
  float S = a.seq_lens[b] - n > 0 ? *sp : 0.f;
  for (int64_t k = 0; k < chunks; ++k) {
    float* wk = a.work + (first + k) * 2 * a.R;
    const float A = wk[c], B = wk[a.R + c];
    wk[a.R + c] = S;
    S = A * S + B;
  }
  *sp = S;
}

}  // namespace semipd

using namespace semipd;

extern "C" int64_t semipd_min_gru_workspace(int64_t num_tokens, int64_t batch, int width) {
  return ((num_tokens + kChunk - 1) / kChunk + batch) * 2 * (int64_t)width * 4;
}

extern "C" int semipd_min_gru(const void* proj, int64_t ld, int64_t z_off, int64_t x_off, int64_t g_off, const void* bias_z,
                              const void* bias_x, void* y, int64_t y_ld, float* state, int64_t state_ld,
                              const int64_t* state_indices, const int64_t* seq_lens, const int32_t* q_start,
                              const int32_t* q_len, int64_t batch, int64_t num_tokens, int64_t max_q_len, int width,
                              float out_scale, float* workspace, int64_t workspace_bytes, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(batch >= 0 && num_tokens >= 0 && width > 0, SEMIPD_EINVAL, "min_gru: bad sizes");
  if (batch == 0 || num_tokens == 0) return 0;
  SEMIPD_CHECK_ARG(proj && y && state && state_indices && seq_lens, SEMIPD_EINVAL, "min_gru: null pointer");
  SEMIPD_CHECK_ARG((q_start == nullptr) == (q_len == nullptr), SEMIPD_EINVAL, "min_gru: q_start and q_len come together");
  SEMIPD_CHECK_ARG(q_start != nullptr || num_tokens == batch, SEMIPD_EINVAL, "min_gru: one row per request without q_start");
  SEMIPD_CHECK_ARG(z_off >= 0 && x_off >= 0 && g_off >= 0 && ld >= z_off + width && ld >= x_off + width && ld >= g_off + width &&
                       y_ld >= width && state_ld >= width,
                   SEMIPD_EINVAL, "min_gru: column ranges leave the row");
  SEMIPD_CHECK_ARG(batch <= 65535, SEMIPD_ESHAPE, "min_gru: at most 65535 requests per launch");
  MinGruArgs a{proj, ld, z_off, x_off, g_off, bias_z, bias_x, y, y_ld, state, state_ld, state_indices, seq_lens, q_start, q_len,
               batch, num_tokens, width, out_scale, workspace, 0};
  // four adjacent channels per thread (one 8- or 16-byte access per row and operand) where every range starts on such a piece
  const int64_t esz = dtype == SEMIPD_F32 ? 4 : 2;
  auto piece = [&](const void* ptr, int64_t stride) { return (reinterpret_cast<uintptr_t>(ptr) % (4 * esz)) == 0 && stride % 4 == 0; };
  const bool v4 = width % 4 == 0 && z_off % 4 == 0 && x_off % 4 == 0 && g_off % 4 == 0 && piece(proj, ld) && piece(y, y_ld) &&
                  (reinterpret_cast<uintptr_t>(state) % 16) == 0 && state_ld % 4 == 0;
  const unsigned cb = (unsigned)((width / (v4 ? 4 : 1) + 255) / 256);
  const unsigned cb1 = (unsigned)((width + 255) / 256);
  // long portions in chunks: from a few chunks per request up the three passes beat one thread walking every row
  const bool chunked = q_start != nullptr && max_q_len > 8 * kChunk && workspace != nullptr;
  if (!chunked) {
    SEMIPD_DISPATCH_DTYPE(dtype, T, {
      if (v4) hipLaunchKernelGGL((min_gru_rows_kernel<T, 4>), dim3(cb, (unsigned)batch), dim3(256), 0, as_stream(stream), a);
      else hipLaunchKernelGGL((min_gru_rows_kernel<T, 1>), dim3(cb, (unsigned)batch), dim3(256), 0, as_stream(stream), a);
    });
    return launch_status("min_gru");
  }
  a.n_chunks = (num_tokens + kChunk - 1) / kChunk + batch;
  SEMIPD_CHECK_ARG(workspace_bytes >= a.n_chunks * 2 * (int64_t)width * 4, SEMIPD_EINVAL, "min_gru: workspace too small");
  SEMIPD_CHECK_ARG(a.n_chunks <= 65535, SEMIPD_ESHAPE, "min_gru: too many chunks for one launch");
  SEMIPD_DISPATCH_DTYPE(dtype, T, {
    if (v4) hipLaunchKernelGGL((min_gru_chunk_kernel<T, 4, false>), dim3(cb, (unsigned)a.n_chunks), dim3(256), 0, as_stream(stream), a);
    else hipLaunchKernelGGL((min_gru_chunk_kernel<T, 1, false>), dim3(cb, (unsigned)a.n_chunks), dim3(256), 0, as_stream(stream), a);
    hipLaunchKernelGGL(min_gru_chain_kernel, dim3(cb1, (unsigned)batch), dim3(256), 0, as_stream(stream), a);
    if (v4) hipLaunchKernelGGL((min_gru_chunk_kernel<T, 4, true>), dim3(cb, (unsigned)a.n_chunks), dim3(256), 0, as_stream(stream), a);
    else hipLaunchKernelGGL((min_gru_chunk_kernel<T, 1, true>), dim3(cb, (unsigned)a.n_chunks), dim3(256), 0, as_stream(stream), a);
  });
  return launch_status("min_gru(chunked)");
}

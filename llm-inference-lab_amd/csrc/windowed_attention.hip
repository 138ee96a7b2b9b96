// Attention over a paged cache with a sliding window, a prefix of first positions that
// stays visible, and a softmax whose denominator holds one more, learned term per head
// (a "sink": it has no key and no value).  Keys and values may differ in width.  gfx950.
//
// Pages are row-major: keys  [page, kv head, P, D], values [page, kv head, P, E].
// Sizes are run-time arguments, so one library serves every head size.
#include "common.h"

extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

constexpr float NEG_INF = -__builtin_huge_valf();

// --------------------------------------------------- projection -> q, cache
// One block per row of the step.  proj[r, :] holds the float32 projections of the row:
// q at column 0 (q_size = heads * D wide), then (if the layer has keys and values of its
// own) k (kv heads * D) and v (kv heads * E).  NORM: q and k are each divided by the root
// mean square over their WHOLE width (all heads together) and multiplied by a weight of
// that width, in float32.  q goes to q_out (compute dtype), k and v to the row's place
// in the pages.
template <typename T>
__global__ __launch_bounds__(256) void project_norm_write_kernel(
    const float* __restrict__ proj, int ld, int q_size, int k_size, int v_size, int norm, float eps,
    const float* __restrict__ q_w, const float* __restrict__ k_w, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int n_kv, int D, int E, int page_size,
    const int* __restrict__ positions, const int* __restrict__ row_req, const int* __restrict__ table,
    int max_pages) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const float* src = proj + (size_t)r * ld;
  float inv_q = 1.f, inv_k = 1.f;
  if (norm) {
    float s = 0.f;
    for (int c = threadIdx.x; c < q_size; c += blockDim.x) s += src[c] * src[c];
    inv_q = 1.0f / sqrtf(block_sum(s, red) / (float)q_size + eps);
    if (k_size > 0) {
      s = 0.f;
      for (int c = threadIdx.x; c < k_size; c += blockDim.x) s += src[q_size + c] * src[q_size + c];
      inv_k = 1.0f / sqrtf(block_sum(s, red) / (float)k_size + eps);
    }
  }
  for (int c = threadIdx.x; c < q_size; c += blockDim.x)
    q_out[(size_t)r * q_size + c] = from_float<T>(norm ? src[c] * inv_q * q_w[c] : src[c]);
  if (k_size <= 0) return;
  const int pos = positions[r];
  const int page = table[(size_t)row_req[r] * max_pages + pos / page_size];
  const int slot = pos % page_size;
  for (int c = threadIdx.x; c < k_size; c += blockDim.x) {
    const int g = c / D, d = c - g * D;
    const float v = norm ? src[q_size + c] * inv_k * k_w[c] : src[q_size + c];
    k_cache[(((size_t)page * n_kv + g) * page_size + slot) * D + d] = from_float<T>(v);
  }
  for (int c = threadIdx.x; c < v_size; c += blockDim.x) {
    const int g = c / E, e = c - g * E;
    v_cache[(((size_t)page * n_kv + g) * page_size + slot) * E + e] = from_float<T>(src[q_size + k_size + c]);
  }
}

extern "C" int llmlab_project_norm_write(const float* proj, int ld, int rows, int n_heads, int n_kv, int D, int E,
                                         int own_kv, int norm, float eps, const float* q_w, const float* k_w,
                                         void* q_out, void* k_cache, void* v_cache, int dtype, int page_size,
                                         const int* positions, const int* row_req, const int* table,
                                         int max_pages, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_kv > 0 && D > 0 && E > 0 && page_size > 0,
                 "project_norm_write: bad sizes rows=%d heads=%d kv=%d D=%d E=%d page=%d", rows, n_heads, n_kv, D, E,
                 page_size);
  const int q_size = n_heads * D, k_size = own_kv ? n_kv * D : 0, v_size = own_kv ? n_kv * E : 0;
  LLMLAB_REQUIRE(ld >= q_size + k_size + v_size, "project_norm_write: rows of %d numbers do not hold %d", ld,
                 q_size + k_size + v_size);
  LLMLAB_REQUIRE(!norm || (q_w && (!own_kv || k_w)), "project_norm_write: the norm needs its weights");
  LLMLAB_REQUIRE(!own_kv || (k_cache && v_cache && positions && row_req && table),
                 "project_norm_write: keys and values need pages to go to");
  if (rows == 0) return 0;
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(project_norm_write_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, proj, ld, q_size, k_size,
                       v_size, norm, eps, q_w, k_w, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, n_kv, D, E,
                       page_size, positions, row_req, table, max_pages);
  else
    hipLaunchKernelGGL(project_norm_write_kernel<float>, dim3(rows), dim3(256), 0, stream, proj, ld, q_size, k_size,
                       v_size, norm, eps, q_w, k_w, (float*)q_out, (float*)k_cache, (float*)v_cache, n_kv, D, E,
                       page_size, positions, row_req, table, max_pages);
  LLMLAB_LAUNCH_CHECK("project_norm_write");
  return 0;
}

// ------------------------------------------------------------------ attention
// The query at position i of its request sees key j if j <= i and (i - j < window or
// j < keep_first); window <= 0: every j <= i.  The visible keys are two runs: the kept
// prefix [0, nA) with nA = min(keep_first, lo), and [lo, i] with lo = max(0, i - window + 1).
// Scores, the running maximum, the denominator and the weighted sum of values are float32.
// With a sink the running maximum starts at sink[h] and the denominator at 1 = exp(sink -
// sink): the term counts once and brings no value.
//
// One wave per (row, head).  Keys are taken 64 at a time: lane n scores one key (its own
// row of D numbers), the weights go through LDS, then lane e sums the values' column e
// (and e + 64, ...), so that every value row is read across the wave.
constexpr int MAX_E_PER_LANE = 4;      // value width up to 256

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ q, const T* __restrict__ k, int D);

template <>
__device__ __forceinline__ float dot_row<float>(const float* __restrict__ q, const float* __restrict__ k, int D) {
  float s = 0.f;
  if ((D & 3) == 0) {
    for (int d = 0; d < D; d += 4) {
      const floatx4 kv = *(const floatx4*)(k + d);
      s = fmaf(q[d], kv[0], s);
      s = fmaf(q[d + 1], kv[1], s);
      s = fmaf(q[d + 2], kv[2], s);
      s = fmaf(q[d + 3], kv[3], s);
    }
  } else {
    for (int d = 0; d < D; ++d) s = fmaf(q[d], k[d], s);
  }
  return s;
}

template <>
__device__ __forceinline__ float dot_row<bf16_t>(const float* __restrict__ q, const bf16_t* __restrict__ k, int D) {
  float s = 0.f;
  if ((D & 7) == 0) {
    for (int d = 0; d < D; d += 8) {
      const bf16x8 kv = *(const bf16x8*)(k + d);
#pragma unroll
      for (int j = 0; j < 8; ++j) s = fmaf(q[d + j], (float)kv[j], s);
    }
  } else {
    for (int d = 0; d < D; ++d) s = fmaf(q[d], (float)k[d], s);
  }
  return s;
}

template <typename T>
__global__ __launch_bounds__(64) void sink_window_attention_kernel(
    const T* __restrict__ q, int n_heads, int n_kv, int D, int E, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ table, int max_pages, int page_size,
    const int* __restrict__ positions, const int* __restrict__ row_req, int window, int keep_first,
    const float* __restrict__ sink, float scale, T* __restrict__ out) {
  extern __shared__ float lds[];       // q [D], weights [64], value rows [64] (as ints)
  float* qs = lds;
  float* ps = lds + D;
  size_t* vrow = (size_t*)(lds + D + 64 + ((D & 1) ? 1 : 0));
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (n_heads / n_kv);
  const int i = positions[r];
  const int* pages = table + (size_t)row_req[r] * max_pages;
  for (int d = lane; d < D; d += 64) qs[d] = to_float(q[((size_t)r * n_heads + h) * D + d]) * scale;
  __syncthreads();
  const int lo = window > 0 ? (i - window + 1 > 0 ? i - window + 1 : 0) : 0;
  const int nA = keep_first < lo ? keep_first : lo;
  const int total = nA + (i - lo + 1);
  float m = sink ? sink[h] : NEG_INF;
  float l = sink ? 1.f : 0.f;
  float acc[MAX_E_PER_LANE];
#pragma unroll
  for (int c = 0; c < MAX_E_PER_LANE; ++c) acc[c] = 0.f;
  for (int base = 0; base < total; base += 64) {
    const int n = base + lane;
    const bool valid = n < total;
    float s = NEG_INF;
    size_t row = 0;
    if (valid) {
      const int j = n < nA ? n : lo + (n - nA);
      const int page = pages[j / page_size];
      row = ((size_t)page * n_kv + g) * page_size + (j % page_size);
      s = dot_row<T>(qs, k_cache + row * D, D);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? __expf(s - m_new) : 0.f;
    const float corr = (m == NEG_INF) ? 0.f : __expf(m - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
    ps[lane] = p;
    vrow[lane] = row;
    __syncthreads();
    const int count = total - base < 64 ? total - base : 64;
#pragma unroll
    for (int c = 0; c < MAX_E_PER_LANE; ++c) {
      const int e = lane + 64 * c;
      if (e < E) {
        float a = acc[c] * corr;
        for (int t = 0; t < count; ++t) a = fmaf(ps[t], to_float(v_cache[vrow[t] * E + e]), a);
        acc[c] = a;
      }
    }
    __syncthreads();
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < MAX_E_PER_LANE; ++c) {
    const int e = lane + 64 * c;
    if (e < E) out[((size_t)r * n_heads + h) * E + e] = from_float<T>(acc[c] * inv);
  }
}

// q [rows, heads * D], out [rows, heads * E] in the compute dtype; sink: float32 [heads] or null.
extern "C" int llmlab_sink_window_attention(const void* q, int dtype, int rows, int n_heads, int n_kv, int D, int E,
                                            const void* k_cache, const void* v_cache, const int* table, int max_pages,
                                            int page_size, const int* positions, const int* row_req, int window,
                                            int keep_first, const float* sink, float scale, void* out,
                                            hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && D > 0 && E > 0,
                 "sink_window_attention: bad sizes rows=%d heads=%d kv=%d D=%d E=%d", rows, n_heads, n_kv, D, E);
  LLMLAB_REQUIRE(E <= 64 * MAX_E_PER_LANE, "sink_window_attention: values up to %d wide, got %d", 64 * MAX_E_PER_LANE, E);
  LLMLAB_REQUIRE(D <= 4096 && n_heads <= 65535, "sink_window_attention: keys up to 4096 wide and 65535 heads");
  LLMLAB_REQUIRE(keep_first >= 0 && page_size > 0 && max_pages > 0, "sink_window_attention: bad window arguments");
  if (rows == 0) return 0;
  const size_t lds = (size_t)(D + 64 + (D & 1)) * sizeof(float) + 64 * sizeof(size_t);
  dim3 grid(rows, n_heads), block(64);
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(sink_window_attention_kernel<bf16_t>, grid, block, lds, stream, (const bf16_t*)q, n_heads, n_kv, D,
                       E, (const bf16_t*)k_cache, (const bf16_t*)v_cache, table, max_pages, page_size, positions,
                       row_req, window, keep_first, sink, scale, (bf16_t*)out);
  else
    hipLaunchKernelGGL(sink_window_attention_kernel<float>, grid, block, lds, stream, (const float*)q, n_heads, n_kv, D,
                       E, (const float*)k_cache, (const float*)v_cache, table, max_pages, page_size, positions,
                       row_req, window, keep_first, sink, scale, (float*)out);
  LLMLAB_LAUNCH_CHECK("sink_window_attention");
  return 0;
}

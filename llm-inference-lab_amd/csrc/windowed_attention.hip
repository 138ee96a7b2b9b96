// Attention over a paged cache with a sliding window, a prefix of first positions that
// stays visible, and a softmax whose denominator holds one more, learned term per head
// (a "sink": it has no key and no value).  Keys and values may differ in width.  gfx950.
//
// Pages: keys [page, kv head, P, D] row by row; values [page, kv head, P, E] with the P * E
// numbers of a (page, kv head) in the order [P / 4][E][4]: the four keys of a quad side by
// side for each value channel, so that the sum over keys reads 8 bytes a lane (the matrix
// cores want runs of keys, the plain kernel four weights a load).
// Sizes are run-time arguments, so one library serves every head size.
#include "common.h"

extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

constexpr float NEG_INF = -__builtin_huge_valf();

// where the value of the key at offset o of its page lies, channel e of E
__host__ __device__ inline size_t value_index(int o, int e, int E) { return ((size_t)(o >> 2) * E + e) * 4 + (o & 3); }

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
    v_cache[((size_t)page * n_kv + g) * page_size * E + value_index(slot, e, E)] = from_float<T>(src[q_size + k_size + c]);
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
// j < keep_first); window <= 0: every j <= i.  Scores, the running maximum, the denominator
// and the weighted sum of values are float32.  With a sink the running maximum starts at
// sink[h] and the denominator at 1 = exp(sink - sink): the term counts once and brings no value.
//
// Both kernels walk the keys in two runs, each from an aligned start, and mask key by key:
// the kept prefix [0, min(keep_first, B)) and [B, i], where B is the window's first key
// rounded down (to a quad of keys here, to 16 in the matrix-core kernel).
__device__ __forceinline__ bool sees(int i, int j, int window, int keep_first) {
  return j <= i && (window <= 0 || i - j < window || j < keep_first);
}

// ---- plain kernel: one wave per (row, head); float32 products.  Keys are taken 64 at a
// time: lane n scores one key (its own row of D numbers), the weights go through LDS, then
// lane e sums the values' channel e (and e + 64, ...) a quad of keys a load.
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

__device__ __forceinline__ void load_quad(const float* p, float (&v)[4]) {
  const floatx4 t = *(const floatx4*)p;
  v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
}
__device__ __forceinline__ void load_quad(const bf16_t* p, float (&v)[4]) {
  const bf16x4 t = *(const bf16x4*)p;
  v[0] = (float)t[0]; v[1] = (float)t[1]; v[2] = (float)t[2]; v[3] = (float)t[3];
}

template <typename T>
__global__ __launch_bounds__(64) void sink_window_attention_kernel(
    const T* __restrict__ q, int n_heads, int n_kv, int D, int E, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ table, int max_pages, int page_size,
    const int* __restrict__ positions, const int* __restrict__ row_req, int window, int keep_first,
    const float* __restrict__ sink, float scale, T* __restrict__ out) {
  extern __shared__ float lds[];       // q [D], weights [64], first value of each key's quad [64]
  float* qs = lds;
  float* ps = lds + D;
  size_t* vquad = (size_t*)(lds + D + 64 + ((D & 1) ? 1 : 0));
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (n_heads / n_kv);
  const int i = positions[r];
  const int* pages = table + (size_t)row_req[r] * max_pages;
  for (int d = lane; d < D; d += 64) qs[d] = to_float(q[((size_t)r * n_heads + h) * D + d]) * scale;
  __syncthreads();
  const int lo = window > 0 ? (i - window + 1 > 0 ? i - window + 1 : 0) : 0;
  const int b_start = lo & ~3;
  const int a_end = keep_first < b_start ? keep_first : b_start;
  float m = sink ? sink[h] : NEG_INF;
  float l = sink ? 1.f : 0.f;
  float acc[MAX_E_PER_LANE];
#pragma unroll
  for (int c = 0; c < MAX_E_PER_LANE; ++c) acc[c] = 0.f;
  for (int run = 0; run < 2; ++run) {
    const int first = run == 0 ? 0 : b_start;
    const int end = run == 0 ? a_end : i + 1;          // keys [first, end)
    for (int base = first; base < end; base += 64) {
      const int j = base + lane;
      const bool valid = j < end && sees(i, j, window, keep_first);
      float s = NEG_INF;
      if (j < end) {
        const int page = pages[j / page_size];
        const size_t head = ((size_t)page * n_kv + g) * page_size;
        if (valid) s = dot_row<T>(qs, k_cache + (head + (j % page_size)) * D, D);
        vquad[lane] = head * E + value_index(j % page_size, 0, E);       // (lanes 4 n are read below)
      }
      const float m_new = fmaxf(m, wave_max(s));
      const float p = valid ? __expf(s - m_new) : 0.f;
      const float corr = (m == NEG_INF) ? 0.f : __expf(m - m_new);
      l = l * corr + wave_sum(p);
      m = m_new;
      ps[lane] = p;
      __syncthreads();
      const int quads = ((end - base < 64 ? end - base : 64) + 3) >> 2;
#pragma unroll
      for (int c = 0; c < MAX_E_PER_LANE; ++c) {
        const int e = lane + 64 * c;
        if (e < E) {
          float a = acc[c] * corr;
          for (int t = 0; t < quads; ++t) {
            float v[4];
            load_quad(v_cache + vquad[4 * t] + (size_t)e * 4, v);
            a = fmaf(ps[4 * t], v[0], a);
            a = fmaf(ps[4 * t + 1], v[1], a);
            a = fmaf(ps[4 * t + 2], v[2], a);
            a = fmaf(ps[4 * t + 3], v[3], a);
          }
          acc[c] = a;
        }
      }
      __syncthreads();
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < MAX_E_PER_LANE; ++c) {
    const int e = lane + 64 * c;
    if (e < E) out[((size_t)r * n_heads + h) * E + e] = from_float<T>(acc[c] * inv);
  }
}

// ---- matrix-core kernel (bfloat16; D a multiple of 32, E of 16).  A wave takes 16
// consecutive rows of the step and one head; a block four such tiles.  Keys come 32 at a
// time as two blocks of 16 (each within a page).  The scores are taken transposed, S^T = K
// Q^T, so that a lane ends up with the weights of ONE query for eight keys: exactly the
// operand the second product O^T = V^T P^T wants, with no trip through LDS.  Lane l = 16 g +
// c holds query c and, of a block of 16 keys, the keys 4 g .. 4 g + 3.  Rows of several
// requests in one tile are served request after request (the others' columns masked).
template <int DC, int EB>
__global__ __launch_bounds__(256) void sink_window_attention_mfma_kernel(
    const bf16_t* __restrict__ q, int n_rows, int n_heads, int n_kv, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ table, int max_pages, int page_size,
    const int* __restrict__ positions, const int* __restrict__ row_req, int window, int keep_first,
    const float* __restrict__ sink, float scale, bf16_t* __restrict__ out) {
  constexpr int D = 32 * DC, E = 16 * EB;
  const int lane = threadIdx.x & 63, c = lane & 15, g4 = lane >> 4;
  const int r0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 16;
  if (r0 >= n_rows) return;
  const int h = blockIdx.y, g = h / (n_heads / n_kv);
  const int r = r0 + c;
  const bool row_ok = r < n_rows;
  const int pos = row_ok ? positions[r] : 0;
  const int req = row_ok ? row_req[r] : -1;
  bf16x8 qf[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) {
    if (row_ok) qf[dc] = *(const bf16x8*)(q + ((size_t)r * n_heads + h) * D + 32 * dc + 8 * g4);
    else
#pragma unroll
      for (int t = 0; t < 8; ++t) qf[dc][t] = (bf16_t)0.f;
  }
  float m = sink ? sink[h] : NEG_INF;
  float l = sink ? 1.f : 0.f;
  floatx4 o[EB];
#pragma unroll
  for (int eb = 0; eb < EB; ++eb) o[eb] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int b_first = __builtin_amdgcn_readfirstlane(row_req[r0]);
  const int b_last = __builtin_amdgcn_readfirstlane(row_req[(r0 + 15 < n_rows ? r0 + 15 : n_rows - 1)]);
  for (int b = b_first; b <= b_last; ++b) {
    const bool mine = req == b;
    // the first and the last position among this request's rows of the tile
    int p_lo = mine ? pos : 0x7fffffff, p_hi = mine ? pos : -1;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      p_lo = min(p_lo, __shfl_xor(p_lo, off, WAVE));
      p_hi = max(p_hi, __shfl_xor(p_hi, off, WAVE));
    }
    if (p_hi < 0) continue;
    const int lo = window > 0 ? (p_lo - window + 1 > 0 ? p_lo - window + 1 : 0) : 0;
    const int b_start = lo & ~15;
    const int a_end = keep_first < b_start ? keep_first : b_start;
    const int* pages = table + (size_t)b * max_pages;
    for (int run = 0; run < 2; ++run) {
      const int first = run == 0 ? 0 : b_start;
      const int end = run == 0 ? a_end : p_hi + 1;
      for (int j0 = first; j0 < end; j0 += 32) {
        floatx4 s[2];
        size_t vbase[2];
        bool have[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int ju = j0 + 16 * u;
          have[u] = ju < end;
          s[u] = floatx4{0.f, 0.f, 0.f, 0.f};
          vbase[u] = 0;
          if (have[u]) {
            const int page = pages[ju / page_size];
            const size_t head = ((size_t)page * n_kv + g) * page_size;
            const int off = ju % page_size;
            const bf16_t* kp = k_cache + (head + off + c) * D + 8 * g4;
#pragma unroll
            for (int dc = 0; dc < DC; ++dc)
              s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(kp + 32 * dc), qf[dc], s[u], 0, 0, 0);
            vbase[u] = head * E + (size_t)((off >> 2) + g4) * E * 4;
          }
        }
        float tmax = NEG_INF;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int j = j0 + 16 * u + 4 * g4 + t;
            const bool ok = have[u] && mine && j < end && sees(pos, j, window, keep_first);
            s[u][t] = ok ? s[u][t] * scale : NEG_INF;
            tmax = fmaxf(tmax, s[u][t]);
          }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
        const float m_new = fmaxf(m, tmax);
        const float m_use = m_new == NEG_INF ? 0.f : m_new;
        const float corr = m == NEG_INF ? 0.f : __expf(m - m_use);
        float sum = 0.f;
        bf16x8 pf;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const float p = __expf(s[u][t] - m_use);       // (exp(-inf) = 0 for a masked key)
            sum += p;
            pf[4 * u + t] = (bf16_t)p;
          }
        sum += __shfl_xor(sum, 16, WAVE);
        sum += __shfl_xor(sum, 32, WAVE);
        l = l * corr + sum;
        m = m_new;
#pragma unroll
        for (int eb = 0; eb < EB; ++eb) {
          bf16x8 vf;
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            bf16x4 quad = bf16x4{(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
            if (have[u]) quad = *(const bf16x4*)(v_cache + vbase[u] + (size_t)(16 * eb + c) * 4);
#pragma unroll
            for (int t = 0; t < 4; ++t) vf[4 * u + t] = quad[t];
          }
#pragma unroll
          for (int t = 0; t < 4; ++t) o[eb][t] *= corr;
          o[eb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[eb], 0, 0, 0);
        }
      }
    }
  }
  if (!row_ok) return;
  const float inv = 1.0f / l;
#pragma unroll
  for (int eb = 0; eb < EB; ++eb) {
    bf16x4 w;
#pragma unroll
    for (int t = 0; t < 4; ++t) w[t] = (bf16_t)(o[eb][t] * inv);
    *(bf16x4*)(out + ((size_t)r * n_heads + h) * E + 16 * eb + 4 * g4) = w;
  }
}

static int g_force_plain = 0;
extern "C" void llmlab_debug_windowed_attention_plain(int on) { g_force_plain = on; }

// Whether a call of these sizes goes to the matrix-core kernel.
extern "C" int llmlab_sink_window_attention_uses_mfma(int dtype, int rows, int D, int E, int page_size) {
  return !g_force_plain && dtype == DT_BF16 && rows >= 32 && D % 32 == 0 && D <= 128 && E % 16 == 0 && E <= 128 &&
         page_size % 16 == 0;
}

template <int DC>
static void launch_mfma(int EBv, dim3 grid, hipStream_t stream, const bf16_t* q, int rows, int n_heads, int n_kv,
                        const bf16_t* k_cache, const bf16_t* v_cache, const int* table, int max_pages, int page_size,
                        const int* positions, const int* row_req, int window, int keep_first, const float* sink,
                        float scale, bf16_t* out) {
#define LLMLAB_MFMA(EBC)                                                                                          \
  case EBC:                                                                                                       \
    hipLaunchKernelGGL((sink_window_attention_mfma_kernel<DC, EBC>), grid, dim3(256), 0, stream, q, rows, n_heads, \
                       n_kv, k_cache, v_cache, table, max_pages, page_size, positions, row_req, window, keep_first, \
                       sink, scale, out);                                                                         \
    break;
  switch (EBv) {
    LLMLAB_MFMA(1) LLMLAB_MFMA(2) LLMLAB_MFMA(3) LLMLAB_MFMA(4) LLMLAB_MFMA(5) LLMLAB_MFMA(6) LLMLAB_MFMA(7) LLMLAB_MFMA(8)
  }
#undef LLMLAB_MFMA
}

// q [rows, heads * D], out [rows, heads * E] in the compute dtype; sink: float32 [heads] or null.
// The rows of a request are adjacent and requests come in rising order of row_req.
extern "C" int llmlab_sink_window_attention(const void* q, int dtype, int rows, int n_heads, int n_kv, int D, int E,
                                            const void* k_cache, const void* v_cache, const int* table, int max_pages,
                                            int page_size, const int* positions, const int* row_req, int window,
                                            int keep_first, const float* sink, float scale, void* out,
                                            hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && D > 0 && E > 0,
                 "sink_window_attention: bad sizes rows=%d heads=%d kv=%d D=%d E=%d", rows, n_heads, n_kv, D, E);
  LLMLAB_REQUIRE(E <= 64 * MAX_E_PER_LANE, "sink_window_attention: values up to %d wide, got %d", 64 * MAX_E_PER_LANE, E);
  LLMLAB_REQUIRE(D <= 4096 && n_heads <= 65535, "sink_window_attention: keys up to 4096 wide and 65535 heads");
  LLMLAB_REQUIRE(keep_first >= 0 && page_size > 0 && page_size % 4 == 0 && max_pages > 0,
                 "sink_window_attention: bad window or page arguments");
  if (rows == 0) return 0;
  if (llmlab_sink_window_attention_uses_mfma(dtype, rows, D, E, page_size)) {
    dim3 grid((rows + 63) / 64, n_heads);
#define LLMLAB_ARGS E / 16, grid, stream, (const bf16_t*)q, rows, n_heads, n_kv, (const bf16_t*)k_cache,             \
                    (const bf16_t*)v_cache, table, max_pages, page_size, positions, row_req, window, keep_first, sink, \
                    scale, (bf16_t*)out
    switch (D / 32) {
      case 1: launch_mfma<1>(LLMLAB_ARGS); break;
      case 2: launch_mfma<2>(LLMLAB_ARGS); break;
      case 3: launch_mfma<3>(LLMLAB_ARGS); break;
      default: launch_mfma<4>(LLMLAB_ARGS); break;
    }
#undef LLMLAB_ARGS
    LLMLAB_LAUNCH_CHECK("sink_window_attention (matrix cores)");
    return 0;
  }
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

// Gated linear attention: a matrix-valued recurrent state per head,
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
// with a decay a_t in (0, 1) per key channel.  The state [D, E] per head lives in float32 in
// a slot per request and is carried from step to step; everything here is float32.  gfx950.
//
// Three kernels: the decays from their low-rank projection; the scan over the tokens of every
// request of the step (prompts' portions and single decoded tokens alike); the output
// (norm over each head's values, gate, rounding to the compute dtype).
#include "common.h"

extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

constexpr int SLICE = 16;      // key channels of the state that one thread keeps in registers

// ---------------------------------------------------------------------- decays
// a[r, c] = sigmoid(z)^(1 / tau), z = bias[c] + sum_j w2[c, j] * low[r, j]  (c over heads * D
// key channels, j over the rank of the projection).  sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau),
// with softplus(u) = max(u, 0) + log1p(exp(-|u|)), so that neither end overflows.
__global__ __launch_bounds__(256) void gla_decay_kernel(const float* __restrict__ low, int ld, int rank,
                                                        const float* __restrict__ w2, const float* __restrict__ bias,
                                                        float inv_tau, float* __restrict__ decay, int channels) {
  const int r = blockIdx.x;
  const float* t = low + (size_t)r * ld;
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float z = bias ? bias[c] : 0.f;
    const float* w = w2 + (size_t)c * rank;
    for (int j = 0; j < rank; ++j) z = fmaf(w[j], t[j], z);
    const float u = -z;
    const float sp = fmaxf(u, 0.f) + log1pf(expf(-fabsf(u)));
    decay[(size_t)r * channels + c] = expf(-sp * inv_tau);
  }
}

extern "C" int llmlab_gla_decay(const float* low, int ld, int rows, int rank, const float* w2, const float* bias,
                                float tau, float* decay, int channels, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && rank > 0 && channels > 0 && ld >= rank && tau > 0.f,
                 "gla_decay: bad sizes rows=%d rank=%d channels=%d ld=%d tau=%g", rows, rank, channels, ld, (double)tau);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(gla_decay_kernel, dim3(rows), dim3(256), 0, stream, low, ld, rank, w2, bias, 1.0f / tau, decay,
                     channels);
  LLMLAB_LAUNCH_CHECK("gla_decay");
  return 0;
}

// ------------------------------------------------------------------------ scan
// Block (request b, head h, slab of value columns).  Thread (s, e) keeps the SLICE rows
// s * SLICE .. of column e of the head's state in registers, walks the request's rows of
// this step in order, and leaves its part of o_t in parts[row, h, s, e]; the output kernel
// adds the parts of the slices.  Threads never talk to each other, so a token costs no
// barrier; the loads of a token do not depend on the state, so they run ahead of the sums.
// The state is read from the request's slot before the first row and written back after
// the last.
__global__ __launch_bounds__(1024) void gla_scan_kernel(
    const float* __restrict__ proj, int ld, int off_q, int off_k, int off_v, const float* __restrict__ decay,
    float q_scale, int n_heads, int D, int E, int cols, int slices, float* __restrict__ state,
    const int* __restrict__ q_start, const int* __restrict__ req_rows, float* __restrict__ parts) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * cols + (int)(threadIdx.x % cols);
  const int s = threadIdx.x / cols;
  if (e >= E || s >= slices) return;
  const int d0 = s * SLICE;
  float S[SLICE];
  float* st = state + (((size_t)req_rows[b] * n_heads + h) * D + d0) * E + e;
#pragma unroll
  for (int i = 0; i < SLICE; ++i) S[i] = d0 + i < D ? st[(size_t)i * E] : 0.f;
  const int first = q_start[b], last = q_start[b + 1];
  const bool whole = d0 + SLICE <= D;
  for (int t = first; t < last; ++t) {
    const float* row = proj + (size_t)t * ld;
    const float* qp = row + off_q + h * D + d0;
    const float* kp = row + off_k + h * D + d0;
    const float* ap = decay + ((size_t)t * n_heads + h) * D + d0;
    const float v = row[off_v + h * E + e];
    float acc = 0.f;
    if (whole) {
#pragma unroll
      for (int i = 0; i < SLICE; ++i) {
        S[i] = fmaf(ap[i], S[i], kp[i] * v);
        acc = fmaf(S[i], qp[i] * q_scale, acc);
      }
    } else {
#pragma unroll
      for (int i = 0; i < SLICE; ++i) {
        if (d0 + i < D) {
          S[i] = fmaf(ap[i], S[i], kp[i] * v);
          acc = fmaf(S[i], qp[i] * q_scale, acc);
        }
      }
    }
    parts[(((size_t)t * n_heads + h) * slices + s) * E + e] = acc;
  }
#pragma unroll
  for (int i = 0; i < SLICE; ++i)
    if (d0 + i < D) st[(size_t)i * E] = S[i];
}

extern "C" int llmlab_gla_slices(int D) { return (D + SLICE - 1) / SLICE; }

// proj [rows, ld] float32 holds q at off_q (heads * D), k at off_k, v at off_v (heads * E);
// decay [rows, heads * D]; state [slots, heads, D, E]; parts [rows, heads, slices, E].
extern "C" int llmlab_gla_scan(const float* proj, int ld, int off_q, int off_k, int off_v, const float* decay,
                               float q_scale, int n_heads, int D, int E, float* state, const int* q_start,
                               const int* req_rows, int n_reqs, float* parts, hipStream_t stream) {
  LLMLAB_REQUIRE(n_reqs >= 0 && n_heads > 0 && D > 0 && E > 0, "gla_scan: bad sizes reqs=%d heads=%d D=%d E=%d", n_reqs,
                 n_heads, D, E);
  const int slices = (D + SLICE - 1) / SLICE;
  int cols = E < 64 ? E : 64;
  while (cols > 1 && slices * cols > 1024) cols /= 2;
  LLMLAB_REQUIRE(slices * cols <= 1024, "gla_scan: %d key channels per head are more than a block holds", D);
  LLMLAB_REQUIRE(n_heads <= 65535 && (E + cols - 1) / cols <= 65535, "gla_scan: too many heads or columns");
  if (n_reqs == 0) return 0;
  dim3 grid(n_reqs, n_heads, (E + cols - 1) / cols), block(slices * cols);
  hipLaunchKernelGGL(gla_scan_kernel, grid, block, 0, stream, proj, ld, off_q, off_k, off_v, decay, q_scale, n_heads, D,
                     E, cols, slices, state, q_start, req_rows, parts);
  LLMLAB_LAUNCH_CHECK("gla_scan");
  return 0;
}

// ---------------------------------------------------------------------- output
// Block (row, head): o = sum over slices of parts; y = o / sqrt(mean(o^2) + eps) * w[e]
// (the weight has one entry per value channel, the same for every head); out = T(y *
// silu(gate)), silu(g) = g / (1 + exp(-g)); gate [rows, ld] float32 at column off_g.
template <typename T>
__global__ __launch_bounds__(1024) void gla_output_kernel(const float* __restrict__ parts, int slices, int n_heads, int E,
                                                          const float* __restrict__ w, float eps,
                                                          const float* __restrict__ proj, int ld, int off_g,
                                                          T* __restrict__ out) {
  __shared__ float red[17];
  const int r = blockIdx.x, h = blockIdx.y, e = threadIdx.x;
  float o = 0.f;
  if (e < E) {
    const float* p = parts + (((size_t)r * n_heads + h) * slices) * E + e;
    for (int s = 0; s < slices; ++s) o += p[(size_t)s * E];
  }
  const float ms = block_sum(o * o, red) / (float)E;
  if (e < E) {
    const float g = proj[(size_t)r * ld + off_g + h * E + e];
    const float y = o * (1.0f / sqrtf(ms + eps)) * w[e];
    out[((size_t)r * n_heads + h) * E + e] = from_float<T>(y * (g / (1.0f + expf(-g))));
  }
}

extern "C" int llmlab_gla_output(const float* parts, int rows, int n_heads, int D, int E, const float* w, float eps,
                                 const float* proj, int ld, int off_g, void* out, int dtype, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && n_heads > 0 && n_heads <= 65535 && E > 0 && E <= 1024,
                 "gla_output: bad sizes rows=%d heads=%d E=%d", rows, n_heads, E);
  if (rows == 0) return 0;
  const int slices = (D + SLICE - 1) / SLICE;
  dim3 grid(rows, n_heads), block((E + 63) / 64 * 64);
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(gla_output_kernel<bf16_t>, grid, block, 0, stream, parts, slices, n_heads, E, w, eps, proj, ld,
                       off_g, (bf16_t*)out);
  else
    hipLaunchKernelGGL(gla_output_kernel<float>, grid, block, 0, stream, parts, slices, n_heads, E, w, eps, proj, ld,
                       off_g, (float*)out);
  LLMLAB_LAUNCH_CHECK("gla_output");
  return 0;
}

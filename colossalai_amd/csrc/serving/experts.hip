// Mixture-of-experts serving kernels:
//   grouped_topk_route : sigmoid (or softmax) scores, a selection-only correction, group-limited
//                        top-k with ties to the lower index, chosen scores renormalised (or kept);
//   expert_ffn_gemv    : a small step's chosen experts as two matrix-vector kernels
//                        (up + squared ReLU per (token, expert) pair, then the weighted
//                        down products of a token summed with its base row) — only the
//                        chosen experts' weights are streamed, nothing goes to the host;
//   expert_sort        : stable counting sort of a step's (token, expert) pairs by expert,
//                        one block, for the grouped matrix-core product (expert_gemm.hip);
//   expert_combine     : base + weighted sum of each token's rows of a sorted-by-expert
//                        output.
#include "serving_common.h"

namespace cai {
namespace serving {

// ------------------------------------------------------------------ router
// One wave per token, four tokens per block; every wave runs every barrier (a wave past the
// last token repeats the last token and writes nothing). LDS per wave: scores [E], choice
// scores [E], group worths [groups], picked scores [top].
__global__ __launch_bounds__(256) void grouped_topk_route_kernel(
    int* __restrict__ ids, float* __restrict__ wts, const float* __restrict__ logits, long ld,
    const float* __restrict__ corr, long N, int E, int top, int groups, int keep, int group_top, float eps,
    int softmax, int renorm) {
  extern __shared__ float lds[];
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* sc = lds + (long)wid * (2 * E + groups + top);
  float* ch = sc + E;
  float* worth = ch + E;
  float* pick = worth + groups;
  const long tok = (long)blockIdx.x * 4 + wid;
  const bool live = tok < N;
  const long n = live ? tok : N - 1;
  if (softmax) {  // over all experts, float32: exp(z - max) / sum
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, logits[n * ld + e]);
    mx = wave_reduce_max(mx);
    float sum = 0.0f;
    for (int e = lane; e < E; e += 64) {
      const float w = expf(logits[n * ld + e] - mx);
      sc[e] = w;
      sum += w;
    }
    sum = wave_reduce_sum(sum);
    for (int e = lane; e < E; e += 64) {
      const float s = sc[e] / sum;
      sc[e] = s;
      ch[e] = s + (corr != nullptr ? corr[e] : 0.0f);
    }
  } else {
    for (int e = lane; e < E; e += 64) {
      const float s = sigmoidf_(logits[n * ld + e]);
      sc[e] = s;
      ch[e] = s + (corr != nullptr ? corr[e] : 0.0f);
    }
  }
  __syncthreads();
  if (groups > 1) {
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
      // the group_top largest of the group, taken in (value desc, index asc) order
      float sum = 0.0f, pv = INFINITY;
      int pi = -1;
      for (int t = 0; t < group_top && t < per; ++t) {
        float bv = -INFINITY;
        int bi = -1;
        for (int k = 0; k < per; ++k) {
          const float v = ch[g * per + k];
          const bool after = v < pv || (v == pv && k > pi);   // not yet taken
          if (after && (bi < 0 || v > bv)) { bv = v; bi = k; }
        }
        if (bi < 0) break;
        sum += bv;
        pv = bv;
        pi = bi;
      }
      worth[g] = sum;
    }
    __syncthreads();
    for (int g = lane; g < groups; g += 64) {
      int rank = 0;
      const float mine = worth[g];
      for (int o = 0; o < groups; ++o) rank += (worth[o] > mine || (worth[o] == mine && o < g)) ? 1 : 0;
      if (rank >= keep)
        for (int k = 0; k < per; ++k) ch[g * per + k] = -INFINITY;
    }
    __syncthreads();
  }
  float total = 0.0f;
  for (int t = 0; t < top; ++t) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = ch[e];
      if (v > bv) { bv = v; bi = e; }   // ascending e: the first of equal values stays
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off);
      const int oi = __shfl_xor(bi, off);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi >= E) bi = 0;  // nothing left to choose from (the host rules this out)
    if (lane == 0) {
      pick[t] = sc[bi];
      ch[bi] = -INFINITY;
      if (live) ids[tok * top + t] = bi;
    }
    total += sc[bi];
    __syncthreads();
  }
  if (live)
    for (int t = lane; t < top; t += 64) wts[tok * top + t] = renorm ? pick[t] / (total + eps) : pick[t];
}

std::vector<at::Tensor> grouped_topk_route(at::Tensor logits, c10::optional<at::Tensor> correction, int64_t top,
                                           int64_t group_count, int64_t group_keep, int64_t group_top,
                                           double renorm_eps, int64_t score_fn, bool renorm) {
  TORCH_CHECK(logits.is_cuda() && is_f32(logits) && logits.dim() == 2 && logits.stride(1) == 1,
              "router logits must be float32 [N, E] with unit inner stride");
  TORCH_CHECK(score_fn == 0 || score_fn == 1, "score function: 0 = sigmoid, 1 = softmax");
  const long N = logits.size(0);
  const int E = (int)logits.size(1);
  TORCH_CHECK(group_count >= 1 && E % group_count == 0 && group_keep >= 1 && group_keep <= group_count && group_top >= 1);
  TORCH_CHECK(top >= 1 && top <= (E / group_count) * group_keep, "more experts to choose than the kept groups hold");
  at::Tensor corr;
  const float* corrp = nullptr;
  if (correction.has_value()) {
    corr = f32c(*correction);
    TORCH_CHECK(corr.numel() == E && corr.is_cuda());
    corrp = corr.data_ptr<float>();
  }
  at::Tensor ids = at::empty({N, top}, logits.options().dtype(at::kInt));
  at::Tensor wts = at::empty({N, top}, logits.options());
  if (N == 0) return {ids, wts};
  const size_t smem = (size_t)4 * (2 * E + group_count + top) * sizeof(float);
  TORCH_CHECK(smem <= 64 * 1024, "too many experts for the router kernel");
  hipLaunchKernelGGL(grouped_topk_route_kernel, dim3((unsigned)((N + 3) / 4)), dim3(256), smem, stream(),
                     ids.data_ptr<int>(), wts.data_ptr<float>(), logits.data_ptr<float>(), (long)logits.stride(0), corrp, N,
                     E, (int)top, (int)group_count, (int)group_keep, (int)group_top, (float)renorm_eps, (int)score_fn,
                     renorm ? 1 : 0);
  HIP_CHECK_LAST();
  return {ids, wts};
}

// ------------------------------------------------------- matrix-vector path
constexpr int GEMV_R = 4;  // output rows per wave: the input slice a lane holds is reused for each

// dot products of R consecutive rows of `w` (row length K, first row `row0`, `rows` rows exist)
// with the vector `x`; every lane holds partial sums over its slices of K.
template <typename T, int R>
DEV_INLINE void rows_dot(const T* __restrict__ x, const T* __restrict__ w, int K, int row0, int rows, int lane, int vec,
                         float scale, float* acc) {
  if (vec) {
    for (int c = lane * 8; c < K; c += 512) {
      float xv[8];
      load8(x + c, xv);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (row0 + r < rows) {
          float wv[8];
          load8(w + (long)(row0 + r) * K + c, wv);
          float d = 0.0f;
#pragma unroll
          for (int i = 0; i < 8; ++i) d += xv[i] * wv[i];
          acc[r] += scale * d;
        }
      }
    }
  } else {
    for (int c = lane; c < K; c += 64) {
      const float xv = ldf(x + c);
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (row0 + r < rows) acc[r] += scale * xv * ldf(w + (long)(row0 + r) * K + c);
    }
  }
}

// block = (pair, chunk of 4 * R hidden rows): hidden[p, f] = relu(up_e[f, :] . h[n, :])^2, or, GATED (the
// expert's matrix stacks F gate rows on F up rows): hidden[p, f] = silu(gate_e[f, :] . h) * (up_e[f, :] . h)
template <typename T, bool GATED>
__global__ __launch_bounds__(256) void expert_up_gemv_kernel(
    T* __restrict__ hidden, const T* __restrict__ h, const T* __restrict__ w_up, const int* __restrict__ ids, int top,
    int E, int F, int W, int vec) {
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long p = blockIdx.x;
  const long n = p / top;
  const int e = ids[p];
  const int row0 = (blockIdx.y * 4 + wid) * GEMV_R;
  if (row0 >= F || e < 0 || e >= E) return;
  float acc[GEMV_R];
#pragma unroll
  for (int r = 0; r < GEMV_R; ++r) acc[r] = 0.0f;
  if constexpr (GATED) {
    float up[GEMV_R];
#pragma unroll
    for (int r = 0; r < GEMV_R; ++r) up[r] = 0.0f;
    const T* we = w_up + (long)e * 2 * F * W;
    rows_dot<T, GEMV_R>(h + n * W, we, W, row0, F, lane, vec, 1.0f, acc);
    rows_dot<T, GEMV_R>(h + n * W, we + (long)F * W, W, row0, F, lane, vec, 1.0f, up);
#pragma unroll
    for (int r = 0; r < GEMV_R; ++r) {
      const float g = wave_reduce_sum(acc[r]), u = wave_reduce_sum(up[r]);
      if (lane == 0 && row0 + r < F) stf(hidden + p * F + row0 + r, g * sigmoidf_(g) * u);
    }
  } else {
    rows_dot<T, GEMV_R>(h + n * W, w_up + (long)e * F * W, W, row0, F, lane, vec, 1.0f, acc);
#pragma unroll
    for (int r = 0; r < GEMV_R; ++r) {
      const float v = fmaxf(wave_reduce_sum(acc[r]), 0.0f);
      if (lane == 0 && row0 + r < F) stf(hidden + p * F + row0 + r, v * v);
    }
  }
}

// block = (token, chunk of 4 * R output rows): out[n, w] = base[n, w] + sum_j weight_j down_{e_j}[w, :] . hidden[n, j, :];
// with base_gate the base row is first multiplied by sigmoid(base_gate[n])
template <typename T, typename TB>
__global__ __launch_bounds__(256) void expert_down_gemv_kernel(
    float* __restrict__ out, const T* __restrict__ hidden, const T* __restrict__ w_down, const int* __restrict__ ids,
    const float* __restrict__ weights, const TB* __restrict__ base, const float* __restrict__ base_gate, long bgs,
    int top, int E, int F, int W, int vec, const T* __restrict__ ident) {
  // ident (the tokens' input rows [N, W], or null): an id >= E then names an identity expert and adds weight * ident[n]
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long n = blockIdx.x;
  const int row0 = (blockIdx.y * 4 + wid) * GEMV_R;
  if (row0 >= W) return;
  float idw = 0.0f;
  const float bscale = base_gate != nullptr ? sigmoidf_(base_gate[n * bgs]) : 1.0f;
  float acc[GEMV_R];
#pragma unroll
  for (int r = 0; r < GEMV_R; ++r) acc[r] = 0.0f;
  for (int j = 0; j < top; ++j) {
    const int e = ids[n * top + j];
    if (e >= E && ident != nullptr) idw += weights[n * top + j];
    if (e < 0 || e >= E) continue;
    rows_dot<T, GEMV_R>(hidden + (n * top + j) * F, w_down + (long)e * W * F, F, row0, W, lane, vec,
                        weights[n * top + j], acc);
  }
#pragma unroll
  for (int r = 0; r < GEMV_R; ++r) {
    const float v = wave_reduce_sum(acc[r]);
    if (lane == 0 && row0 + r < W) {
      const long at = n * W + row0 + r;
      out[at] = (base != nullptr ? ldf(base + at) * bscale : 0.0f) + v + (ident != nullptr ? idw * ldf(ident + at) : 0.0f);
    }
  }
}

static void check_experts(const at::Tensor& h, const at::Tensor& w_up, const at::Tensor& w_down, const at::Tensor& ids,
                          const at::Tensor& weights, const c10::optional<at::Tensor>& base, bool gated = false) {
  check_act(h, "h");
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous(), "h must be contiguous [N, W]");
  TORCH_CHECK(w_up.dim() == 3 && w_down.dim() == 3 && w_up.is_contiguous() && w_down.is_contiguous() && w_up.is_cuda() &&
              w_down.is_cuda(), "expert matrices must be contiguous [E, out, in] GPU tensors");
  TORCH_CHECK(w_up.scalar_type() == h.scalar_type() && w_down.scalar_type() == h.scalar_type(),
              "experts and their input share one dtype");
  TORCH_CHECK(w_up.size(2) == h.size(1) && w_down.size(0) == w_up.size(0) && w_down.size(1) == h.size(1) &&
              w_down.size(2) * (gated ? 2 : 1) == w_up.size(1),
              "expert matrix shapes do not fit [E, F, W] (gated: [E, 2F, W]) / [E, W, F]");
  check_i32(ids, "ids");
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == h.size(0));
  TORCH_CHECK(weights.is_cuda() && is_f32(weights) && weights.is_contiguous() && weights.sizes() == ids.sizes(),
              "weights must be contiguous float32 of the ids' shape");
  if (base.has_value()) {
    check_act(*base, "base");
    TORCH_CHECK(base->is_contiguous() && base->sizes() == h.sizes(), "base must be contiguous and of h's shape");
  }
}

// logits of the base row's sigmoid gate: float32, one per token, any stride
static const float* base_gate_ptr(const c10::optional<at::Tensor>& base_gate, const c10::optional<at::Tensor>& base,
                                  long N, long* stride) {
  *stride = 0;
  if (!base_gate.has_value()) return nullptr;
  TORCH_CHECK(base.has_value(), "a base gate needs a base");
  TORCH_CHECK(base_gate->is_cuda() && is_f32(*base_gate) && base_gate->numel() == N && base_gate->dim() <= 2 &&
              (base_gate->dim() < 2 || base_gate->size(1) == 1), "base_gate must be float32 [N] logits");
  *stride = N > 0 ? base_gate->stride(0) : 0;
  return base_gate->data_ptr<float>();
}

at::Tensor expert_ffn_gemv(at::Tensor h, at::Tensor w_up, at::Tensor w_down, at::Tensor ids, at::Tensor weights,
                           c10::optional<at::Tensor> base, c10::optional<at::Tensor> base_gate, bool gated,
                           bool identity) {
  check_experts(h, w_up, w_down, ids, weights, base, gated);
  long bgs = 0;
  const float* bgp = base_gate_ptr(base_gate, base, h.size(0), &bgs);
  const long N = h.size(0);
  const int W = (int)h.size(1), E = (int)w_up.size(0), F = (int)w_down.size(2), top = (int)ids.size(1);
  at::Tensor out = at::empty({N, W}, h.options().dtype(at::kFloat));
  if (N == 0) return out;
  at::Tensor hidden = at::empty({N * top, F}, h.options());
  const int rows_per_block = 4 * GEMV_R;
  // 8-element slices need rows that start 16 bytes (bfloat16) / 32 bytes (float32) apart
  auto aligned = [](const at::Tensor& t) { return reinterpret_cast<uintptr_t>(t.data_ptr()) % 32 == 0; };
  const int vec_up = (W % 8 == 0 && aligned(h) && aligned(w_up)) ? 1 : 0;
  const int vec_down = (F % 8 == 0 && aligned(hidden) && aligned(w_down)) ? 1 : 0;
  SERVING_DISPATCH_ACT(h, T, {
    const dim3 up_grid((unsigned)(N * top), (unsigned)((F + rows_per_block - 1) / rows_per_block));
    if (gated)
      hipLaunchKernelGGL((expert_up_gemv_kernel<T, true>), up_grid, dim3(256), 0, stream(), ptr<T>(hidden), ptr<T>(h),
                         ptr<T>(w_up), ids.data_ptr<int>(), top, E, F, W, vec_up);
    else
      hipLaunchKernelGGL((expert_up_gemv_kernel<T, false>), up_grid, dim3(256), 0, stream(), ptr<T>(hidden), ptr<T>(h),
                         ptr<T>(w_up), ids.data_ptr<int>(), top, E, F, W, vec_up);
    const T* idp = identity ? ptr<T>(h) : (const T*)nullptr;
    const dim3 grid((unsigned)N, (unsigned)((W + rows_per_block - 1) / rows_per_block));
    if (base.has_value()) {
      SERVING_DISPATCH_ACT(*base, TB, {
        hipLaunchKernelGGL((expert_down_gemv_kernel<T, TB>), grid, dim3(256), 0, stream(), out.data_ptr<float>(),
                           ptr<T>(hidden), ptr<T>(w_down), ids.data_ptr<int>(), weights.data_ptr<float>(), ptr<TB>(*base),
                           bgp, bgs, top, E, F, W, vec_down, idp);
      });
    } else {
      hipLaunchKernelGGL((expert_down_gemv_kernel<T, float>), grid, dim3(256), 0, stream(), out.data_ptr<float>(),
                         ptr<T>(hidden), ptr<T>(w_down), ids.data_ptr<int>(), weights.data_ptr<float>(),
                         (const float*)nullptr, (const float*)nullptr, 0L, top, E, F, W, vec_down, idp);
    }
  });
  HIP_CHECK_LAST();
  return out;
}

// ------------------------------------------------------------------ combine
// out[n, w] = base[n, w] (* sigmoid(base_gate[n])) + sum_j weights[n, j] * y[inv[n, j], w], slots in order, float32.
// VEC: eight columns per thread (W a multiple of 8, 32-byte aligned operands).
template <typename T, typename TB, bool VEC>
__global__ __launch_bounds__(256) void expert_combine_kernel(
    float* __restrict__ out, const T* __restrict__ y, const int* __restrict__ inv, const float* __restrict__ weights,
    const TB* __restrict__ base, const float* __restrict__ base_gate, long bgs, int top, int W, long rows,
    const int* __restrict__ ids, int E, const T* __restrict__ ident) {
  // ident (the tokens' input rows [N, W], with ids [N, top] and the number E of real experts; or null): a pair whose
  // id is >= E names an identity expert, has no row in y and adds weight * ident[n]
  const long n = blockIdx.x;
  const float bscale = base_gate != nullptr ? sigmoidf_(base_gate[n * bgs]) : 1.0f;
  float idw = 0.0f;
  if (ident != nullptr)
    for (int j = 0; j < top; ++j)
      if (ids[n * top + j] >= E) idw += weights[n * top + j];
  if (VEC) {
    for (int w = threadIdx.x * 8; w < W; w += blockDim.x * 8) {
      float acc[8];
      if (base != nullptr) {
        load8(base + n * W + w, acc);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] *= bscale;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
      }
      if (ident != nullptr) {
        float v[8];
        load8(ident + n * W + w, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += idw * v[e];
      }
      for (int j = 0; j < top; ++j) {
        const long r = inv[n * top + j];
        if (r >= 0 && r < rows && (ident == nullptr || ids[n * top + j] < E)) {
          float v[8];
          load8(y + r * W + w, v);
          const float wj = weights[n * top + j];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] += wj * v[e];
        }
      }
      store8(out + n * W + w, acc);
    }
  } else {
    for (int w = threadIdx.x; w < W; w += blockDim.x) {
      float acc = base != nullptr ? ldf(base + n * W + w) * bscale : 0.0f;
      if (ident != nullptr) acc += idw * ldf(ident + n * W + w);
      for (int j = 0; j < top; ++j) {
        const long r = inv[n * top + j];
        if (r >= 0 && r < rows && (ident == nullptr || ids[n * top + j] < E))
          acc += weights[n * top + j] * ldf(y + r * W + w);
      }
      out[n * W + w] = acc;
    }
  }
}

at::Tensor expert_combine(at::Tensor y, at::Tensor inv, at::Tensor weights, c10::optional<at::Tensor> base,
                          c10::optional<at::Tensor> base_gate, c10::optional<at::Tensor> ids, int64_t num_experts,
                          c10::optional<at::Tensor> identity_rows) {
  check_act(y, "y");
  check_i32(inv, "inv");
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() && inv.dim() == 2 && inv.size(0) * inv.size(1) == y.size(0),
              "y must be contiguous [N * top, W] and inv [N, top]");
  TORCH_CHECK(weights.is_cuda() && is_f32(weights) && weights.is_contiguous() && weights.sizes() == inv.sizes());
  const long N = inv.size(0);
  const int top = (int)inv.size(1), W = (int)y.size(1);
  if (base.has_value()) {
    check_act(*base, "base");
    TORCH_CHECK(base->is_contiguous() && base->dim() == 2 && base->size(0) == N && base->size(1) == W);
  }
  long bgs = 0;
  const float* bgp = base_gate_ptr(base_gate, base, N, &bgs);
  const int* idsp = nullptr;
  const void* identp = nullptr;
  if (identity_rows.has_value()) {
    TORCH_CHECK(ids.has_value(), "identity experts are told from real ones by their ids");
    check_i32(*ids, "ids");
    TORCH_CHECK(ids->sizes() == inv.sizes() && identity_rows->is_cuda() && identity_rows->is_contiguous() &&
                identity_rows->dim() == 2 && identity_rows->size(0) == N && identity_rows->size(1) == W &&
                identity_rows->scalar_type() == y.scalar_type(), "identity rows must be contiguous [N, W] of y's type");
    idsp = ids->data_ptr<int>();
    identp = identity_rows->data_ptr();
  }
  const int E = (int)num_experts;
  at::Tensor out = at::empty({N, W}, y.options().dtype(at::kFloat));
  if (N == 0) return out;
  auto al32 = [](const at::Tensor& t) { return reinterpret_cast<uintptr_t>(t.data_ptr()) % 32 == 0; };
  const bool vec = W % 8 == 0 && al32(y) && al32(out) && (!base.has_value() || al32(*base)) &&
                   (!identity_rows.has_value() || al32(*identity_rows));
  const float* nobase = nullptr;
#define COMBINE_LAUNCH(TB_, bp)                                                                                       \
  do {                                                                                                                \
    if (vec)                                                                                                          \
      hipLaunchKernelGGL((expert_combine_kernel<T, TB_, true>), dim3((unsigned)N), dim3(256), 0, stream(),           \
                         out.data_ptr<float>(), ptr<T>(y), inv.data_ptr<int>(), weights.data_ptr<float>(), bp, bgp,  \
                         bgs, top, W, (long)y.size(0), idsp, E, (const T*)identp);                                    \
    else                                                                                                              \
      hipLaunchKernelGGL((expert_combine_kernel<T, TB_, false>), dim3((unsigned)N), dim3(256), 0, stream(),          \
                         out.data_ptr<float>(), ptr<T>(y), inv.data_ptr<int>(), weights.data_ptr<float>(), bp, bgp,  \
                         bgs, top, W, (long)y.size(0), idsp, E, (const T*)identp);                                    \
  } while (0)
  SERVING_DISPATCH_ACT(y, T, {
    if (base.has_value()) {
      SERVING_DISPATCH_ACT(*base, TB, { COMBINE_LAUNCH(TB, ptr<TB>(*base)); });
    } else {
      COMBINE_LAUNCH(float, nobase);
    }
  });
#undef COMBINE_LAUNCH
  HIP_CHECK_LAST();
  return out;
}

// ------------------------------------------------------------------- sort
// Stable counting sort of the (token, expert) pairs of a step by expert, one block, the ids held in LDS:
//   offsets[e] .. offsets[e + 1] = sorted rows of expert e; src[r] = token of sorted row r; inv[p] = sorted row of
//   pair p. Each wave takes every nw-th expert and walks the pairs 64 at a time (ballot + prefix count), so rows of
//   one expert keep the order of their pairs and the result does not depend on timing.
constexpr int SORT_MAX_PAIRS = 8192;

__global__ __launch_bounds__(1024) void expert_sort_kernel(
    int* __restrict__ offsets, int* __restrict__ src, int* __restrict__ inv, const int* __restrict__ ids, int P, int E,
    int top) {
  extern __shared__ int sort_lds[];
  int* held = sort_lds;          // [P]
  int* count = sort_lds + P;     // [E + 1]
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  for (int p = threadIdx.x; p < P; p += blockDim.x) held[p] = ids[p];
  __syncthreads();
  for (int e = wid; e < E; e += nw) {
    int n = 0;
    for (int p0 = 0; p0 < P; p0 += 64) {
      const bool hit = p0 + lane < P && held[p0 + lane] == e;
      n += __popcll(__ballot(hit));
    }
    if (lane == 0) count[e] = n;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      const int n = count[e];
      count[e] = run;
      offsets[e] = run;
      run += n;
    }
    count[E] = run;
    offsets[E] = run;
  }
  __syncthreads();
  for (int e = wid; e < E; e += nw) {
    int at = count[e];
    for (int p0 = 0; p0 < P; p0 += 64) {
      const int p = p0 + lane;
      const bool hit = p < P && held[p] == e;
      const unsigned long long mask = __ballot(hit);
      if (hit) {
        const int r = at + __popcll(mask & ((1ull << lane) - 1ull));
        src[r] = p / top;
        inv[p] = r;
      }
      at += __popcll(mask);
    }
  }
}

std::vector<at::Tensor> expert_sort(at::Tensor ids, int64_t num_experts) {
  check_i32(ids, "ids");
  TORCH_CHECK(ids.dim() == 2, "ids must be [N, top]");
  const int P = (int)ids.numel(), top = (int)ids.size(1), E = (int)num_experts;
  TORCH_CHECK(P <= SORT_MAX_PAIRS, "too many pairs for the one-block sort");
  TORCH_CHECK(E >= 1 && (size_t)(P + E + 1) * sizeof(int) <= 64 * 1024);
  at::Tensor offsets = at::empty({E + 1}, ids.options());
  at::Tensor src = at::empty({P}, ids.options());
  at::Tensor inv = at::empty({ids.size(0), ids.size(1)}, ids.options());
  if (P == 0) {
    offsets.zero_();
    return {offsets, src, inv};
  }
  // an id outside [0, E) would leave rows of src / inv unwritten: the router never produces one
  hipLaunchKernelGGL(expert_sort_kernel, dim3(1), dim3(1024), (size_t)(P + E + 1) * sizeof(int), stream(),
                     offsets.data_ptr<int>(), src.data_ptr<int>(), inv.data_ptr<int>(), ids.data_ptr<int>(), P, E, top);
  HIP_CHECK_LAST();
  return {offsets, src, inv};
}

}  // namespace serving
}  // namespace cai

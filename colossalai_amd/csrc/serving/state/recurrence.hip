// Matrix-state linear recurrences over a ragged batch (float32 state).
//
// Each head keeps S [D, Dv] per state slot. Columns of S (value channels) are
// independent in both update rules, so a value channel is owned by P adjacent
// lanes that split the D rows between them (8 or 16 rows per lane, in
// registers); the two dot products per token are reduced across those P lanes.
// A wave walks its sequence's new tokens in order, so prompt portions and
// single decode tokens are the same code, and the state only touches memory at
// the start and the end of a portion: cutting a prompt differently cannot
// change a result.
//
//   delta: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q
//   tied : S <- diag(f) S + (1 - f) v^T;                          o = S^T q
//   ssd  : S <- a S + (dt v) k^T  (one decay a per head and token);   o = S^T q + D_skip v
//
// A prologue kernel turns the raw projections into float32 operands once per
// token (unit-length q/k, decay from its logits, gates), so the sequential
// loop holds no transcendental.
#include "../serving_common.h"

namespace cai {
namespace serving {


// ------------------------------------------------------------------ prologue
// One block per token. q/k [N, G, D] row-strided; dt [N, H*D] row-strided.
// T: type of q/k (the convolution's output), TL: type of the gate and decay logits (projections).
template <typename T, typename TL>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ dec, float* __restrict__ beta,
    const T* __restrict__ q, long qs, const T* __restrict__ k, long ks, const TL* __restrict__ bl, long bs,
    const TL* __restrict__ dt, long ds, const float* __restrict__ A_log, const float* __restrict__ dt_bias, int G, int H,
    int D, float unit_eps, float q_scale) {
  const long n = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int u = wid; u < 2 * G; u += nw) {
    const bool isq = u < G;
    const int g = isq ? u : u - G;
    const T* src = (isq ? q + n * qs : k + n * ks) + (long)g * D;
    float ssq = 0.0f;
    for (int i = lane; i < D; i += 64) {
      const float v = ldf(src + i);
      ssq += v * v;
    }
    ssq = wave_reduce_sum(ssq);
    const float inv = (1.0f / sqrtf(ssq + unit_eps)) * (isq ? q_scale : 1.0f);
    float* dst = (isq ? qn : kn) + (n * G + g) * (long)D;
    for (int i = lane; i < D; i += 64) dst[i] = ldf(src + i) * inv;
  }
  const int HD = H * D;
  for (int i = threadIdx.x; i < HD; i += blockDim.x) {
    const float a = expf(A_log[i / D]);
    dec[n * HD + i] = expf(-a * softplusf_(ldf(dt + n * ds + i) + dt_bias[i]));
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) beta[n * H + h] = sigmoidf_(ldf(bl + n * bs + h));
}

template <typename T>
__global__ __launch_bounds__(256) void tied_prepare_kernel(
    float* __restrict__ qa, float* __restrict__ f, const T* __restrict__ q, long qs, const T* __restrict__ fl, long fs,
    const float* __restrict__ f_bias, const float* __restrict__ lower, int HD) {
  const long n = blockIdx.x;
  for (int i = threadIdx.x; i < HD; i += blockDim.x) {
    const float qv = ldf(q + n * qs + i);
    qa[n * HD + i] = qv * sigmoidf_(qv);
    const float lo = lower[i];
    f[n * HD + i] = lo + (1.0f - lo) * sigmoidf_(ldf(fl + n * fs + i) + f_bias[i]);
  }
}

// scal[n, h] = (a, dt): dt = softplus(dt_raw + dt_bias) (no clamp), a = exp(-exp(A_log) dt).
template <typename TL>
__global__ __launch_bounds__(256) void ssd_prepare_kernel(float* __restrict__ scal, const TL* __restrict__ dt, long ds,
                                                          const float* __restrict__ A_log,
                                                          const float* __restrict__ dt_bias, long N, int H) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * H) return;
  const long n = i / H;
  const int h = (int)(i % H);
  const float d = softplusf_(ldf(dt + n * ds + h) + dt_bias[h]);
  scal[2 * i] = expf(-expf(A_log[h]) * d);
  scal[2 * i + 1] = d;
}

// ---------------------------------------------------------------------- scan
// Sum over the P adjacent lanes that share a value channel, on the DPP path
// (no LDS traffic): xor 1 and 2 inside a quad, then the half-row and row
// mirrors pair up quads and octets whose lanes already hold equal sums.
template <int CTRL>
DEV_INLINE float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
  return v + __builtin_bit_cast(float, moved);
}

template <int P>
DEV_INLINE float reduce_p(float v) {
  if (P >= 2) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  if (P >= 4) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  if (P >= 8) v = dpp_add<0x141>(v);  // row_half_mirror
  if (P >= 16) v = dpp_add<0x140>(v); // row_mirror
  return v;
}

// grid (ceil(Dv / (4 * 64 / P)), H, B), four waves per block; lane = (value channel, row slice p).
// q, k: [N, Hq, D] float (Hq = H / rep); gate: [N, H, D] float (decay g or forget f).
// The block stages CT tokens' operand rows of its head in LDS (double-buffered: the next chunk's
// global loads are in flight while this chunk's tokens are stepped through).
// A lane can carry NC value channels that share the operand reads. Measured on a 4096-token
// prompt (D = 128): NC = 2 is 1.5x slower per layer than NC = 1 - a single long sequence is
// bound by the instructions a wave issues per token, not by latencies that a second chain could
// hide - so NC stays 1.
// MODE: 0 = tied, 1 = delta, 2 = ssd. In ssd mode the operand rows are q and k (no per-channel gate) with the
// token stride qk_ts, `beta` holds two scalars per (token, head), the decay a and the step dt, and `skip` [H] the
// weight of the direct path.
constexpr int SCAN_TIED = 0, SCAN_DELTA = 1, SCAN_SSD = 2;

template <int P, int DPL, int MODE, typename TV>
__global__ __launch_bounds__(256) void matrix_state_scan_kernel(
    float* __restrict__ out, const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ gate,
    const float* __restrict__ beta, const TV* __restrict__ v, long vs, float* __restrict__ state, long ss,
    const int* __restrict__ cu, const int* __restrict__ start, const int* __restrict__ slots, int H, int rep, int D,
    int Dv, long qk_ts, int vec_ok, const float* __restrict__ skip) {
  constexpr bool DELTA = MODE == SCAN_DELTA, SSD = MODE == SCAN_SSD;
  constexpr int Dp = P * DPL;                 // padded key size
  constexpr int CT = Dp > 128 ? 8 : 16;       // tokens per staged chunk
  constexpr int NOPS = DELTA ? 3 : 2;         // q, (k,) gate; ssd: q, k
  constexpr int NB = SSD ? 2 : 1;             // scalars per (token, head)
  constexpr int NC = 1;                       // value channels per lane
  constexpr int CPW = 4 * 64 / P;             // lanes groups (one channel each) per block
  constexpr int CPB = CPW * NC;               // value channels per block
  constexpr int OPF = CT * NOPS * Dp;         // operand floats per chunk
  constexpr int R_V = (CT * CPB + 255) / 256;
  extern __shared__ __align__(16) float lds[];
  float* ops_buf = lds;                       // [2][CT][NOPS][Dp]
  float* v_buf = lds + 2 * OPF;               // [2][CT][CPB]
  float* b_buf = v_buf + 2 * CT * CPB;        // [2][CT][NB]

  const int b = blockIdx.z, h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int p = lane % P;
  const int cl = wid * (64 / P) + lane / P;   // channel inside the block
  int c[NC], cc[NC];
  bool live[NC];
#pragma unroll
  for (int x = 0; x < NC; ++x) {
    c[x] = blockIdx.x * CPB + x * CPW + cl;
    live[x] = c[x] < Dv;
    cc[x] = live[x] ? c[x] : Dv - 1;
  }
  const int d0 = p * DPL;
  const int Hq = H / rep, hq = h / rep;
  const int t0 = cu[b], t1 = cu[b + 1];
  float* Sg = state + (long)slots[b] * ss + (long)h * D * Dv;

  float S[NC][DPL];
  const bool fresh = start[b] == 0;
#pragma unroll
  for (int x = 0; x < NC; ++x)
#pragma unroll
    for (int j = 0; j < DPL; ++j) S[x][j] = (!fresh && d0 + j < D) ? Sg[(long)(d0 + j) * Dv + cc[x]] : 0.0f;

  // operand rows move as float4: a chunk is CT * NOPS rows of Dp / 4 float4 each
  constexpr int RF4 = Dp / 4, OPF4 = CT * NOPS * RF4, R_OP4 = (OPF4 + 255) / 256;
  float4v r_op[R_OP4];
  float r_v[R_V], r_b = 0.0f;
  const bool rows_vec = (D % 4) == 0 && vec_ok;
  const float* q_head = q + (long)hq * D;
  const float* k_head = (DELTA || SSD) ? k + (long)hq * D : nullptr;
  const float* g_head = SSD ? nullptr : gate + (long)h * D;
  const long qk_stride = SSD ? qk_ts : (long)Hq * D, g_stride = (long)H * D;
  const float dskip = SSD ? skip[h] : 0.0f;
  auto fetch = [&](int tb) {  // chunk starting at token tb -> registers
#pragma unroll
    for (int r = 0; r < R_OP4; ++r) {
      const int i = tid + 256 * r;
      const int rowi = i / RF4, f4 = i % RF4;
      const int tok = rowi / NOPS, op = rowi % NOPS;
      const int t = tb + tok, d = f4 * 4;
      const bool is_gate = !SSD && op == NOPS - 1;
      const float fill = is_gate ? 1.0f : 0.0f;
      float4v val = {fill, fill, fill, fill};
      if (i < OPF4 && t < t1 && d < D) {
        const float* src = is_gate ? g_head + t * g_stride : ((op == 0) ? q_head : k_head) + t * qk_stride;
        if (rows_vec) {
          val = *reinterpret_cast<const float4v*>(src + d);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (d + e < D) val[e] = src[d + e];
        }
      }
      r_op[r] = val;
    }
#pragma unroll
    for (int r = 0; r < R_V; ++r) {
      const int i = tid + 256 * r;
      const int tok = i / CPB, ch = min((int)(blockIdx.x * CPB + i % CPB), Dv - 1);
      const int t = tb + tok;
      r_v[r] = (i < CT * CPB && t < t1) ? ldf(v + (long)t * vs + (long)h * Dv + ch) : 0.0f;
    }
    if (DELTA) r_b = (tid < CT && tb + tid < t1) ? beta[(long)(tb + tid) * H + h] : 0.0f;
    if (SSD) r_b = (tid < 2 * CT && tb + tid / 2 < t1) ? beta[((long)(tb + tid / 2) * H + h) * 2 + (tid & 1)] : 0.0f;
  };
  auto stash = [&](int buf) {  // registers -> LDS buffer ([CT][NOPS][Dp], the order the rows were fetched in)
#pragma unroll
    for (int r = 0; r < R_OP4; ++r) {
      const int i = tid + 256 * r;
      if (i < OPF4) *reinterpret_cast<float4v*>(ops_buf + buf * OPF + i * 4) = r_op[r];
    }
#pragma unroll
    for (int r = 0; r < R_V; ++r) {
      const int i = tid + 256 * r;
      if (i < CT * CPB) v_buf[buf * CT * CPB + i] = r_v[r];
    }
    if ((DELTA || SSD) && tid < NB * CT) b_buf[buf * NB * CT + tid] = r_b;
  };

  fetch(t0);
  stash(0);
  __syncthreads();
  int buf = 0;
  for (int tb = t0; tb < t1; tb += CT, buf ^= 1) {
    const bool more = tb + CT < t1;
    if (more) fetch(tb + CT);
    const int cnt = min(CT, t1 - tb);
    for (int tt = 0; tt < cnt; ++tt) {
      const float* row = ops_buf + buf * OPF + tt * NOPS * Dp + d0;
      float qc[DPL], kc[DPL], gc[DPL];
#pragma unroll
      for (int j = 0; j < DPL; j += 4) {
        const float4v a = *reinterpret_cast<const float4v*>(row + j);
        qc[j] = a[0]; qc[j + 1] = a[1]; qc[j + 2] = a[2]; qc[j + 3] = a[3];
        if (DELTA || SSD) {
          const float4v kk = *reinterpret_cast<const float4v*>(row + Dp + j);
          kc[j] = kk[0]; kc[j + 1] = kk[1]; kc[j + 2] = kk[2]; kc[j + 3] = kk[3];
        }
        if (!SSD) {
          const float4v gg = *reinterpret_cast<const float4v*>(row + (NOPS - 1) * Dp + j);
          gc[j] = gg[0]; gc[j + 1] = gg[1]; gc[j + 2] = gg[2]; gc[j + 3] = gg[3];
        }
      }
      const float bc = (DELTA || SSD) ? b_buf[(buf * CT + tt) * NB] : 0.0f;         // delta: beta; ssd: the decay a
      const float dtc = SSD ? b_buf[(buf * CT + tt) * NB + 1] : 0.0f;               // ssd: the step dt
#pragma unroll
      for (int x = 0; x < NC; ++x) {
        const float vc = v_buf[buf * CT * CPB + tt * CPB + x * CPW + cl];
        float oa = 0.0f, ob = 0.0f;  // two chains per sum: half the dependent depth
        if (DELTA) {
          float da = 0.0f, db = 0.0f;
#pragma unroll
          for (int j = 0; j < DPL; j += 2) {
            S[x][j] *= gc[j];
            S[x][j + 1] *= gc[j + 1];
            da += S[x][j] * kc[j];
            db += S[x][j + 1] * kc[j + 1];
          }
          const float dot = reduce_p<P>(da + db);
          const float u = bc * (vc - dot);
#pragma unroll
          for (int j = 0; j < DPL; j += 2) {
            S[x][j] += kc[j] * u;
            S[x][j + 1] += kc[j + 1] * u;
            oa += S[x][j] * qc[j];
            ob += S[x][j + 1] * qc[j + 1];
          }
        } else if (SSD) {
          const float xv = dtc * vc;
#pragma unroll
          for (int j = 0; j < DPL; j += 2) {
            S[x][j] = bc * S[x][j] + kc[j] * xv;
            S[x][j + 1] = bc * S[x][j + 1] + kc[j + 1] * xv;
            oa += S[x][j] * qc[j];
            ob += S[x][j + 1] * qc[j + 1];
          }
        } else {
#pragma unroll
          for (int j = 0; j < DPL; j += 2) {
            S[x][j] = gc[j] * S[x][j] + (1.0f - gc[j]) * vc;
            S[x][j + 1] = gc[j + 1] * S[x][j + 1] + (1.0f - gc[j + 1]) * vc;
            oa += S[x][j] * qc[j];
            ob += S[x][j + 1] * qc[j + 1];
          }
        }
        const float o = reduce_p<P>(oa + ob) + dskip * vc;
        if (p == 0 && live[x]) out[((long)(tb + tt) * H + h) * Dv + c[x]] = o;
      }
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int x = 0; x < NC; ++x)
    if (live[x]) {
#pragma unroll
      for (int j = 0; j < DPL; ++j)
        if (d0 + j < D) Sg[(long)(d0 + j) * Dv + c[x]] = S[x][j];
    }
}

template <int MODE, typename TV>
static void launch_scan(float* out, const float* q, const float* k, const float* gate, const float* beta, const TV* v,
                        long vs, float* state, long ss, const int* cu, const int* start, const int* slots, int B,
                        int H, int rep, int D, int Dv, long qk_ts = 0, int vec_ok = 1, const float* skip = nullptr,
                        bool short_step = false) {
  constexpr bool DELTA = MODE == SCAN_DELTA;
  TORCH_CHECK(D <= 256, "key size above 256 is not supported by the recurrence kernel");
  // A step of single tokens (decoding) is all state traffic: a lane then holds 32 rows of its channel, so that few
  // lanes share a channel, a wave's loads of one state row cover 16 to 64 neighbouring channels and a block 64 to
  // 256 (whole cache lines), instead of 4 channels per wave when 16 lanes split a channel of 128 rows.
  const bool wide = MODE == SCAN_SSD && short_step;
  const int dpl = wide ? 32 : D > 128 ? 16 : 8;
  int P = 1;
  while (P * dpl < D) P <<= 1;
  const int cpb = 4 * 64 / P /* times NC of the kernel */, Dp = P * dpl, ct = Dp > 128 ? 8 : 16, nops = DELTA ? 3 : 2;
  const dim3 grid((unsigned)((Dv + cpb - 1) / cpb), (unsigned)H, (unsigned)B);
  const size_t smem = (size_t)(2 * ct * nops * Dp + 2 * ct * cpb + 4 * ct) * sizeof(float);
#define SCAN_CASE(PP, DD)                                                                                          \
  hipLaunchKernelGGL((matrix_state_scan_kernel<PP, DD, MODE, TV>), grid, dim3(256), smem, stream(), out, q, k,    \
                     gate, beta, v, vs, state, ss, cu, start, slots, H, rep, D, Dv, qk_ts, vec_ok, skip)
  if constexpr (MODE == SCAN_SSD) {
    if (wide) {
      if (P == 1) SCAN_CASE(1, 32);
      else if (P == 2) SCAN_CASE(2, 32);
      else if (P == 4) SCAN_CASE(4, 32);
      else SCAN_CASE(8, 32);
      HIP_CHECK_LAST();
      return;
    }
  }
  if (dpl == 16) SCAN_CASE(16, 16);
  else if (P == 1) SCAN_CASE(1, 8);
  else if (P == 2) SCAN_CASE(2, 8);
  else if (P == 4) SCAN_CASE(4, 8);
  else if (P == 8) SCAN_CASE(8, 8);
  else SCAN_CASE(16, 8);
#undef SCAN_CASE
  HIP_CHECK_LAST();
}

static void check_state(const at::Tensor& state, int H, int D, int Dv) {
  TORCH_CHECK(state.is_cuda() && is_f32(state) && state.dim() == 4 && state.size(1) == H && state.size(2) == D &&
              state.size(3) == Dv && state.stride(3) == 1 && state.stride(2) == Dv && state.stride(1) == (long)D * Dv,
              "state must be float32 [slots, H, D, Dv], dense inside a slot");
}

static void check_rows3(const at::Tensor& t, const char* name) {
  check_act(t, name);
  TORCH_CHECK(t.dim() == 3 && t.stride(2) == 1 && t.stride(1) == t.size(2), name, " must be [N, heads, dim] with dense rows");
}

at::Tensor gated_delta_rule(at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor beta_logit, at::Tensor dt,
                            at::Tensor A_log, at::Tensor dt_bias, at::Tensor state, at::Tensor cu, at::Tensor start,
                            at::Tensor slots, double unit_eps, double q_scale) {
  check_rows3(q, "q"); check_rows3(k, "k"); check_rows3(v, "v");
  check_act(beta_logit, "beta_logit"); check_act(dt, "dt");
  const long N = q.size(0);
  const int G = (int)q.size(1), D = (int)q.size(2), H = (int)v.size(1), Dv = (int)v.size(2);
  TORCH_CHECK(k.size(0) == N && v.size(0) == N && k.size(1) == G && k.size(2) == D && H % G == 0);
  TORCH_CHECK(beta_logit.dim() == 2 && beta_logit.size(0) == N && beta_logit.size(1) == H && beta_logit.stride(1) == 1);
  TORCH_CHECK(dt.dim() == 2 && dt.size(0) == N && dt.size(1) == (long)H * D && dt.stride(1) == 1);
  TORCH_CHECK(q.scalar_type() == k.scalar_type() && q.scalar_type() == v.scalar_type() &&
              beta_logit.scalar_type() == dt.scalar_type(), "q/k/v share one dtype, the logits another or the same");
  check_state(state, H, D, Dv);
  check_i32(cu, "cu"); check_i32(start, "start"); check_i32(slots, "slots");
  const int B = (int)start.numel();
  at::Tensor Af = f32c(A_log), bf = f32c(dt_bias);
  TORCH_CHECK(Af.numel() == H && bf.numel() == (long)H * D);
  auto fo = q.options().dtype(at::kFloat);
  at::Tensor out = at::empty({N, H, Dv}, fo);
  if (N == 0) return out;
  at::Tensor qn = at::empty({N, G, D}, fo), kn = at::empty({N, G, D}, fo), dec = at::empty({N, H, D}, fo),
             beta = at::empty({N, H}, fo);
  SERVING_DISPATCH_ACT(q, T, {
    SERVING_DISPATCH_ACT(dt, TL, {
      hipLaunchKernelGGL((delta_prepare_kernel<T, TL>), dim3((unsigned)N), dim3(256), 0, stream(), qn.data_ptr<float>(),
                         kn.data_ptr<float>(), dec.data_ptr<float>(), beta.data_ptr<float>(), ptr<T>(q),
                         (long)q.stride(0), ptr<T>(k), (long)k.stride(0), ptr<TL>(beta_logit),
                         (long)beta_logit.stride(0), ptr<TL>(dt), (long)dt.stride(0), Af.data_ptr<float>(),
                         bf.data_ptr<float>(), G, H, D, (float)unit_eps, (float)q_scale);
    });
    HIP_CHECK_LAST();
    launch_scan<SCAN_DELTA, T>(out.data_ptr<float>(), qn.data_ptr<float>(), kn.data_ptr<float>(), dec.data_ptr<float>(),
                         beta.data_ptr<float>(), ptr<T>(v), (long)v.stride(0), state.data_ptr<float>(),
                         (long)state.stride(0), cu.data_ptr<int>(), start.data_ptr<int>(), slots.data_ptr<int>(), B, H,
                         H / G, D, Dv);
  });
  return out;
}

at::Tensor tied_gate_recurrence(at::Tensor q, at::Tensor f_logit, at::Tensor v, at::Tensor f_bias, at::Tensor lower,
                                at::Tensor state, at::Tensor cu, at::Tensor start, at::Tensor slots) {
  check_rows3(q, "q"); check_rows3(f_logit, "f_logit"); check_rows3(v, "v");
  const long N = q.size(0);
  const int H = (int)q.size(1), D = (int)q.size(2), Dv = (int)v.size(2);
  TORCH_CHECK(f_logit.sizes() == q.sizes() && v.size(0) == N && v.size(1) == H);
  TORCH_CHECK(q.scalar_type() == f_logit.scalar_type() && q.scalar_type() == v.scalar_type());
  check_state(state, H, D, Dv);
  check_i32(cu, "cu"); check_i32(start, "start"); check_i32(slots, "slots");
  const int B = (int)start.numel();
  at::Tensor fb = f32c(f_bias), lo = f32c(lower);
  TORCH_CHECK(fb.numel() == (long)H * D && lo.numel() == (long)H * D);
  auto fo = q.options().dtype(at::kFloat);
  at::Tensor out = at::empty({N, H, Dv}, fo);
  if (N == 0) return out;
  at::Tensor qa = at::empty({N, H, D}, fo), f = at::empty({N, H, D}, fo);
  SERVING_DISPATCH_ACT(q, T, {
    hipLaunchKernelGGL(tied_prepare_kernel<T>, dim3((unsigned)N), dim3(256), 0, stream(), qa.data_ptr<float>(),
                       f.data_ptr<float>(), ptr<T>(q), (long)q.stride(0), ptr<T>(f_logit), (long)f_logit.stride(0),
                       fb.data_ptr<float>(), lo.data_ptr<float>(), H * D);
    HIP_CHECK_LAST();
    launch_scan<SCAN_TIED, T>(out.data_ptr<float>(), qa.data_ptr<float>(), (const float*)nullptr, f.data_ptr<float>(),
                          (const float*)nullptr, ptr<T>(v), (long)v.stride(0), state.data_ptr<float>(),
                          (long)state.stride(0), cu.data_ptr<int>(), start.data_ptr<int>(), slots.data_ptr<int>(), B, H,
                          1, D, Dv);
  });
  return out;
}

at::Tensor ssd_recurrence(at::Tensor x, at::Tensor Bm, at::Tensor Cm, at::Tensor dt_raw, at::Tensor A_log,
                          at::Tensor dt_bias, at::Tensor D_skip, at::Tensor state, at::Tensor cu, at::Tensor start,
                          at::Tensor slots) {
  check_act(x, "x"); check_act(dt_raw, "dt_raw");
  TORCH_CHECK(x.dim() == 3 && x.stride(2) == 1 && x.stride(1) == x.size(2), "x must be [N, H, Dv] with dense rows");
  const long N = x.size(0);
  const int H = (int)x.size(1), Dv = (int)x.size(2);
  // B and C feed the recurrence unrounded: float32 rows [N, G, D], dense inside a row, one token stride for both
  TORCH_CHECK(Bm.is_cuda() && is_f32(Bm) && Cm.is_cuda() && is_f32(Cm) && Bm.dim() == 3 && Bm.sizes() == Cm.sizes() &&
              Bm.size(0) == N, "B and C must be float32 [N, G, D]");
  const int G = (int)Bm.size(1), D = (int)Bm.size(2);
  TORCH_CHECK(Bm.stride(2) == 1 && Cm.stride(2) == 1 && Bm.stride(1) == D && Cm.stride(1) == D &&
              Bm.stride(0) == Cm.stride(0), "B and C rows must be dense and share a token stride");
  TORCH_CHECK(G > 0 && H % G == 0, "heads must split evenly into the groups");
  TORCH_CHECK(dt_raw.dim() == 2 && dt_raw.size(0) == N && dt_raw.size(1) == H && dt_raw.stride(1) == 1);
  check_state(state, H, D, Dv);
  check_i32(cu, "cu"); check_i32(start, "start"); check_i32(slots, "slots");
  const int B = (int)start.numel();
  at::Tensor Af = f32c(A_log), bf = f32c(dt_bias), Df = f32c(D_skip);
  TORCH_CHECK(Af.numel() == H && bf.numel() == H && Df.numel() == H && Af.is_cuda() && bf.is_cuda() && Df.is_cuda());
  auto fo = x.options().dtype(at::kFloat);
  at::Tensor out = at::empty({N, H, Dv}, fo);
  if (N == 0) return out;
  at::Tensor scal = at::empty({N, H, 2}, fo);
  SERVING_DISPATCH_ACT(dt_raw, TL, {
    hipLaunchKernelGGL(ssd_prepare_kernel<TL>, dim3((unsigned)((N * H + 255) / 256)), dim3(256), 0, stream(),
                       scal.data_ptr<float>(), ptr<TL>(dt_raw), (long)dt_raw.stride(0), Af.data_ptr<float>(),
                       bf.data_ptr<float>(), N, H);
  });
  HIP_CHECK_LAST();
  const int vec_ok = (Bm.stride(0) % 4 == 0 && reinterpret_cast<uintptr_t>(Bm.data_ptr()) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(Cm.data_ptr()) % 16 == 0) ? 1 : 0;
  SERVING_DISPATCH_ACT(x, T, {
    launch_scan<SCAN_SSD, T>(out.data_ptr<float>(), Cm.data_ptr<float>(), Bm.data_ptr<float>(), (const float*)nullptr,
                             scal.data_ptr<float>(), ptr<T>(x), (long)x.stride(0), state.data_ptr<float>(),
                             (long)state.stride(0), cu.data_ptr<int>(), start.data_ptr<int>(), slots.data_ptr<int>(),
                             B, H, H / G, D, Dv, (long)Bm.stride(0), vec_ok, Df.data_ptr<float>(), N <= 2L * B);
  });
  return out;
}

}  // namespace serving
}  // namespace cai

// Attention of a ragged batch over paged keys/values with a sliding window,
// kept first tokens, a linear distance penalty, a per-head output gate, a tanh
// soft cap on the scaled score and an optional sink (one more place of score 0
// in the softmax denominator that carries no value; with sink logits its score is learned per
// head), an additive per-distance table, block summaries (one mean key/value per block of
// positions that lies wholly before the window, kept in a small pool of their own) and, for
// talking heads, every query head's weights applied to every key/value head's values.
//
// One wave per (token, query head). The visible keys of a token are two
// position ranges: the kept prefix [0, min(keep_first, lo)) and the window
// [lo, pos] with lo = max(0, pos - window + 1) (lo = 0 without a window); the
// wave walks their concatenation 64 keys at a time. Phase 1: lane = key, each
// lane takes the full dot product of its key with the query (query in LDS,
// key row read with its own page lookup). Online softmax in float32 across
// the 64-key blocks. Phase 2: lane = value channel, the block's weights and
// pool rows are broadcast from LDS. A prompt portion and a decode token run
// the same code, so a position's result depends on nothing but the pages.
#include "serving_common.h"

namespace cai {
namespace serving {

constexpr int ATT_WAVES = 16;  // most waves of a block: they split the key blocks of one (token, kv head)
constexpr int RC_MAX = 4;      // most query heads of a kv head's group that one block handles together
constexpr int MFMA_TILES_PER_STEP = 2;  // 32-key tiles the matrix-core kernel stages and multiplies between two barriers

template <int CTRL>
DEV_INLINE float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
  return v + __builtin_bit_cast(float, moved);
}
// sum over the 8 adjacent lanes that share a key (quad xor 1, quad xor 2, half-row mirror)
DEV_INLINE float reduce8(float v) { return dpp_add<0x141>(dpp_add<0x4E>(dpp_add<0xB1>(v))); }

// Scalar kernel (decode tokens, float32 serving, shapes the MFMA kernel does not take).
// One block per (token, kv head, group of up to RC query heads of that kv head): keys and
// values are read once for the whole group. The block's nw waves (16, or 8 when the partial
// states of 16 would not fit in LDS) take every nw-th block of 64 keys and merge their partial
// softmax states through LDS at the end. The eight key steps of a block are unrolled so that
// their page lookups and key loads are all in flight before the first product.
// Scores: 8 adjacent lanes share a key, each takes a contiguous slice of the head size
// (16-byte loads, few cache lines per instruction) and the slices are summed on the DPP path.
// Values: lane = a pair of value channels, the block's weights and pool rows come from LDS.
// RC = query heads per block: 4 shares each key/value read between the most heads; 2 or 1 are
// chosen when a decode step would otherwise leave most CUs without a block (the re-reads hit L2).
// V8 (value head sizes that are multiples of 8 up to 512): a lane takes 8 consecutive value channels of a key with
// one 16/32-byte load, vl = Dv / 8 rounded up to a power of two lanes cover a key's row and the 64 / vl lane groups
// take different keys of the block, so a block of 64 keys is read by vl load instructions instead of 64; the groups' sums meet in a butterfly of
// shuffles after the last block.
template <typename T, int RC, bool V8>
__global__ __launch_bounds__(64 * ATT_WAVES) void paged_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ kpool,
    const T* __restrict__ vpool, const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ tok_seq,
    const int* __restrict__ positions, const float* __restrict__ slopes, const T* __restrict__ gate, long gate_stride,
    int H, int G, int D, int Dv, int page_shift, float scale, int window, int keep_first, int kvec, int vvec,
    float softcap, int sink, long vrow, long vhead, const float* __restrict__ sink_logits,
    const float* __restrict__ dist_bias, int dist_rows, const T* __restrict__ ksum, const T* __restrict__ vsum,
    int sum_shift, int sum_block, float* __restrict__ cross_out) {
  // sink_logits [H]: the sink's score per head instead of 0. dist_bias [dist_rows, H]: added to the score of a key at
  // distance d (row min(d, dist_rows - 1)). ksum / vsum: block summaries, rows [pages << sum_shift]; a query at
  // `pos` sees the first max(0, (pos - window + 1) / sum_block) of its sequence's, ahead of its other keys and
  // without distance terms. cross_out [N, H, G, Dv] float32: the grid then has G blocks per (token, kv head, chunk),
  // block c applies the heads' weights to the values of kv head c.
  // vrow / vhead: elements between the value rows of neighbouring pool rows / kv heads (G * Dv and Dv for a
  // pool of its own; a value pool that is a view into wider rows, e.g. the leading channels of the keys, has others)
  extern __shared__ __align__(16) float lds[];
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const int Dp = (D + 7) & ~7;
  const int R = H / G, chunks = (R + RC - 1) / RC;
  float* qs = lds;                                        // [RC][Dp] queries
  float* pw = lds + RC * Dp + wid * (RC * 64 + 64);       // [RC][64] scores, then weights, of this wave's key block
  int* prow = reinterpret_cast<int*>(pw + RC * 64);       // [64] pool rows of the block
  float* part = lds + RC * Dp + nw * (RC * 64 + 64);      // [waves][RC][2 + Dv] partial states
  const int VC = cross_out != nullptr ? G : 1;
  const long bx = blockIdx.x / VC;
  const long n = bx / (G * chunks);
  const int g = (int)(bx / chunks) % G;
  const int vg = cross_out != nullptr ? (int)(blockIdx.x % VC) : g;  // kv head whose values this block reads
  const int h0 = g * R + (int)(bx % chunks) * RC;  // first query head of this block
  const int nh = min(RC, g * R + R - h0);
  const int b = tok_seq[n];
  const int pos = positions[n];
  const int* bt = block_tables + (long)b * bt_stride;
  const int page_mask = (1 << page_shift) - 1;

  for (int i = threadIdx.x; i < RC * Dp; i += blockDim.x) {
    const int r = i / Dp, d = i % Dp;
    qs[i] = (r < nh && d < D) ? ldf(q + n * q_stride + (long)(h0 + r) * D + d) : 0.0f;
  }
  __syncthreads();
  float slope[RC];
#pragma unroll
  for (int r = 0; r < RC; ++r) slope[r] = (slopes != nullptr && r < nh) ? slopes[h0 + r] : 0.0f;

  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int n_sum = (ksum != nullptr && window > 0) ? max(0, (pos - window + 1) / sum_block) : 0;
  const int sum_mask = (1 << sum_shift) - 1;
  const int n_keep = (window > 0 ? min(keep_first, lo) : 0) + n_sum;  // summaries, then kept first tokens
  const int total = n_keep + (pos - lo + 1);
  const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;
  const int part8 = lane & 7, ksub = lane >> 3;
  const int DS = (((D + 7) >> 3) + 7) & ~7;  // slice of the head size per lane, a multiple of 8
  const int d_lo = part8 * DS, d_hi = min(D, d_lo + DS);

  constexpr int NA = V8 ? 8 : 4;  // value channels a lane accumulates
  float m[RC], l[RC], acc[RC][NA];
#pragma unroll
  for (int r = 0; r < RC; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.0f;
#pragma unroll
    for (int i = 0; i < NA; ++i) acc[r][i] = 0.0f;
  }
  int vl = 1;                                 // V8: lanes per key row: the power of two that holds Dv / 8 ...
  while (vl * 8 < Dv) vl <<= 1;               // (lanes of a row beyond Dv / 8 idle when Dv / 8 is no power of two)
  const int vks = V8 ? 64 / vl : 1;           // ... keys per load instruction ...
  const int vsub = V8 ? lane / vl : 0;        // ... this lane's key group ...
  const int vch = V8 ? (lane % vl) * 8 : 0;   // ... and its first value channel
  const bool vlive = vch < Dv;

  for (int base = wid * 64; base < total; base += 64 * nw) {
    const int cnt = min(64, total - base);
    auto score_step = [&](int sub) {
      const int idx = base + sub * 8 + ksub;
      const bool valid = idx < total;
      const bool summary = valid && idx < n_sum;
      const int j = valid ? (idx < n_keep ? idx - n_sum : lo + (idx - n_keep)) : pos;
      const int row = summary ? (bt[idx >> sum_shift] << sum_shift) + (idx & sum_mask)
                              : (bt[j >> page_shift] << page_shift) + (j & page_mask);
      float dots[RC];
#pragma unroll
      for (int r = 0; r < RC; ++r) dots[r] = 0.0f;
      const T* kr = (summary ? ksum : kpool) + ((long)row * G + g) * D;
      if (kvec) {
        for (int d = d_lo; d < d_hi; d += 8) {
          float kv[8];
          load8(kr + d, kv);
#pragma unroll
          for (int r = 0; r < RC; ++r) {
            const float4v qa = *reinterpret_cast<const float4v*>(qs + r * Dp + d);
            const float4v qb = *reinterpret_cast<const float4v*>(qs + r * Dp + d + 4);
            dots[r] += kv[0] * qa[0] + kv[1] * qa[1] + kv[2] * qa[2] + kv[3] * qa[3] + kv[4] * qb[0] + kv[5] * qb[1] +
                       kv[6] * qb[2] + kv[7] * qb[3];
          }
        }
      } else {
        for (int d = d_lo; d < d_hi; ++d) {
          const float kv = ldf(kr + d);
#pragma unroll
          for (int r = 0; r < RC; ++r) dots[r] += kv * qs[r * Dp + d];
        }
      }
#pragma unroll
      for (int r = 0; r < RC; ++r) dots[r] = reduce8(dots[r]);
      if (part8 == 0) {
#pragma unroll
        for (int r = 0; r < RC; ++r) {
          float sc = dots[r] * scale;
          if (softcap > 0.0f) sc = softcap * tanhf(sc * inv_cap);
          if (!summary) {
            sc -= slope[r] * (float)(pos - j);
            if (dist_bias != nullptr && r < nh) sc += dist_bias[(long)min(pos - j, dist_rows - 1) * H + h0 + r];
          }
          pw[r * 64 + sub * 8 + ksub] = valid ? sc : -INFINITY;
        }
        prow[sub * 8 + ksub] = summary ? -1 - row : row;  // a summary row is marked by its sign
      }
    };
    if (cnt == 64) {  // straight-line: all eight steps' lookups and key loads issue before the first product
#pragma unroll
      for (int sub = 0; sub < 8; ++sub) score_step(sub);
    } else {          // the last block of a key range: only the steps that hold keys
      for (int sub = 0; sub * 8 < cnt; ++sub) score_step(sub);
    }
    // the wave is its own producer and consumer of pw/prow: wait for its LDS writes
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    float corr[RC];
#pragma unroll
    for (int r = 0; r < RC; ++r) {
      const float s = lane < cnt ? pw[r * 64 + lane] : -INFINITY;
      const float m_new = fmaxf(m[r], wave_reduce_max(s));  // a block holds at least one visible key
      const float w = expf(s - m_new);                      // exp(-inf) = 0 for the block's empty places
      corr[r] = expf(m[r] - m_new);                         // m = -inf before the first block: 0
      l[r] = l[r] * corr[r] + wave_reduce_sum(w);
      m[r] = m_new;
      pw[r * 64 + lane] = w;
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
#pragma unroll
    for (int r = 0; r < RC; ++r)
#pragma unroll
      for (int i = 0; i < NA; ++i) acc[r][i] *= corr[r];
    if constexpr (V8) {
#pragma unroll 4
      for (int jj = vsub; jj < cnt; jj += vks) {
        float v[8];
        if (vlive) {
          const int pr = prow[jj];
          load8((pr < 0 ? vsum : vpool) + (long)(pr < 0 ? -1 - pr : pr) * vrow + (long)vg * vhead + vch, v);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = 0.0f;
        }
#pragma unroll
        for (int r = 0; r < RC; ++r) {
          const float w = pw[r * 64 + jj];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[r][e] += w * v[e];
        }
      }
    } else {
    const int dva = 2 * lane, dvb = 128 + 2 * lane;
#pragma unroll 8
    for (int jj = 0; jj < cnt; ++jj) {
      const int pr = prow[jj];
      const T* vr = (pr < 0 ? vsum : vpool) + (long)(pr < 0 ? -1 - pr : pr) * vrow + (long)vg * vhead;
      float v0 = 0.0f, v1 = 0.0f, v2 = 0.0f, v3 = 0.0f;
      if (vvec) {
        if (dva < Dv) load2(vr + dva, v0, v1);
        if (dvb < Dv) load2(vr + dvb, v2, v3);
      } else {
        if (dva < Dv) v0 = ldf(vr + dva);
        if (dva + 1 < Dv) v1 = ldf(vr + dva + 1);
        if (dvb < Dv) v2 = ldf(vr + dvb);
        if (dvb + 1 < Dv) v3 = ldf(vr + dvb + 1);
      }
#pragma unroll
      for (int r = 0; r < RC; ++r) {
        const float w = pw[r * 64 + jj];
        acc[r][0] += w * v0; acc[r][1] += w * v1; acc[r][2] += w * v2; acc[r][3] += w * v3;
      }
    }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
  const int PS = 2 + Dv;
  float* mine = part + (long)wid * RC * PS;
#pragma unroll
  for (int r = 0; r < RC; ++r) {
    if (lane == 0) { mine[r * PS] = m[r]; mine[r * PS + 1] = l[r]; }
    if constexpr (V8) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float v = acc[r][e];
        for (int off = vl; off < 64; off <<= 1) v += __shfl_xor(v, off);  // the key groups' sums of this channel
        if (vsub == 0 && vlive) mine[r * PS + 2 + vch + e] = v;
      }
    } else {
      const int dva = 2 * lane, dvb = 128 + 2 * lane;
      if (dva < Dv) mine[r * PS + 2 + dva] = acc[r][0];
      if (dva + 1 < Dv) mine[r * PS + 2 + dva + 1] = acc[r][1];
      if (dvb < Dv) mine[r * PS + 2 + dvb] = acc[r][2];
      if (dvb + 1 < Dv) mine[r * PS + 2 + dvb + 1] = acc[r][3];
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < nh * Dv; i += blockDim.x) {
    const int r = i / Dv, dv = i % Dv;
    float mm = -INFINITY;
    for (int w = 0; w < nw; ++w) mm = fmaxf(mm, part[(w * RC + r) * PS]);
    float ll = 0.0f, o = 0.0f;
    for (int w = 0; w < nw; ++w) {
      const float mw = part[(w * RC + r) * PS];
      if (mw != -INFINITY) {
        const float f = expf(mw - mm);
        ll += part[(w * RC + r) * PS + 1] * f;
        o += part[(w * RC + r) * PS + 2 + dv] * f;
      }
    }
    if (sink_logits != nullptr) {  // a learned score: it may be the largest of the row
      const float sk = sink_logits[h0 + r], m2 = fmaxf(mm, sk), f2 = expf(mm - m2);
      ll = ll * f2 + expf(sk - m2);
      o *= f2;
    } else if (sink) {
      ll += expf(-mm);  // the sink's score is 0
    }
    float scale_out = 1.0f / ll;
    if (gate != nullptr) scale_out *= sigmoidf_(ldf(gate + n * gate_stride + h0 + r));
    if (cross_out != nullptr) cross_out[((n * H + h0 + r) * G + vg) * (long)Dv + dv] = o * scale_out;
    else stf(out + (n * H + h0 + r) * (long)Dv + dv, o * scale_out);
  }
}

// MFMA kernel (bfloat16 prompt portions). One block per (32-token tile of one sequence, kv head,
// pass); its waves are query heads of that kv head's group, so a key/value tile is fetched once
// for all of them: 16-byte loads through the page table into LDS, double-buffered (the next
// tile's loads are in flight while this tile is multiplied). All per-token quantities are
// lane-local because the products are formed transposed:
//   S^T = K Q^T   (A = key rows from LDS, B = query rows kept in registers)
//   O^T = V^T P^T (B = the float32 weights in the C layout they were born in, split into a
//                  high and a low bfloat16 half so that no weight loses its float32 mantissa
//                  to the matrix unit; A = values, stored transposed in LDS in the same key
//                  order, one 16-byte read per product)
// so column = token = lane & 31 everywhere: running max, running sum, rescaling and the gate
// never cross lanes except for one exchange between the two half-waves.
// The tiles are DS * 16 key channels by VT * 32 value channels; a head whose sizes Dr / Dvr are
// smaller (multiples of 8) is padded with zeros on its way into registers and LDS, and only its
// own channels are stored.
template <int DS, int VT>
__global__ __launch_bounds__(256) void paged_attention_mfma_kernel(
    bf16s* __restrict__ out, const bf16s* __restrict__ q, long q_stride, const bf16s* __restrict__ kpool,
    const bf16s* __restrict__ vpool, const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ cu,
    const int* __restrict__ start, const float* __restrict__ slopes, const bf16s* __restrict__ gate, long gate_stride,
    int H, int G, int Dr, int Dvr, int page_shift, float scale, int window, int keep_first, float softcap, int sink,
    int qsplit, const float* __restrict__ sink2, const float* __restrict__ dist2, int dist_rows,
    const bf16s* __restrict__ ksum, const bf16s* __restrict__ vsum, int sum_shift, int sum_block,
    float* __restrict__ cross_out) {
  // The optional extras of the split-key kernel, in the base-2 domain: sink2 [H] = learned sink scores * log2e;
  // dist2 [H, dist_rows] = the per-distance bias * log2e, one row per head; ksum / vsum = block summaries, staged as
  // the first tiles of a block (summary idx of a sequence is seen by a token at pos when idx < (pos - window + 1) /
  // sum_block); cross_out [N, H, G, Dv] float32: the grid's z axis then also counts the kv head whose values a block
  // multiplies the weights with.
  // qsplit (kv heads with a single query head each): the four waves of a block are four consecutive 32-token tiles
  // of that head instead of four heads, so a block covers 128 tokens, the grid's x axis counts 128-token tiles, and
  // the staged key/value tiles are still shared by all computing waves. The block stages the key range of all its
  // tokens; a wave skips the tiles that lie wholly after its own tokens.
  constexpr int D = DS * 16, Dv = VT * 32;
  bf16x8_v zero8;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero8[e] = (__bf16)0.0f;
  constexpr int KP = D + 8;            // key row pitch in LDS (elements): 16-byte reads of 16 rows hit 64 banks
  constexpr int VP = 40;               // transposed value row pitch: 32 key slots + 8
  constexpr int KT = 32 * KP, VTT = Dv * VP;   // elements of one staged tile
  constexpr int KCH = 32 * D / 8, VCH = 32 * Dv / 8;  // 16-byte chunks of a key / value tile
  constexpr int TP = MFMA_TILES_PER_STEP;
  extern __shared__ __align__(16) bf16s tiles[];  // [2][TP][KT + VTT]
  constexpr int nthreads = 256;  // always four waves: those beyond the group's heads only help staging
  const int tid = threadIdx.x;
  const int wid = tid >> 6, lane = tid & 63;
  const int rep = H / G, g = blockIdx.y;
  const int VC = cross_out != nullptr ? G : 1;
  const int vg = cross_out != nullptr ? (int)(blockIdx.z % VC) : g;   // kv head of the values
  const int hl = qsplit ? 0 : (blockIdx.z / VC) * (nthreads >> 6) + wid;  // head inside the group
  const int h = g * rep + (hl < rep ? hl : 0);
  const int bshift = qsplit ? 7 : 5;                  // log2 of the tokens a block covers
  // Under a causal mask a late tile of a long prompt has many more key tiles than an early one. Rows of the grid
  // (kv head, pass) walk the tiles alternately from the back and from the front, switching with every 256 blocks of
  // dispatch order, so that blocks which come to share a CU tend to pair a long tile with a short one and the
  // longest tiles start first.
  const bool from_back = ((gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) >> 8 & 1) == 0;
  int tile = from_back ? gridDim.x - 1 - blockIdx.x : blockIdx.x, b = 0;
  for (;; ++b) {  // the grid holds exactly sum_b ceil(count_b / tokens per block) tiles
    const int nt = (cu[b + 1] - cu[b] + (1 << bshift) - 1) >> bshift;
    if (tile < nt) break;
    tile -= nt;
  }
  const int cnt = cu[b + 1] - cu[b];
  const int col = lane & 31, hf = lane >> 5;
  const int bt_off = tile << bshift;                          // first token of the block
  const int t_off = bt_off + (qsplit ? wid * 32 : 0);         // first token of this wave
  const bool head_ok = qsplit ? t_off < cnt : hl < rep;       // this wave computes
  const bool tok_ok = t_off + col < cnt;
  const int my_i = tok_ok ? t_off + col : cnt - 1;
  const long n = cu[b] + my_i;
  const int s0 = start[b];
  const int pos = s0 + my_i;
  const int p0 = s0 + t_off, p1 = s0 + min(t_off + 31, cnt - 1);              // this wave's positions
  const int bp0 = s0 + bt_off, bp1 = s0 + min(bt_off + (1 << bshift) - 1, cnt - 1);  // the block's
  const int* bt = block_tables + (long)b * bt_stride;
  const int page_mask = (1 << page_shift) - 1;
  const float slope = slopes != nullptr ? slopes[h] : 0.0f;

  bf16x8_v qf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s)
    qf[s] = 16 * s + hf * 8 < Dr ? ld_g16b(q + n * q_stride + (long)h * Dr + 16 * s + hf * 8) : zero8;

  const int lo_min = window > 0 ? max(0, bp0 - window + 1) : 0;   // the staged key range is the block's
  const int wstart = lo_min & ~31;
  const int n_sink = window > 0 ? min(keep_first, wstart) : 0;  // kept keys below the window's first tile
  const int n_sum = (ksum != nullptr && window > 0) ? max(0, (bp1 - window + 1) / sum_block) : 0;  // the block's last token's
  const int sum_tiles = (n_sum + 31) >> 5;
  const int sum_mask = (1 << sum_shift) - 1;
  const int sink_tiles = sum_tiles + ((n_sink + 31) >> 5);   // summary tiles, then kept-prefix tiles, then the window's
  const int tiles_n = sink_tiles + ((bp1 - wstart) >> 5) + 1;
  const int my_sum = (ksum != nullptr && window > 0) ? max(0, (pos - window + 1) / sum_block) : 0;  // this token's
  const float* db = dist2 != nullptr ? dist2 + (long)h * dist_rows : nullptr;

  // staging: key chunk c = key c / (row chunks), 8 elements starting at 8 * (c % row chunks), stored as a row;
  // value chunk c = key c % 32, 8 channels starting at 8 * (c / 32): the values are stored transposed, two bytes at
  // a time, and with neighbouring threads on neighbouring keys these stores spread over the LDS banks
  constexpr int KR = (KCH + 255) / 256, VR = (VCH + 255) / 256;  // chunks per thread of the 256
  // TP key tiles are staged, and multiplied, between two barriers: their loads are all in flight over the
  // products of the TP tiles before them
  bf16x8_v rk[TP][KR], rv[TP][VR];
  auto tile_base = [&](int it) {
    return it < sum_tiles ? it * 32 : it < sink_tiles ? (it - sum_tiles) * 32 : wstart + (it - sink_tiles) * 32;
  };
  auto pool_row = [&](int j) {
    const int jc = min(j, bp1);  // keys past the sequence's end are masked; read a row that exists
    return ((long)bt[jc >> page_shift] << page_shift) + (jc & page_mask);
  };
  auto sum_row = [&](int idx) {
    const int ic = min(idx, n_sum - 1);  // a summary tile exists only when n_sum > 0
    return ((long)bt[ic >> sum_shift] << sum_shift) + (ic & sum_mask);
  };
  // The page-table lookups of a tile run one tile ahead of its key/value loads (two ahead of its use), so that a
  // load's address never waits for a lookup issued in the same iteration.
  int krow[TP][KR], vrow[TP][VR];
  bool from_sum[TP];  // the tiles of the last lookup that are summary tiles
  auto lookup = [&](int step) {
#pragma unroll
    for (int u = 0; u < TP; ++u) {
      const int kbase = tile_base(step * TP + u);  // a tile past the last one reads rows that exist and is not used
      from_sum[u] = step * TP + u < sum_tiles;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        const int c = tid + nthreads * r;
        const int j = kbase + c / (D / 8);
        krow[u][r] = c < KCH ? (int)(from_sum[u] ? sum_row(j) : pool_row(j)) : 0;
      }
#pragma unroll
      for (int r = 0; r < VR; ++r) {
        const int c = tid + nthreads * r;
        const int j = kbase + (c & 31);
        vrow[u][r] = c < VCH ? (int)(from_sum[u] ? sum_row(j) : pool_row(j)) : 0;
      }
    }
  };
  auto fetch = [&]() {  // the tiles whose rows the last lookup left in krow / vrow
#pragma unroll
    for (int u = 0; u < TP; ++u) {
      const bf16s* kp = from_sum[u] ? ksum : kpool;
      const bf16s* vp = from_sum[u] ? vsum : vpool;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        const int c = tid + nthreads * r;
        if (c < KCH) {
          const int off = 8 * (c % (D / 8));
          rk[u][r] = off < Dr ? ld_g16b(kp + ((long)krow[u][r] * G + g) * Dr + off) : zero8;
        }
      }
#pragma unroll
      for (int r = 0; r < VR; ++r) {
        const int c = tid + nthreads * r;
        if (c < VCH) {
          const int off = 8 * (c >> 5);
          rv[u][r] = off < Dvr ? ld_g16b(vp + ((long)vrow[u][r] * G + vg) * Dvr + off) : zero8;
        }
      }
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int u = 0; u < TP; ++u) {
      bf16s* ks = tiles + (buf * TP + u) * (KT + VTT);
      bf16s* vt = ks + KT;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        const int c = tid + nthreads * r;
        if (c < KCH) *reinterpret_cast<bf16x8_v*>(ks + (c / (D / 8)) * KP + 8 * (c % (D / 8))) = rk[u][r];
      }
#pragma unroll
      for (int r = 0; r < VR; ++r) {
        const int c = tid + nthreads * r;
        if (c < VCH) {
          const int kk = c & 31, dv0 = 8 * (c >> 5);
          // contraction slot of key kk: the order in which the C layout of S^T hands the weights to P^T
          const int r16 = kk & 15;
          const int slot = (kk & 16) + ((r16 >> 2) & 1) * 8 + (r16 >> 3) * 4 + (r16 & 3);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const __bf16 x = rv[u][r][e];
            vt[(dv0 + e) * VP + slot] = *reinterpret_cast<const bf16s*>(&x);
          }
        }
      }
    }
  };

  // With a sink and a soft cap the scores live in [-cap2, cap2] (a distance penalty only lowers them) and the
  // denominator holds the sink's exp2(0) = 1: the weights can be taken against the fixed reference 0 instead of a
  // running maximum. exp2(cap2) cannot overflow for cap2 <= 96, and a weight that underflows is nothing beside the
  // sink's 1. No maximum to track, no accumulator to rescale.
  const bool fixed_ref = sink != 0 && softcap > 0.0f && softcap * 1.4426950408889634f <= 96.0f;
  float m = fixed_ref ? 0.0f : -INFINITY, l = 0.0f;  // m in the base-2 domain
  f32x16 oacc[VT];
#pragma unroll
  for (int t = 0; t < VT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[t][i] = 0.0f;
  constexpr float LOG2E = 1.4426950408889634f;
  const float c1 = scale * LOG2E, sl2 = slope * LOG2E;
  // soft cap in the base-2 domain: cap log2e tanh(x scale / cap), tanh(y) = 1 - 2 / (exp2(2 log2e y) + 1)
  const bool capped = softcap > 0.0f;
  const float cap2 = softcap * LOG2E, t2 = capped ? 2.0f * LOG2E * scale / softcap : 0.0f;
  auto base2 = [&](float dot) {
    if (!capped) return dot * c1;
    const float e = __builtin_amdgcn_exp2f(fminf(dot * t2, 64.0f));  // beyond 2^64 the quotient is 0 in float32 anyway
    return cap2 - 2.0f * cap2 * __builtin_amdgcn_rcpf(e + 1.0f);
  };
  float row_bias[16];  // + slope log2e * (row of the C layout): the key's offset inside its tile
#pragma unroll
  for (int i = 0; i < 16; ++i) row_bias[i] = sl2 * (float)((i & 3) + 8 * (i >> 2) + 4 * hf);

  const int steps_n = (tiles_n + TP - 1) / TP;
  lookup(0);
  fetch();
  if (steps_n > 1) lookup(1);
  stash(0);
  __syncthreads();
  for (int step = 0; step < steps_n; ++step) {
    const int buf = step & 1;
    const bool more = step + 1 < steps_n;
    if (more) {
      fetch();
      if (step + 2 < steps_n) lookup(step + 2);
    }
#pragma unroll
    for (int u = 0; u < TP; ++u) {
      const int it = step * TP + u;
      if (!head_ok || it >= tiles_n) continue;
      const bool summ = it < sum_tiles;
      const bool sink = it < sink_tiles;  // a tile ahead of the window's: summaries or kept first tokens
      const int kbase = tile_base(it);
      if (!sink && kbase > p1) continue;  // (query split) a tile wholly after this wave's tokens
      const int klimit = sink ? n_sink : p1 + 1;  // keys of this tile at or above it are not this tile's to count
      const bf16s* ks = tiles + (buf * TP + u) * (KT + VTT);
      const bf16s* vt = ks + KT;
      f32x16 sacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[i] = 0.0f;
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const bf16x8_v kf = *reinterpret_cast<const bf16x8_v*>(ks + col * KP + 16 * s + hf * 8);
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], sacc, 0, 0, 0);
      }
      // scores in the base-2 domain: s2 = (q.k) scale log2e - slope log2e (pos - j), one add and one fma each
      float sv[16];
      const float tile_bias = -sl2 * (float)(pos - kbase);
      // interior tile: every key is visible to every token of the tile, no masks to evaluate
      const bool interior = !sink && t_off + 31 < cnt && kbase + 31 <= p0 && (window == 0 || p1 - kbase < window);
      if (summ) {  // summaries: seen by count, no distance terms
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int j = kbase + (i & 3) + 8 * (i >> 2) + 4 * hf;
          sv[i] = (tok_ok && j < my_sum) ? base2(sacc[i]) : -INFINITY;
        }
      } else if (interior) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          sv[i] = base2(sacc[i]) + (tile_bias + row_bias[i]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int j = kbase + (i & 3) + 8 * (i >> 2) + 4 * hf;
          const bool seen = tok_ok && j < klimit && j <= pos && (window == 0 || pos - j < window || j < keep_first);
          sv[i] = seen ? base2(sacc[i]) + (tile_bias + row_bias[i]) : -INFINITY;
        }
      }
      if (db != nullptr && !summ) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int j = kbase + (i & 3) + 8 * (i >> 2) + 4 * hf;
          sv[i] += db[min(max(pos - j, 0), dist_rows - 1)];   // -inf stays -inf
        }
      }
      float m_ref = 0.0f, corr = 1.0f;
      if (!fixed_ref) {
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, sv[i]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m, tmax);
        m_ref = (m_new == -INFINITY) ? 0.0f : m_new;  // nothing visible yet: every weight is exp2(-inf) = 0
        corr = (m == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m - m_new);  // nothing accumulated: nothing to rescale
        m = m_new;
      }
      float psum = 0.0f;
      bf16x8_v phi[2], plo[2];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float p = __builtin_amdgcn_exp2f(sv[i] - m_ref);
        psum += p;
        const __bf16 hi = (__bf16)p;
        phi[i >> 3][i & 7] = hi;
        plo[i >> 3][i & 7] = (__bf16)(p - (float)hi);
      }
      l = l * corr + psum;
      if (!fixed_ref && !__all(corr == 1.0f)) {  // the running maxima of all 32 tokens stood still: no rescaling
#pragma unroll
        for (int t = 0; t < VT; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[t][i] *= corr;
      }
      // O^T += V^T P^T: slot hf * 8 + e of step s2 holds key kbase + 16 s2 + 8 (e >> 2) + 4 hf + (e & 3)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int t = 0; t < VT; ++t) {
          const bf16x8_v va = *reinterpret_cast<const bf16x8_v*>(vt + (t * 32 + col) * VP + 16 * s2 + hf * 8);
          oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, phi[s2], oacc[t], 0, 0, 0);
          oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, plo[s2], oacc[t], 0, 0, 0);
        }
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
  }
  l += __shfl_xor(l, 32);
  if (sink2 != nullptr) l += __builtin_amdgcn_exp2f(sink2[h] - m);  // a learned score; a sink far above every key: 1 / inf = 0
  else if (sink) l += __builtin_amdgcn_exp2f(-m);  // the sink's score is 0 in either base; m is finite (a token sees itself)
  if (!tok_ok || !head_ok) return;
  float scale_out = 1.0f / l;
  if (gate != nullptr) scale_out *= sigmoidf_(ldf(gate + n * gate_stride + h));
  if (cross_out != nullptr) {
    float* crow = cross_out + ((n * H + h) * G + vg) * (long)Dvr;
#pragma unroll
    for (int t = 0; t < VT; ++t)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        if (t * 32 + 8 * a + 4 * hf >= Dvr) continue;
        *reinterpret_cast<float4v*>(crow + t * 32 + 8 * a + 4 * hf) =
            float4v{oacc[t][4 * a] * scale_out, oacc[t][4 * a + 1] * scale_out, oacc[t][4 * a + 2] * scale_out,
                    oacc[t][4 * a + 3] * scale_out};
      }
    return;
  }
  bf16s* orow = out + (n * H + h) * (long)Dvr;
#pragma unroll
  for (int t = 0; t < VT; ++t)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      if (t * 32 + 8 * a + 4 * hf >= Dvr) continue;  // padding channels (sizes are multiples of 8: four at a time)
      short4v pk;
#pragma unroll
      for (int c = 0; c < 4; ++c) pk[c] = (short)f2bf(oacc[t][4 * a + c] * scale_out);
      *reinterpret_cast<short4v*>(orow + t * 32 + 8 * a + 4 * hf) = pk;
    }
}

// What the split-key kernel takes beyond the common parameters (all optional).
struct ScalarExtras {
  const float* sink_logits = nullptr;
  const float* dist_bias = nullptr;
  int dist_rows = 0;
  const void* ksum = nullptr;
  const void* vsum = nullptr;
  int sum_shift = 0, sum_block = 1;
  float* cross_out = nullptr;
};

static void launch_scalar_attention(at::Tensor& out, const at::Tensor& q, const at::Tensor& kpool, const at::Tensor& vpool,
                                    const at::Tensor& block_tables, const at::Tensor& tok_seq, const at::Tensor& positions,
                                    const float* slp, const c10::optional<at::Tensor>& gate, long gstride, double scale,
                                    int64_t window, int64_t keep_first, double softcap, bool sink, int page_shift,
                                    long vrow, long vhead, const ScalarExtras& x) {
  const long N = q.size(0);
  const int H = (int)q.size(1), D = (int)q.size(2);
  const int G = (int)kpool.size(2), Dv = (int)vpool.size(3);
  const int VC = x.cross_out != nullptr ? G : 1;
  const int Dp = (D + 7) & ~7;
  const int R = H / G;
  int rc = RC_MAX;
  while (rc > 1 && (rc > R || N * G * VC * ((R + rc - 1) / rc) < 256)) rc >>= 1;  // enough blocks to cover the CUs
  auto lds_bytes = [&](int nw) { return (size_t)(rc * Dp + nw * (rc * 64 + 64) + nw * rc * (2 + Dv)) * sizeof(float); };
  // wide value rows (a latent of several hundred channels): fewer waves, then fewer heads per block
  int nwaves = ATT_WAVES;
  while (lds_bytes(nwaves) > 64 * 1024 && nwaves > 4) nwaves >>= 1;
  while (lds_bytes(nwaves) > 64 * 1024 && rc > 1) rc >>= 1;
  const int chunks = (R + rc - 1) / rc;
  const size_t smem = lds_bytes(nwaves);
  TORCH_CHECK(smem <= 64 * 1024, "head sizes too large for the scalar attention kernel");
  const int kvec = D % 8 == 0 ? 1 : 0;   // 16-byte (bfloat16) / 32-byte (float32) aligned key slices
  const int vvec_even = Dv % 2 == 0 ? 1 : 0;
  // value rows of a multiple of 8 channels whose loads are aligned take the 8-channels-per-lane value phase
  const bool v8 = Dv >= 8 && Dv % 8 == 0 && reinterpret_cast<uintptr_t>(vpool.data_ptr()) % 32 == 0 &&
                  vrow % 8 == 0 && vhead % 8 == 0;
  TORCH_CHECK(v8 || Dv <= 256, "value rows above 256 channels must be a multiple of 8 channels and aligned");
  const int vvec_ok = (vrow % 2 == 0 && vhead % 2 == 0) ? 1 : 0;
#define SCALAR_CASE(RC_)                                                                                            \
  if (v8) SCALAR_LAUNCH(RC_, true);                                                                                 \
  else SCALAR_LAUNCH(RC_, false)
#define SCALAR_LAUNCH(RC_, V8_)                                                                                     \
  hipLaunchKernelGGL((paged_attention_kernel<T, RC_, V8_>), dim3((unsigned)(N * G * chunks * VC)), dim3(64 * nwaves), smem,   \
                     stream(), x.cross_out != nullptr ? (T*)nullptr : ptr<T>(out), ptr<T>(q), (long)q.stride(0), ptr<T>(kpool), ptr<T>(vpool),             \
                     block_tables.data_ptr<int>(), (int)block_tables.stride(0), tok_seq.data_ptr<int>(),            \
                     positions.data_ptr<int>(), slp, gate.has_value() ? ptr<T>(*gate) : (const T*)nullptr, gstride, \
                     H, G, D, Dv, page_shift, (float)scale, (int)window, (int)keep_first, kvec,                      \
                     vvec_even & vvec_ok, (float)softcap, sink ? 1 : 0, vrow, vhead, x.sink_logits, x.dist_bias, x.dist_rows,      \
                     (const T*)x.ksum, (const T*)x.vsum, x.sum_shift, x.sum_block, x.cross_out)
  SERVING_DISPATCH_ACT(q, T, {
    if (rc == 4) { SCALAR_CASE(4); }
    else if (rc == 2) { SCALAR_CASE(2); }
    else { SCALAR_CASE(1); }
  });
#undef SCALAR_CASE
#undef SCALAR_LAUNCH
  HIP_CHECK_LAST();
}

// The matrix-core kernel for prompt portions in bfloat16 whose head sizes fit a tiling; false when it does not apply.
// In `x`, sink_logits and dist_bias are already in the base-2 domain (times log2 e), dist_bias one row per head.
static bool launch_mfma_attention(at::Tensor& out, const at::Tensor& q, const at::Tensor& kpool, const at::Tensor& vpool,
                                  const at::Tensor& block_tables, const at::Tensor& cu, const at::Tensor& start,
                                  const float* slp, const c10::optional<at::Tensor>& gate, long gstride, double scale,
                                  int64_t window, int64_t keep_first, double softcap, bool sink, int page_shift,
                                  int64_t num_tiles, int64_t num_tiles128, const ScalarExtras& x) {
  const int H = (int)q.size(1), D = (int)q.size(2);
  const int G = (int)kpool.size(2), Dv = (int)vpool.size(3);
  // prompt portions in bfloat16 go to the matrix cores when the head sizes fit a tiling;
  // num_tiles = sum over sequences of ceil(new tokens / 32), 0 asks for the scalar kernel
  const bool aligned = q.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0;
  // head sizes that are multiples of 8 ride in the next larger tiling, zero-padded
  const bool mfma_shape = D % 8 == 0 && Dv % 8 == 0 && D <= 128 && Dv <= 128;
  if (!(num_tiles > 0 && is_bf16(q) && aligned && mfma_shape && vpool.is_contiguous())) return false;
  {
    const int rep = H / G, nw = 4;
    // one query head per kv head: the waves of a block take four consecutive token tiles instead of four heads
    const int qsplit = (rep == 1 && num_tiles128 > 0) ? 1 : 0;
    const int VC = x.cross_out != nullptr ? G : 1;
    const dim3 grid((unsigned)(qsplit ? num_tiles128 : num_tiles), (unsigned)G, (unsigned)((rep + nw - 1) / nw * VC));
    const int ds = D <= 32 ? 2 : D <= 48 ? 3 : D <= 64 ? 4 : D <= 96 ? 6 : 8, vt = (Dv + 31) / 32;
    const size_t msmem = (size_t)2 * MFMA_TILES_PER_STEP * (32 * (ds * 16 + 8) + vt * 32 * 40) * sizeof(bf16s);
#define MFMA_CASE(DS_, VT_)                                                                                        \
  do {                                                                                                             \
    auto kfn = paged_attention_mfma_kernel<DS_, VT_>;                                                              \
    if (msmem > 65536) /* more dynamic LDS than a kernel gets without asking */                                    \
      (void)hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)msmem);         \
    hipLaunchKernelGGL(kfn, grid, dim3(64 * nw), msmem, stream(),                                                 \
                       x.cross_out != nullptr ? (bf16s*)nullptr : ptr<bf16s>(out), ptr<bf16s>(q),                  \
                       (long)q.stride(0), ptr<bf16s>(kpool), ptr<bf16s>(vpool), block_tables.data_ptr<int>(),      \
                       (int)block_tables.stride(0), cu.data_ptr<int>(), start.data_ptr<int>(), slp,                \
                       gate.has_value() ? ptr<bf16s>(*gate) : (const bf16s*)nullptr, gstride, H, G, D, Dv,         \
                       page_shift, (float)scale, (int)window, (int)keep_first, (float)softcap, sink ? 1 : 0,       \
                       qsplit, x.sink_logits, x.dist_bias, x.dist_rows, (const bf16s*)x.ksum,                      \
                       (const bf16s*)x.vsum, x.sum_shift, x.sum_block, x.cross_out);                               \
  } while (0)
#define MFMA_ROW(DS_)                     \
  do {                                    \
    if (vt == 1) MFMA_CASE(DS_, 1);       \
    else if (vt == 2) MFMA_CASE(DS_, 2);  \
    else if (vt == 3) MFMA_CASE(DS_, 3);  \
    else MFMA_CASE(DS_, 4);               \
  } while (0)
    if (ds == 2) MFMA_ROW(2);
    else if (ds == 3) MFMA_ROW(3);
    else if (ds == 4) MFMA_ROW(4);
    else if (ds == 6) MFMA_ROW(6);
    else MFMA_ROW(8);
#undef MFMA_ROW
#undef MFMA_CASE
    HIP_CHECK_LAST();
    return true;
  }
}

at::Tensor paged_attention(at::Tensor q, at::Tensor kpool, at::Tensor vpool, at::Tensor block_tables, at::Tensor cu,
                           at::Tensor start, at::Tensor tok_seq, at::Tensor positions, double scale, int64_t window,
                           int64_t keep_first, c10::optional<at::Tensor> slopes, c10::optional<at::Tensor> gate,
                           int64_t num_tiles, double softcap, bool sink, int64_t num_tiles128) {
  check_act(q, "q");
  TORCH_CHECK(softcap >= 0.0, "softcap must not be negative (0 = none)");
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && q.stride(1) == q.size(2), "q must be [N, H, D] with dense rows");
  // the value pool may be a view into wider rows (values that are leading channels of the keys): dense
  // channels, pages of `page` rows, any row and head stride
  TORCH_CHECK(kpool.dim() == 4 && vpool.dim() == 4 && kpool.is_contiguous() && vpool.stride(3) == 1 &&
              vpool.stride(0) == vpool.size(1) * vpool.stride(1), "pools must be [pages, page, G, D] with dense rows");
  TORCH_CHECK(kpool.scalar_type() == q.scalar_type() && vpool.scalar_type() == q.scalar_type(),
              "query and pools share one dtype");
  const long N = q.size(0);
  const int H = (int)q.size(1), D = (int)q.size(2);
  const int page = (int)kpool.size(1), G = (int)kpool.size(2), Dv = (int)vpool.size(3);
  TORCH_CHECK(kpool.size(3) == D && vpool.size(2) == G && vpool.size(1) == page && vpool.size(0) == kpool.size(0));
  TORCH_CHECK(H % G == 0 && Dv <= 512 && page > 0 && (page & (page - 1)) == 0);
  const long vrow = vpool.stride(1), vhead = G > 1 ? vpool.stride(2) : Dv;
  check_i32(block_tables, "block_tables"); check_i32(tok_seq, "tok_seq"); check_i32(positions, "positions");
  TORCH_CHECK(block_tables.dim() == 2 && tok_seq.numel() == N && positions.numel() == N);
  TORCH_CHECK(window >= 0 && keep_first >= 0);
  int page_shift = 0;
  while ((1 << page_shift) < page) ++page_shift;
  at::Tensor sl;
  const float* slp = nullptr;
  if (slopes.has_value()) {
    sl = f32c(*slopes);
    TORCH_CHECK(sl.numel() == H);
    slp = sl.data_ptr<float>();
  }
  long gstride = 0;
  if (gate.has_value()) {
    TORCH_CHECK(gate->scalar_type() == q.scalar_type() && gate->dim() == 2 && gate->size(0) == N &&
                gate->size(1) == H && gate->stride(1) == 1, "gate must be [N, H] of q's dtype");
    gstride = gate->stride(0);
  }
  at::Tensor out = at::empty({N, H, Dv}, q.options());
  if (N == 0) return out;
  check_i32(cu, "cu"); check_i32(start, "start");
  if (launch_mfma_attention(out, q, kpool, vpool, block_tables, cu, start, slp, gate, gstride, scale, window, keep_first,
                            softcap, sink, page_shift, num_tiles, num_tiles128, ScalarExtras()))
    return out;
  launch_scalar_attention(out, q, kpool, vpool, block_tables, tok_seq, positions, slp, gate, gstride, scale, window,
                          keep_first, softcap, sink, page_shift, vrow, vhead, ScalarExtras());
  return out;
}

// The split-key kernel with its optional extras, for prompt portions and decode tokens alike: a learned sink per
// head, a per-distance bias table, block summaries ahead of the window, and (cross) every query head's weights
// applied to every kv head's values, returned as float32 [N, H, G, Dv] for a talking-heads mix.
at::Tensor paged_attention_ext(at::Tensor q, at::Tensor kpool, at::Tensor vpool, at::Tensor block_tables, at::Tensor cu,
                               at::Tensor start, at::Tensor tok_seq, at::Tensor positions, double scale, int64_t window,
                               int64_t keep_first, c10::optional<at::Tensor> slopes, c10::optional<at::Tensor> gate,
                               double softcap, bool sink, c10::optional<at::Tensor> sink_logits,
                               c10::optional<at::Tensor> dist_bias, c10::optional<at::Tensor> ksum,
                               c10::optional<at::Tensor> vsum, int64_t sum_block, bool cross, int64_t num_tiles,
                               int64_t num_tiles128) {
  check_act(q, "q");
  TORCH_CHECK(softcap >= 0.0, "softcap must not be negative (0 = none)");
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && q.stride(1) == q.size(2), "q must be [N, H, D] with dense rows");
  TORCH_CHECK(kpool.dim() == 4 && vpool.dim() == 4 && kpool.is_contiguous() && vpool.is_contiguous(),
              "pools must be contiguous [pages, page, G, D]");
  TORCH_CHECK(kpool.scalar_type() == q.scalar_type() && vpool.scalar_type() == q.scalar_type(),
              "query and pools share one dtype");
  const long N = q.size(0);
  const int H = (int)q.size(1), D = (int)q.size(2);
  const int page = (int)kpool.size(1), G = (int)kpool.size(2), Dv = (int)vpool.size(3);
  TORCH_CHECK(kpool.size(3) == D && vpool.size(2) == G && vpool.size(1) == page && vpool.size(0) == kpool.size(0));
  TORCH_CHECK(H % G == 0 && Dv <= 512 && page > 0 && (page & (page - 1)) == 0);
  check_i32(block_tables, "block_tables"); check_i32(tok_seq, "tok_seq"); check_i32(positions, "positions");
  TORCH_CHECK(block_tables.dim() == 2 && tok_seq.numel() == N && positions.numel() == N);
  TORCH_CHECK(window >= 0 && keep_first >= 0);
  int page_shift = 0;
  while ((1 << page_shift) < page) ++page_shift;
  at::Tensor sl, sk, db;
  const float* slp = nullptr;
  if (slopes.has_value()) {
    sl = f32c(*slopes);
    TORCH_CHECK(sl.numel() == H);
    slp = sl.data_ptr<float>();
  }
  long gstride = 0;
  if (gate.has_value()) {
    TORCH_CHECK(gate->scalar_type() == q.scalar_type() && gate->dim() == 2 && gate->size(0) == N &&
                gate->size(1) == H && gate->stride(1) == 1, "gate must be [N, H] of q's dtype");
    gstride = gate->stride(0);
  }
  ScalarExtras x;
  if (sink_logits.has_value()) {
    sk = f32c(*sink_logits);
    TORCH_CHECK(sk.is_cuda() && sk.numel() == H, "sink_logits must be [H]");
    x.sink_logits = sk.data_ptr<float>();
  }
  if (dist_bias.has_value()) {
    db = f32c(*dist_bias);
    TORCH_CHECK(db.is_cuda() && db.dim() == 2 && db.size(1) == H && db.size(0) >= 1, "dist_bias must be [rows, H]");
    x.dist_bias = db.data_ptr<float>();
    x.dist_rows = (int)db.size(0);
  }
  if (ksum.has_value()) {
    TORCH_CHECK(vsum.has_value() && window > 0 && sum_block >= 1, "block summaries need both pools, a window and a block length");
    const int rows = (int)ksum->size(1);
    TORCH_CHECK(ksum->dim() == 4 && vsum->dim() == 4 && ksum->is_contiguous() && vsum->is_contiguous() &&
                ksum->scalar_type() == q.scalar_type() && vsum->scalar_type() == q.scalar_type() &&
                ksum->size(0) == kpool.size(0) && vsum->size(0) == kpool.size(0) && vsum->size(1) == rows &&
                ksum->size(2) == G && ksum->size(3) == D && vsum->size(2) == G && vsum->size(3) == Dv &&
                rows > 0 && (rows & (rows - 1)) == 0 && (long)rows * sum_block >= page,
                "summary pools must be [pages, rows, G, D] / [.., Dv] of the pools' type, rows a power of two with "
                "rows * block >= page size");
    while ((1 << x.sum_shift) < rows) ++x.sum_shift;
    x.sum_block = (int)sum_block;
    x.ksum = ksum->data_ptr();
    x.vsum = vsum->data_ptr();
  }
  at::Tensor out = cross ? at::empty({N, H, G, Dv}, q.options().dtype(at::kFloat)) : at::empty({N, H, Dv}, q.options());
  if (N == 0) return out;
  if (cross) x.cross_out = out.data_ptr<float>();
  if (num_tiles > 0 && is_bf16(q)) {  // prompt portions in bfloat16: the matrix-core kernel, extras in the base-2 domain
    check_i32(cu, "cu"); check_i32(start, "start");
    constexpr double LOG2E = 1.4426950408889634;
    ScalarExtras x2 = x;
    at::Tensor sk2, db2;
    if (sink_logits.has_value()) {
      sk2 = sk * LOG2E;
      x2.sink_logits = sk2.data_ptr<float>();
    }
    if (dist_bias.has_value()) {
      db2 = (db * LOG2E).t().contiguous();   // [H, rows]
      x2.dist_bias = db2.data_ptr<float>();
    }
    if (launch_mfma_attention(out, q, kpool, vpool, block_tables, cu, start, slp, gate, gstride, scale, window,
                              keep_first, softcap, sink, page_shift, num_tiles, num_tiles128, x2))
      return out;
  }
  launch_scalar_attention(out, q, kpool, vpool, block_tables, tok_seq, positions, slp, gate, gstride, scale, window,
                          keep_first, softcap, sink, page_shift, (long)vpool.stride(1), (long)vpool.stride(2), x);
  return out;
}

// ------------------------------------------------------------------ block summaries
// One wave per (sequence, block completed in this step, kv head): the float32 mean of the block's `block` cached
// key rows and value rows goes to row b of the summary pools (page bt[b >> sum_shift], row b & mask).
template <typename T>
__global__ __launch_bounds__(64) void paged_pool_write_kernel(
    T* __restrict__ ksum, T* __restrict__ vsum, const T* __restrict__ kpool, const T* __restrict__ vpool,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ cu, const int* __restrict__ start,
    int G, int D, int Dv, int page_shift, int sum_shift, int block) {
  const int b = blockIdx.x, g = blockIdx.z;
  const int s0 = start[b], n = cu[b + 1] - cu[b];
  const int blk = s0 / block + (int)blockIdx.y;
  if (blk >= (s0 + n) / block) return;
  const int* bt = block_tables + (long)b * bt_stride;
  const int page_mask = (1 << page_shift) - 1, sum_mask = (1 << sum_shift) - 1;
  const long srow = ((long)bt[blk >> sum_shift] << sum_shift) + (blk & sum_mask);
  const float inv = 1.0f / (float)block;
  for (int d = threadIdx.x; d < D + Dv; d += 64) {
    const bool key = d < D;
    float acc = 0.0f;
    for (int i = 0; i < block; ++i) {
      const int j = blk * block + i;
      const long row = ((long)bt[j >> page_shift] << page_shift) + (j & page_mask);
      acc += key ? ldf(kpool + (row * G + g) * D + d) : ldf(vpool + (row * G + g) * Dv + (d - D));
    }
    if (key) stf(ksum + (srow * G + g) * D + d, acc * inv);
    else stf(vsum + (srow * G + g) * Dv + (d - D), acc * inv);
  }
}

void paged_pool_write(at::Tensor kpool, at::Tensor vpool, at::Tensor ksum, at::Tensor vsum, at::Tensor block_tables,
                      at::Tensor cu, at::Tensor start, int64_t block, int64_t most_blocks) {
  check_act(kpool, "kpool");
  TORCH_CHECK(kpool.dim() == 4 && vpool.dim() == 4 && ksum.dim() == 4 && vsum.dim() == 4 && kpool.is_contiguous() &&
              vpool.is_contiguous() && ksum.is_contiguous() && vsum.is_contiguous(), "pools must be contiguous");
  TORCH_CHECK(vpool.scalar_type() == kpool.scalar_type() && ksum.scalar_type() == kpool.scalar_type() &&
              vsum.scalar_type() == kpool.scalar_type(), "pools share one dtype");
  const int page = (int)kpool.size(1), G = (int)kpool.size(2), D = (int)kpool.size(3), Dv = (int)vpool.size(3);
  const int rows = (int)ksum.size(1);
  TORCH_CHECK(ksum.size(0) == kpool.size(0) && vsum.size(0) == kpool.size(0) && vsum.size(1) == rows &&
              ksum.size(2) == G && ksum.size(3) == D && vsum.size(2) == G && vsum.size(3) == Dv && vpool.size(2) == G &&
              vpool.size(1) == page, "summary pools do not fit the pools");
  TORCH_CHECK(block >= 1 && rows > 0 && (rows & (rows - 1)) == 0 && (page & (page - 1)) == 0 &&
              (long)rows * block >= page, "rows per page: a power of two with rows * block >= page size");
  check_i32(block_tables, "block_tables"); check_i32(cu, "cu"); check_i32(start, "start");
  const int B = (int)start.numel();
  if (B == 0 || most_blocks <= 0) return;
  int page_shift = 0, sum_shift = 0;
  while ((1 << page_shift) < page) ++page_shift;
  while ((1 << sum_shift) < rows) ++sum_shift;
  SERVING_DISPATCH_ACT(kpool, T, {
    hipLaunchKernelGGL(paged_pool_write_kernel<T>, dim3((unsigned)B, (unsigned)most_blocks, (unsigned)G), dim3(64), 0,
                       stream(), ptr<T>(ksum), ptr<T>(vsum), ptr<T>(kpool), ptr<T>(vpool), block_tables.data_ptr<int>(),
                       (int)block_tables.stride(0), cu.data_ptr<int>(), start.data_ptr<int>(), G, D, Dv, page_shift,
                       sum_shift, (int)block);
  });
  HIP_CHECK_LAST();
}

}  // namespace serving
}  // namespace cai

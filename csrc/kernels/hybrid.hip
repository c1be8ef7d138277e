// Kernels of hybrid decoder designs: an fp32 residual stream with scalar-gain RMS norms on the
// sublayer outputs, gated recurrences whose state lives in per-sequence fp32 slots (minGRU,
// gated linear attention), attention with separate key / value widths under a chunk or window
// mask over a paged cache, and a shape-agnostic GEMM for the projections that the MFMA kernels
// (gemm*.hip: bf16, K a multiple of 64) do not take, including every product of the true-fp32
// mode. Everything a recurrence or a softmax touches is fp32; only tensors that feed the next
// matrix product are written in the activation type (bf16 or fp32, a launch-time flag).
// Pre-norm designs add: a residual step fused with a per-coordinate RMS norm or with a Dynamic Tanh
// norm, latent attention's cached row, matrix memories, per-head products, gated units (plain and
// clamped), and attention whose values are its keys before they rotate in neighbouring pairs.
// The two attention kernels take options that further designs combine: row strides of the planes (values that are a
// column block of the key rows), a cap on the scores, a sink in the softmax, several value heads under one head's weights.
//
// A step's sequences are described by cu_q [B+1] (row ranges), positions [T] and slots [B]
// (state slot of the sequence; < 0: padding row of a recorded step, skipped). A sequence whose
// first row is at position 0 starts from a zero state, so slots are never cleared.
#include "hybrid_common.h"

namespace {

// ---------------------------------------------------------------- embedding -> fp32 stream (+ activation copy)
template <bool EF32, bool AF32>
__global__ void embed_rows_kernel(const int32_t* __restrict__ ids, const void* __restrict__ E, float* __restrict__ x,
                                  void* __restrict__ xa, int T, int d, int vocab, const int32_t* __restrict__ feed_tok,
                                  const int32_t* __restrict__ feed_rows, float scale,
                                  const int32_t* __restrict__ positions, const double* __restrict__ inv_freq) {
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= T) return;
  int id = ids[row];
  if (feed_rows != nullptr) {
    const int src = feed_rows[row];
    if (src >= 0) id = feed_tok[src];
  }
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const typename Act<EF32>::type* e = static_cast<const typename Act<EF32>::type*>(E) + static_cast<size_t>(id) * d;
  typename Act<AF32>::type* a = static_cast<typename Act<AF32>::type*>(xa);
  // optional sinusoidal position vector: entry 2i = sin(p f_i), entry 2i + 1 = cos(p f_i), f an fp64 table
  if (inv_freq != nullptr) {                      // a lane owns the (sin, cos) pair of one angle; d is even
    // the angle p * f and its reduction to [-pi, pi] in fp64 (thousands of radians would cost an fp32
    // angle four digits), sine and cosine of the reduced angle in fp32
    const double pos = static_cast<double>(positions[row]);
    for (int i = lane; 2 * i < d; i += 64) {
      const double ang = pos * inv_freq[i];
      const double red = ang - 6.283185307179586476925 * rint(ang * 0.159154943091895335769);
      float sn, cs;
      sincosf(static_cast<float>(red), &sn, &cs);
      const float v0 = Act<EF32>::load(e, 2 * i) * scale + sn, v1 = Act<EF32>::load(e, 2 * i + 1) * scale + cs;
      *reinterpret_cast<float2*>(x + static_cast<size_t>(row) * d + 2 * i) = make_float2(v0, v1);
      if (a != nullptr) {
        Act<AF32>::store(a, static_cast<size_t>(row) * d + 2 * i, v0);
        Act<AF32>::store(a, static_cast<size_t>(row) * d + 2 * i + 1, v1);
      }
    }
    return;
  }
  for (int c = lane; c < d; c += 64) {
    const float v = Act<EF32>::load(e, c) * scale;
    x[static_cast<size_t>(row) * d + c] = v;
    if (a != nullptr) Act<AF32>::store(a, static_cast<size_t>(row) * d + c, v);
  }
}

// ---------------------------------------------------------------- scalar-gain RMS norm of a sublayer output
// With y: x += y * rsqrt(mean(y^2) + eps) * gain, xa = x. Without: xa = x * rsqrt(mean(x^2) + eps) * gain.
// WAVES = 1: one wave per row, four rows per block (many rows: bandwidth-bound). WAVES = 4: one
// block per row (decode steps: few rows, latency-bound, so a row is spread over 256 lanes).
template <bool AF32, int WAVES>
__global__ __launch_bounds__(256) void scalar_norm_add_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                              const float* __restrict__ gain, float eps,
                                                              void* __restrict__ xa, int T, int d) {
  __shared__ float red[16];
  constexpr int LANES = 64 * WAVES;
  const int row = WAVES == 1 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  const int lane = WAVES == 1 ? (threadIdx.x & 63) : threadIdx.x;
  if (WAVES == 1 && row >= T) return;
  float* xr = x + static_cast<size_t>(row) * d;
  const float* src = y != nullptr ? y + static_cast<size_t>(row) * d : xr;
  const float g = gain[0];
  float ss = 0.f;
  for (int c = lane; c < d; c += LANES) {
    const float v = src[c];
    ss += v * v;
  }
  ss = WAVES == 1 ? wave_sum(ss) : block_sum(ss, red);
  const float r = g / sqrtf(ss / static_cast<float>(d) + eps);
  typename Act<AF32>::type* a = static_cast<typename Act<AF32>::type*>(xa);
  for (int c = lane; c < d; c += LANES) {
    float v = src[c] * r;
    if (y != nullptr) {
      v += xr[c];
      xr[c] = v;
    }
    if (a != nullptr) Act<AF32>::store(a, static_cast<size_t>(row) * d + c, v);
  }
}

// out [T, cols] = relu(y[:, :cols])^2 for y of row stride ld.
template <bool AF32>
__global__ void relu2_kernel(const float* __restrict__ y, void* __restrict__ out, long long n, int cols, int ld) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long long t = i / cols;
  const float v = fmaxf(y[t * ld + (i - t * cols)], 0.f);
  Act<AF32>::store(static_cast<typename Act<AF32>::type*>(out), i, v * v);
}

// ---------------------------------------------------------------- minGRU
// zxg [T, 3w]: update-gate logits | candidate pre-activations | output-gate logits.
// One thread per (sequence, channel); the recurrence runs over the sequence's rows in order.
// Long portions are cut into segments of seg_len rows that run side by side (blockIdx.z):
//   mode 1  every segment scans its rows from zero and leaves (product of (1 - z), local result)
//           in ``carry`` [B, nseg, 2, w];
//   mode 2  every segment folds the pairs of the segments before it onto the sequence's state
//           (S <- a S + b is associative), scans its rows again from there and writes the outputs;
//           the last segment stores the state.
// mode 0 is the whole sequence in one go (decoded tokens, short portions): nseg = 1, no carry.
template <bool AF32>
__global__ void mingru_scan_kernel(const float* __restrict__ zxg, float* __restrict__ state,
                                   const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
                                   const int32_t* __restrict__ slots, void* __restrict__ out, int w, int mode,
                                   int seg_len, float* __restrict__ carry) {
  const int b = blockIdx.y;
  const int seg = blockIdx.z, nseg = gridDim.z;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int slot = slots[b];
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (c >= w || slot < 0 || q1 <= q0) return;
  const int r0 = mode == 0 ? q0 : q0 + seg * seg_len;
  const int r1 = mode == 0 ? q1 : min(q1, r0 + seg_len);
  if (r0 >= q1) return;
  float* cb = carry != nullptr ? carry + static_cast<size_t>(b) * nseg * 2 * w : nullptr;
  float S = 0.f, A = 1.f;
  if (mode != 1) {
    S = positions[q0] == 0 ? 0.f : state[static_cast<size_t>(slot) * w + c];
    for (int k = 0; k < seg && mode == 2; ++k)
      S = cb[(static_cast<size_t>(k) * 2) * w + c] * S + cb[(static_cast<size_t>(k) * 2 + 1) * w + c];
  }
  typename Act<AF32>::type* o = static_cast<typename Act<AF32>::type*>(out);
  for (int t = r0; t < r1; ++t) {
    const float* row = zxg + static_cast<size_t>(t) * 3 * w;
    const float z = sigmoidf_(row[c]);
    const float u = row[w + c];
    const float cand = u >= 0.f ? u + 0.5f : sigmoidf_(u);
    S = (1.f - z) * S + z * cand;
    if (mode == 1) A *= 1.f - z;
    else Act<AF32>::store(o, static_cast<size_t>(t) * w + c, S * siluf_(row[2 * w + c]));
  }
  if (mode == 1) {
    cb[(static_cast<size_t>(seg) * 2) * w + c] = A;
    cb[(static_cast<size_t>(seg) * 2 + 1) * w + c] = S;
  } else if (r1 == q1) {
    state[static_cast<size_t>(slot) * w + c] = S;
  }
}

// ---------------------------------------------------------------- gated linear attention
// proj [T, ld]: q | k | v at columns 0, H*D, 2*H*D; decay [T, H*D] logits. One block per
// (value-column tile of 64, head, sequence x segment); thread dv keeps column dv of the head's
// state S [D, Dv] in registers (DMAX >= D). q, k and the decay come prepared (gla_prepare_kernel);
// per token S = a * S + k v^T, o = S^T q.
// Long portions run as segments of seg_len rows side by side, in three passes:
//   scan_segment_state_kernel: what each segment's rows alone add to the state (from zero) goes to
//           ``cs`` [B, nseg, H, D, Dv] and the product of its decays to ``ca`` [B, nseg, H, D]. No
//           outputs are needed here, so every state ELEMENT is its own short recurrence and a
//           thread owns a few of them: thousands of independent chains instead of one per column;
//   gla_carry_kernel turns the local states into each segment's incoming state, in place;
//   mode 2  each segment starts from its incoming state, writes its outputs; the last one stores
//           the sequence's state.
// mode 0: the whole sequence in one block (decoded tokens, short portions).
// Everything the recurrence reads per (token, head, key channel), computed once and in parallel:
// (q / sqrt(D), k, decay, -) with decay = sigmoid(logit)^(1/tau) = exp(log_sigmoid(logit) / tau).
__global__ void gla_prepare_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ decay,
                                   float4* __restrict__ prep, long long n, int HD, float inv_tau, float qscale) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long long t = i / HD;
  const int c = static_cast<int>(i - t * HD);
  const float* row = proj + t * ld;
  const float z = decay[i];
  const float a = expf(logsigmoidf_(z) * inv_tau);
  prep[i] = make_float4(row[c] * qscale, row[HD + c], a, 0.f);
}

template <int DMAX>
__global__ __launch_bounds__(64) void gla_scan_kernel(const float* __restrict__ proj, int ld,
                                                      const float4* __restrict__ prep, float* __restrict__ state,
                                                      const int32_t* __restrict__ cu_q,
                                                      const int32_t* __restrict__ positions,
                                                      const int32_t* __restrict__ slots, float* __restrict__ out, int H,
                                                      int D, int Dv, int mode, int nseg, int seg_len,
                                                      const float* __restrict__ cs, long long state_stride, int ones) {
  const int b = blockIdx.z / nseg, seg = blockIdx.z % nseg, h = blockIdx.y;
  const int dv = blockIdx.x * 64 + threadIdx.x;
  const int slot = slots[b];
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (slot < 0 || q1 <= q0) return;
  const int r0 = mode == 0 ? q0 : q0 + seg * seg_len;
  const int r1 = mode == 0 ? q1 : min(q1, r0 + seg_len);
  if (r0 >= q1) return;
  const bool live = dv < Dv;
  float S[DMAX];
  float* st = state + static_cast<size_t>(slot) * state_stride + static_cast<size_t>(h) * D * Dv;
  const int Dvr = Dv - ones;                      // value columns that come from the projection
  const float* seg_s = cs != nullptr ? cs + ((static_cast<size_t>(b) * nseg + seg) * H + h) * D * Dv : nullptr;
  const float* from = mode == 2 ? seg_s : st;
  const bool zero = mode == 0 && positions[q0] == 0;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (!zero && live && d < D) ? from[static_cast<size_t>(d) * Dv + dv] : 0.f;
  // Lane j of the wave loads the prepared operands of key channels j, j + 64, ... of the token (one
  // coalesced 16-byte load per lane, the next token's in flight during the current one); the
  // channel loop then broadcasts them lane by lane (v_readlane) to meet every lane's state column.
  // No LDS, no barrier.
  constexpr int NCH = (DMAX + 63) / 64;
  float4 cur[NCH], nxt[NCH];
  float vcur, vnxt = 0.f;
  auto fetch = [&](int t, float4* dst, float& vv) {
    const float4* x = prep + (static_cast<size_t>(t) * H + h) * D;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int d = threadIdx.x + 64 * i;
      dst[i] = d < D ? x[d] : make_float4(0.f, 0.f, 1.f, 0.f);
    }
    vv = !live ? 0.f : (dv < Dvr ? proj[static_cast<size_t>(t) * ld + 2 * H * D + h * Dvr + dv] : 1.f);
  };
  fetch(r0, nxt, vnxt);
  for (int t = r0; t < r1; ++t) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) cur[i] = nxt[i];
    vcur = vnxt;
    if (t + 1 < r1) fetch(t + 1, nxt, vnxt);
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
#pragma unroll
      for (int j = 0; j < 64; ++j) {
        const int d = 64 * i + j;
        if (d < DMAX && d < D) {
          const float qd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cur[i].x), j));
          const float kd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cur[i].y), j));
          const float ad = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cur[i].z), j));
          S[d] = ad * S[d] + kd * vcur;
          o += S[d] * qd;
        }
      }
    }
    if (live) out[static_cast<size_t>(t) * H * Dv + h * Dv + dv] = o;
  }
  if (live && r1 == q1) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < D) st[static_cast<size_t>(d) * Dv + dv] = S[d];
  }
}

// A segment's own contribution to the state, from zero: cs[d, dv] = sum_t (prod_{r > t} a_r[d]) k_t[d] v_t[dv] over
// its rows, and ca[d] = prod_t a_t[d]. One block per (tile of 32 key channels x 128 value columns, head,
// sequence x segment); the segment's operands are staged in LDS once (seg_len <= kSegRows), a thread
// owns 4 x 4 state elements and walks the rows: acc <- a acc + k v.
constexpr int kSegRows = 64, kSegD = 32, kSegV = 128;

__global__ __launch_bounds__(256) void scan_segment_state_kernel(
    const float* __restrict__ proj, int ld, const float4* __restrict__ prep, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ slots, int H, int D, int Dv, int nseg, int seg_len, float* __restrict__ cs,
    float* __restrict__ ca, int ones) {
  __shared__ float2 ka[kSegRows][kSegD];            // (k, a) of the tile's key channels
  __shared__ float vs[kSegRows][kSegV];
  const int b = blockIdx.z / nseg, seg = blockIdx.z % nseg, h = blockIdx.y;
  const int ndt = (D + kSegD - 1) / kSegD;
  const int d0 = (blockIdx.x % ndt) * kSegD, v0 = (blockIdx.x / ndt) * kSegV;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (slots[b] < 0 || q1 <= q0) return;
  const int r0 = q0 + seg * seg_len;
  if (r0 >= q1) return;                               // the same for the whole block
  const int n = min(seg_len, q1 - r0);
  const int Dvr = Dv - ones;
  for (int i = threadIdx.x; i < kSegRows * kSegD; i += 256) {
    const int t = i / kSegD, d = d0 + i % kSegD;
    float2 e = make_float2(0.f, 1.f);                 // rows and channels past the end change nothing
    if (t < n && d < D) {
      const float4 x = prep[(static_cast<size_t>(r0 + t) * H + h) * D + d];
      e = make_float2(x.y, x.z);
    }
    ka[t][i % kSegD] = e;
  }
  for (int i = threadIdx.x; i < kSegRows * kSegV; i += 256) {
    const int t = i / kSegV, dv = v0 + i % kSegV;
    float v = 0.f;
    if (t < n && dv < Dv) v = dv < Dvr ? proj[static_cast<size_t>(r0 + t) * ld + 2 * H * D + h * Dvr + dv] : 1.f;
    vs[t][i % kSegV] = v;
  }
  __syncthreads();
  const int td = (threadIdx.x >> 5) * 4, tv = threadIdx.x & 31;   // channels td .. td + 3, columns tv + 32 j
  float acc[4][4] = {};
  float ap[4] = {1.f, 1.f, 1.f, 1.f};
  for (int t = 0; t < n; ++t) {
    float vv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) vv[j] = vs[t][tv + 32 * j];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float2 e = ka[t][td + i];
      ap[i] *= e.y;
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = e.y * acc[i][j] + e.x * vv[j];
    }
  }
  float* out = cs + ((static_cast<size_t>(b) * nseg + seg) * H + h) * D * Dv;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = d0 + td + i;
    if (d >= D) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int dv = v0 + tv + 32 * j;
      if (dv < Dv) out[static_cast<size_t>(d) * Dv + dv] = acc[i][j];
    }
    if (v0 == 0 && tv == 0) ca[((static_cast<size_t>(b) * nseg + seg) * H + h) * D + d] = ap[i];
  }
}

// Between the two segment passes: cs[b, s] holds segment s's local state on entry and the state the
// segment STARTS from on exit (the sequence's own state for s = 0). One thread per state element.
__global__ void gla_carry_kernel(float* __restrict__ cs, const float* __restrict__ ca, const float* __restrict__ state,
                                 const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
                                 const int32_t* __restrict__ slots, int H, int D, int Dv, int nseg, int seg_len,
                                 long long state_stride) {
  const int b = blockIdx.y;
  const size_t n = static_cast<size_t>(H) * D * Dv;
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int slot = slots[b];
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (i >= n || slot < 0 || q1 <= q0) return;
  const size_t hd = i / Dv;                         // (head, key channel)
  float carry = positions[q0] == 0 ? 0.f : state[static_cast<size_t>(slot) * state_stride + i];
  const int used = (q1 - q0 + seg_len - 1) / seg_len;
  for (int s = 0; s < used; ++s) {
    float* p = cs + (static_cast<size_t>(b) * nseg + s) * n + i;
    const float local = *p;
    *p = carry;
    carry = ca[(static_cast<size_t>(b) * nseg + s) * H * D + hd] * carry + local;
  }
}

// Per head: o / sqrt(mean(o^2) + eps) * w, times act(gate). One wave per (row, head). Heads are
// ``ld_head`` apart in o (>= Dv); head h reads the weights w[h * w_stride ...] (w_stride 0: one
// weight vector for all heads); act is silu (gate_kind 0) or sigmoid (1). With ``m`` [T, H] the
// read-out is first divided by max(|o[Dv]|, exp(-m)) + 1e-6, o[Dv] being the column behind the head's values
// (a matrix memory's normaliser . q, m its running maximum).
template <bool AF32>
__global__ void headnorm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                     const float* __restrict__ gate, int ld_gate, void* __restrict__ out, int T, int H,
                                     int Dv, float eps, int ld_head, int w_stride, int gate_kind,
                                     const float* __restrict__ m) {
  const int idx = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (idx >= T * H) return;
  const int row = idx / H, h = idx % H;
  const float* orow = o + (static_cast<size_t>(row) * H + h) * ld_head;
  const float* grow = gate + static_cast<size_t>(row) * ld_gate + h * Dv;
  const float* wh = w + static_cast<size_t>(h) * w_stride;
  float inv = 1.f;
  if (m != nullptr) inv = 1.f / (fmaxf(fabsf(orow[Dv]), expf(-m[idx])) + 1e-6f);
  float ss = 0.f;
  for (int c = lane; c < Dv; c += 64) {
    const float v = orow[c] * inv;
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float r = inv / sqrtf(ss / static_cast<float>(Dv) + eps);
  typename Act<AF32>::type* dst = static_cast<typename Act<AF32>::type*>(out);
  for (int c = lane; c < Dv; c += 64) {
    const float g = grow[c];
    Act<AF32>::store(dst, static_cast<size_t>(row) * H * Dv + h * Dv + c,
                     orow[c] * r * wh[c] * (gate_kind == 0 ? siluf_(g) : sigmoidf_(g)));
  }
}

// ---------------------------------------------------------------- mLSTM: gates and prepared operands
// proj [T, ld]: q | k | v | output gate | input-gate logits [H] | forget-gate logits [H]. Per head, with
// i = cap tanh(. / cap) and f = log sigmoid(cap tanh(. / cap)) (cap 0: no cap), the running maximum
// m_t = max(f_t + m_(t-1), i_t) (0 before the first token) stabilises
//   S_t = a_t S_(t-1) + b_t k_t v_t^T,  a_t = exp(f_t + m_(t-1) - m_t),  b_t = exp(i_t - m_t).
// One wave per (head, sequence): 64 tokens at a time, the lanes compute the gates of their tokens and
// the maxima come from a wave scan (m -> max(m + F, I) composes as (F1 + F2, max(I1 + F2, I2))).
// Writes (a, b) per (token, head), m per (token, head), and the sequence's last m behind its state.
LC_DEVICE float soft_cap(float x, float cap) { return cap > 0.f ? cap * tanhf(x / cap) : x; }

__global__ __launch_bounds__(64) void mlstm_gates_kernel(const float* __restrict__ proj, int ld, int col_i,
                                                         float* __restrict__ state, long long state_stride,
                                                         long long m_offset, const int32_t* __restrict__ cu_q,
                                                         const int32_t* __restrict__ positions,
                                                         const int32_t* __restrict__ slots, float2* __restrict__ gates,
                                                         float* __restrict__ m_out, int H, float cap) {
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const int slot = slots[b];
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (slot < 0 || q1 <= q0) return;
  float* ms = state + static_cast<size_t>(slot) * state_stride + m_offset + h;
  float m = positions[q0] == 0 ? 0.f : *ms;
  for (int r0 = q0; r0 < q1; r0 += 64) {
    const int t = r0 + lane;
    const bool valid = t < q1;
    const float iv = valid ? soft_cap(proj[static_cast<size_t>(t) * ld + col_i + h], cap) : -INFINITY;
    const float fv = valid ? logsigmoidf_(soft_cap(proj[static_cast<size_t>(t) * ld + col_i + H + h], cap)) : 0.f;
    float F = fv, I = iv;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float Fp = __shfl_up(F, off, 64), Ip = __shfl_up(I, off, 64);
      if (lane >= off) {
        I = fmaxf(Ip + F, I);
        F = Fp + F;
      }
    }
    const float mt = fmaxf(m + F, I);
    float mp = __shfl_up(mt, 1, 64);
    if (lane == 0) mp = m;
    if (valid) {
      gates[static_cast<size_t>(t) * H + h] = make_float2(expf(fv + mp - mt), expf(iv - mt));
      m_out[static_cast<size_t>(t) * H + h] = mt;
    }
    m = __shfl(mt, min(63, q1 - 1 - r0), 64);
  }
  if (lane == 0) *ms = m;
}

// (q / sqrt(D), b k, a, -) per (token, head, key channel): the operands of the scan below.
__global__ void mlstm_prepare_kernel(const float* __restrict__ proj, int ld, const float2* __restrict__ gates,
                                     float4* __restrict__ prep, long long n, int H, int D, float qscale) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int HD = H * D;
  const long long t = i / HD;
  const int c = static_cast<int>(i - t * HD);
  const float* row = proj + t * ld;
  const float2 g = gates[t * H + c / D];
  prep[i] = make_float4(row[c] * qscale, row[HD + c] * g.y, g.x, 0.f);
}

// ---------------------------------------------------------------- pre-norm residual step
// x += y (when y is given), xa = x * rsqrt(mean(x^2) + eps) * w (when w is given). WAVES as in the
// scalar-gain kernel above.
template <bool AF32, int WAVES>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                          const float* __restrict__ w, float eps,
                                                          void* __restrict__ xa, int T, int d) {
  __shared__ float red[16];
  constexpr int LANES = 64 * WAVES;
  const int row = WAVES == 1 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  const int lane = WAVES == 1 ? (threadIdx.x & 63) : threadIdx.x;
  if (WAVES == 1 && row >= T) return;
  float* xr = x + static_cast<size_t>(row) * d;
  const float* yr = y != nullptr ? y + static_cast<size_t>(row) * d : nullptr;
  float ss = 0.f;
  for (int c = lane; c < d; c += LANES) {
    float v = xr[c];
    if (yr != nullptr) {
      v += yr[c];
      xr[c] = v;
    }
    ss += v * v;
  }
  if (w == nullptr) return;                         // the same for every thread
  ss = WAVES == 1 ? wave_sum(ss) : block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / static_cast<float>(d) + eps);
  typename Act<AF32>::type* a = static_cast<typename Act<AF32>::type*>(xa);
  for (int c = lane; c < d; c += LANES) Act<AF32>::store(a, static_cast<size_t>(row) * d + c, xr[c] * r * w[c]);
}

// act(gate) * up of y [T, 2n] = (gate | up); act: relu (kind 0) or silu (1).
template <bool AF32>
__global__ void glu_kernel(const float* __restrict__ y, void* __restrict__ out, long long total, int n, int kind) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long long t = i / n;
  const int c = static_cast<int>(i - t * n);
  const float g = y[t * 2 * n + c], u = y[t * 2 * n + n + c];
  Act<AF32>::store(static_cast<typename Act<AF32>::type*>(out), i, (kind == 0 ? fmaxf(g, 0.f) : siluf_(g)) * u);
}

// ---------------------------------------------------------------- residual step with a Dynamic Tanh norm
// x += mult * y (when y is given); then, when an output is given, out = tanh(alpha * x) * w + b (w given) or
// out = x (no w: the stream itself in the activation type). Nothing is reduced over a row, so a thread owns V
// neighbouring coordinates (V = 4 when the width allows 16-byte accesses). ``ldo``: row stride of ``out``
// (a column block of a wider matrix).
template <bool AF32, int V>
__global__ void add_dyt_kernel(float* __restrict__ x, const float* __restrict__ y, float mult, float alpha,
                               const float* __restrict__ w, const float* __restrict__ b, void* __restrict__ out, int ldo,
                               long long total, int d) {
  const long long i = (static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x) * V;
  if (i >= total) return;
  const long long t = i / d;
  const int c = static_cast<int>(i - t * d);
  float v[V];
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = x[i + e];
  if (y != nullptr) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      v[e] += mult * y[i + e];
      x[i + e] = v[e];
    }
  }
  if (out == nullptr) return;
  typename Act<AF32>::type* o = static_cast<typename Act<AF32>::type*>(out);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float r = w != nullptr ? tanhf(alpha * v[e]) * w[c + e] + b[c + e] : v[e];
    Act<AF32>::store(o, static_cast<size_t>(t) * ldo + c + e, r);
  }
}

// Clamped gated unit of y = (gate | up) columns of an fp32 matrix: g = min(s * gate, limit),
// u = clamp(s * up, -limit, limit), out = g * sigmoid(slope * g) * (u + shift). Row r of the work list is
// row slot_of[r] of y and of out with s = wts[r] (expert-sorted rows of a routed feed-forward, whose
// weight scales the expert's INPUT: the products are linear, so the scale is applied to them), or row r
// itself with s = 1 when no list is given.
template <bool AF32>
__global__ void glu_clamped_kernel(const float* __restrict__ y, int ld, int col_gate, int col_up, int n, float limit,
                                   float slope, float shift, const int32_t* __restrict__ slot_of,
                                   const float* __restrict__ wts, void* __restrict__ out, long long total) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long long r = i / n;
  const int c = static_cast<int>(i - r * n);
  const long long p = slot_of != nullptr ? slot_of[r] : r;
  const float s = wts != nullptr ? wts[r] : 1.f;
  const float* row = y + p * ld;
  const float g = fminf(row[col_gate + c] * s, limit);
  const float u = fminf(fmaxf(row[col_up + c] * s, -limit), limit);
  Act<AF32>::store(static_cast<typename Act<AF32>::type*>(out), static_cast<size_t>(p) * n + c,
                   g * sigmoidf_(slope * g) * (u + shift));
}

// ---------------------------------------------------------------- latent attention: the cached row
// One wave per token: c = rms_norm(proj[t, col0 : col0 + R]) * w goes to cache [blocks, 1, BS, R] at the
// token's slot.
template <bool CF32>
__global__ void latent_write_kernel(const float* __restrict__ proj, int ld, int col0, int R, const float* __restrict__ w,
                                    float eps, const int32_t* __restrict__ slot_mapping, void* __restrict__ cache,
                                    int BS, int T) {
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= T) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const float* row = proj + static_cast<size_t>(t) * ld + col0;
  float ss = 0.f;
  for (int c = lane; c < R; c += 64) ss += row[c] * row[c];
  ss = wave_sum(ss);
  const float r = 1.f / sqrtf(ss / static_cast<float>(R) + eps);
  typename Act<CF32>::type* dst = static_cast<typename Act<CF32>::type*>(cache);
  for (int c = lane; c < R; c += 64) Act<CF32>::store(dst, static_cast<size_t>(slot) * R + c, row[c] * r * w[c]);
}

// ---------------------------------------------------------------- attention: norms, rotation, cache write
// One block per token. qkv [T, ld] fp32: q [H*D] | k [G*D] | v [G*Dv]. q and k are RMS-normed over
// their whole projection (weights qn, kn), the first rot_dims coordinates of each head rotate by
// position * inv_freq[i] (coordinate i with i + rot_dims/2), each value head is scaled to unit RMS.
template <bool CF32>
__global__ __launch_bounds__(256) void qkv_prep_kernel(
    const float* __restrict__ qkv, int ld, const float* __restrict__ qn, const float* __restrict__ kn,
    const float* __restrict__ inv_freq, const int32_t* __restrict__ positions, const int32_t* __restrict__ slot_mapping,
    void* __restrict__ kc, void* __restrict__ vc, float* __restrict__ q_out, int H, int G, int D, int Dv, int BS,
    int rot_dims, float eps, int has_kv) {
  __shared__ float red[16];
  __shared__ float cs_tab[2][128];                 // cos / sin of the token's angles (rot_dims / 2 <= 128 of them)
  const int t = blockIdx.x;
  const float* row = qkv + static_cast<size_t>(t) * ld;
  const float pos = static_cast<float>(positions[t]);
  const int half = rot_dims >> 1;
  const int nq = H * D, nk = G * D;
  const bool tab = half <= 128;                    // the same angles serve every head: computed once per token
  if (tab)
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
      const float ang = pos * inv_freq[j];
      cs_tab[0][j] = cosf(ang);
      cs_tab[1][j] = sinf(ang);
    }                                               // (published by the barriers of the reductions below)
  float ssq = 0.f, ssk = 0.f;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) ssq += row[i] * row[i];
  if (has_kv)
    for (int i = threadIdx.x; i < nk; i += blockDim.x) ssk += row[nq + i] * row[nq + i];
  const float rq = 1.f / sqrtf(block_sum(ssq, red) / static_cast<float>(nq) + eps);
  const float rk = has_kv ? 1.f / sqrtf(block_sum(ssk, red) / static_cast<float>(nk) + eps) : 0.f;
  auto rotated = [&](const float* src, const float* w, float r, int idx) {
    const int i = idx % D;
    const float a = src[idx] * r * w[idx];
    if (i >= rot_dims) return a;
    const int j = i < half ? i : i - half;
    float c, s;
    if (tab) {
      c = cs_tab[0][j];
      s = cs_tab[1][j];
    } else {
      const float ang = pos * inv_freq[j];
      c = cosf(ang);
      s = sinf(ang);
    }
    if (i < half) return a * c - src[idx + half] * r * w[idx + half] * s;
    return a * c + src[idx - half] * r * w[idx - half] * s;
  };
  for (int i = threadIdx.x; i < nq; i += blockDim.x) q_out[static_cast<size_t>(t) * nq + i] = rotated(row, qn, rq, i);
  if (!has_kv) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const size_t blk = slot / BS, off = slot % BS;
  typename Act<CF32>::type* kd = static_cast<typename Act<CF32>::type*>(kc);
  typename Act<CF32>::type* vd = static_cast<typename Act<CF32>::type*>(vc);
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int g = i / D;
    Act<CF32>::store(kd, ((blk * G + g) * BS + off) * D + (i % D), rotated(row + nq, kn, rk, i));
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const float* v = row + nq + nk;
  for (int g = wave; g < G; g += nw) {
    float ss = 0.f;
    for (int c = lane; c < Dv; c += 64) ss += v[g * Dv + c] * v[g * Dv + c];
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / static_cast<float>(Dv) + eps);
    for (int c = lane; c < Dv; c += 64) Act<CF32>::store(vd, ((blk * G + g) * BS + off) * Dv + c, v[g * Dv + c] * r);
  }
}

// ---------------------------------------------------------------- attention whose values are its keys
// One block per token. qk [T, ld] fp32: q [H*D] | k [G*D], no norms and no biases. The first rot_dims
// coordinates of each head rotate in NEIGHBOURING pairs: (x[2i], x[2i+1]) turns by position * inv_freq[i].
// The rotated key goes to the key plane [blocks, G, BS, D]; the key as projected, BEFORE the rotation, is
// the value and goes to the value plane of the same shape (no value plane is given when nothing rotates:
// one plane serves as both). The angle is formed and reduced to [-pi, pi] in fp64 (frequencies fp64).
template <bool CF32>
__global__ __launch_bounds__(256) void rope_pairs_write_kernel(
    const float* __restrict__ qk, int ld, const double* __restrict__ inv_freq, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ slot_mapping, void* __restrict__ kc, void* __restrict__ vc, float* __restrict__ q_out,
    int H, int G, int D, int BS, int rot_dims) {
  extern __shared__ float cs_dyn[];                // cos [half], sin [half] of the token's angles
  const int t = blockIdx.x;
  const float* row = qk + static_cast<size_t>(t) * ld;
  const double pos = static_cast<double>(positions[t]);
  const int half = rot_dims >> 1;
  const int nq = H * D, nk = G * D;
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    constexpr double kTwoPi = 6.283185307179586476925286766559;
    double a = pos * inv_freq[j];
    a -= kTwoPi * rint(a / kTwoPi);
    float s, c;
    sincosf(static_cast<float>(a), &s, &c);
    cs_dyn[j] = c;
    cs_dyn[half + j] = s;
  }
  __syncthreads();
  auto rotated = [&](const float* src, int idx) {
    const int i = idx % D;
    const float a = src[idx];
    if (i >= rot_dims) return a;
    const float c = cs_dyn[i >> 1], s = cs_dyn[half + (i >> 1)];
    const float other = src[idx - i + (i ^ 1)];
    return (i & 1) ? a * c + other * s : a * c - other * s;
  };
  for (int i = threadIdx.x; i < nq; i += blockDim.x) q_out[static_cast<size_t>(t) * nq + i] = rotated(row, i);
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const size_t blk = slot / BS, off = slot % BS;
  typename Act<CF32>::type* kd = static_cast<typename Act<CF32>::type*>(kc);
  typename Act<CF32>::type* vd = static_cast<typename Act<CF32>::type*>(vc);
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const size_t at = ((blk * G + i / D) * BS + off) * D + (i % D);
    Act<CF32>::store(kd, at, rotated(row + nq, i));
    if (vd != nullptr) Act<CF32>::store(vd, at, row[nq + i]);
  }
}

// ---------------------------------------------------------------- attention over the paged cache
// One wave per (row, query head), four heads of a row per block (same trip count for all four). Keys visible to the row at
// position p: lo <= j <= p with lo = max(floor(p / chunk) * chunk, p - window + 1) (either limit
// off when 0). Per tile of 64 keys: lane j scores key lo + 64 * tile + j in fp32 (q from LDS),
// online softmax across the wave, then the lanes split the value columns and walk the tile's
// keys (weights and cache rows from LDS). Serves prompt portions and single decoded tokens.
// Options: key / value rows may be column blocks of wider cache rows (row strides k_ld / v_ld); ``softcap`` > 0
// bounds the scaled score s to softcap * tanh(s / softcap); ``sink``: a silent extra key of score 0 without a value
// joins the softmax (the running maximum starts at 0 and the running sum at 1); ``vh0`` >= 0: the head's weights are
// applied to the ``nvh`` value heads vh0 .. vh0 + nvh - 1 side by side instead of its own group's (designs that
// mix the heads' weights afterwards need every head's weights on every value head). Output row (t, h) has ``o_ld``
// columns, written from column ``o_col0`` on.
constexpr int kMaxVCols = 8;   // value width up to 512

template <bool CF32, bool AF32>
__global__ __launch_bounds__(256) void attn_masked_kernel(
    const float* __restrict__ q, const void* __restrict__ kc, const void* __restrict__ vc,
    const int32_t* __restrict__ block_tables, int MB, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ positions, void* __restrict__ out, int H, int G, int D, int Dv, int BS, float scale,
    int chunk, int window, int k_ld, int v_ld, float softcap, int sink, int vh0, int nvh, int o_ld, int o_col0) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x;
  const bool live = blockIdx.y * 4 + wave < H;     // idle waves still take part in the barriers
  const int h = live ? blockIdx.y * 4 + wave : H - 1;
  float* qs = lds + wave * (D + 128);
  float* ps = qs + D;
  int* rows = reinterpret_cast<int*>(ps + 64);
  const int seq = row_seq[t];
  const int p = positions[t];
  if (seq < 0 || p < 0) return;             // the same for every wave of the block
  const int g = h / (H / G);
  for (int d = lane; d < D; d += 64) qs[d] = q[(static_cast<size_t>(t) * H + h) * D + d] * scale;
  int lo = 0;
  if (chunk > 0) lo = (p / chunk) * chunk;
  if (window > 0) lo = max(lo, p - window + 1);
  const int32_t* table = block_tables + static_cast<size_t>(seq) * MB;
  const typename Act<CF32>::type* kbase = static_cast<const typename Act<CF32>::type*>(kc);
  const typename Act<CF32>::type* vbase = static_cast<const typename Act<CF32>::type*>(vc);
  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[kMaxVCols];
  int vcol[kMaxVCols], voff[kMaxVCols];            // a lane's value columns: column inside the head, row offset of the head's plane
  const int ncols = nvh * Dv;
  if (vh0 >= 0) {                                   // blocks along z take nvh value heads each (scores are formed again: short rows)
    vh0 += blockIdx.z * nvh;
    o_col0 += blockIdx.z * ncols;
  }
#pragma unroll
  for (int i = 0; i < kMaxVCols; ++i) {
    acc[i] = 0.f;
    const int c = lane + 64 * i;
    const int vh = c / Dv;
    vcol[i] = c - vh * Dv;
    voff[i] = vh0 < 0 ? 0 : (vh0 + vh - g) * BS;
  }
  __syncthreads();
  for (int j0 = lo; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= p;
    float s = -INFINITY;
    int crow = 0;
    if (valid) {
      crow = (table[j / BS] * G + g) * BS + (j % BS);
      const typename Act<CF32>::type* kr = kbase + static_cast<size_t>(crow) * k_ld;
      float dot = 0.f;
      if (!CF32 && D % 8 == 0 && k_ld % 8 == 0) {
        // a bf16 key row in 16-byte pieces (rows start on 16-byte borders when D is a multiple of 8)
        const u32x4* kv = reinterpret_cast<const u32x4*>(kr);
        for (int c = 0; c < D / 8; ++c) {
          const u32x4 w = kv[c];
          const float* qc = qs + 8 * c;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            dot += qc[2 * e] * __uint_as_float(w[e] << 16) + qc[2 * e + 1] * __uint_as_float(w[e] & 0xffff0000u);
        }
      } else {
        for (int d = 0; d < D; ++d) dot += qs[d] * Act<CF32>::load(kr, d);
      }
      s = softcap > 0.f ? softcap * tanhf(dot / softcap) : dot;
    }
    const float mt = fmaxf(m, wave_max(s));
    const float pj = valid ? expf(s - mt) : 0.f;
    const float corr = expf(m - mt);         // exp(-inf) = 0 on the first tile
    l = l * corr + wave_sum(pj);
    m = mt;
    ps[lane] = pj;
    rows[lane] = crow;
    __syncthreads();
    const int n = min(64, p - j0 + 1);
#pragma unroll
    for (int i = 0; i < kMaxVCols; ++i) {
      const int c = lane + 64 * i;
      if (c < ncols) {
        float a = acc[i] * corr;
#pragma unroll 8                                    // eight value loads in flight at a time
        for (int jj = 0; jj < n; ++jj)
          a += ps[jj] * Act<CF32>::load(vbase, static_cast<size_t>(rows[jj] + voff[i]) * v_ld + vcol[i]);
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  typename Act<AF32>::type* o = static_cast<typename Act<AF32>::type*>(out);
#pragma unroll
  for (int i = 0; i < kMaxVCols; ++i) {
    const int c = lane + 64 * i;
    if (live && c < ncols) Act<AF32>::store(o, (static_cast<size_t>(t) * H + h) * o_ld + o_col0 + c, acc[i] / l);
  }
}

// ---------------------------------------------------------------- attention of prompt portions on the matrix cores
// fp32 products on the matrix cores (v_mfma_f32_16x16x4_f32: both operands fp32, so scores and
// weights stay 32-bit as in the row kernel above). A block is four waves = four consecutive tiles
// of 16 query rows of ONE sequence and ONE query head; key / value tiles of 16 positions are staged
// in LDS as fp32 once per block (16-byte loads, the next tile's loads in flight during the current
// tile's products) and serve all 64 rows. Per key tile and wave:
//   S = Q K^T   D/4 MFMAs (A: q[row l&15][d + (l>>4)], B: k[key l&15][d + (l>>4)]; S[row 4(l>>4)+r][key l&15])
//   masking per element (rows of a tile may lie in different chunks), online softmax per row
//   (the 16 lanes of a row's keys reduce by shuffles), P through LDS into the A layout,
//   O += P V    4 MFMAs per 16 value columns (B: v[key 4j + (l>>4)][col l&15]).
// Row strides in LDS are padded so that the 16 rows of an operand fall into different banks.
// The options of the row kernel (row strides, score cap, sink, value heads side by side) apply here too; the value
// tile then holds nvh * Dv columns.
// A wave holds up to 16 accumulator tiles (256 value columns; with 32 tiles, 512 columns in one launch, the kernel ran
// slower than two launches of 256 that each form the scores again). A block may use more than 64 KB of LDS (wide queries).
constexpr int kTileMaxVT = 16;
constexpr int kTileMaxLds = 160 * 1024;

LC_DEVICE int lds_stride(int n, int want) { return n + ((want - n % 32 + 32) % 32); }

// Eight consecutive cache elements as they come from memory (converted when they go to LDS, so
// that the loads of the NEXT tile stay in flight while the current one is computed).
template <bool CF32>
struct Raw8 {
  u32x4 v[CF32 ? 2 : 1];
};

template <bool CF32>
LC_DEVICE Raw8<CF32> load_raw8(const void* base, size_t elem, bool on) {
  Raw8<CF32> r;
#pragma unroll
  for (int i = 0; i < (CF32 ? 2 : 1); ++i) r.v[i] = u32x4{0u, 0u, 0u, 0u};
  if (on) {
    const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const char*>(base) + elem * (CF32 ? 4 : 2));
    r.v[0] = p[0];
    if (CF32) r.v[CF32 ? 1 : 0] = p[1];
  }
  return r;
}

template <bool CF32>
LC_DEVICE void store_raw8(const Raw8<CF32>& r, float* dst) {
  float4* d4 = reinterpret_cast<float4*>(dst);
  if (CF32) {
    d4[0] = make_float4(__uint_as_float(r.v[0][0]), __uint_as_float(r.v[0][1]), __uint_as_float(r.v[0][2]),
                        __uint_as_float(r.v[0][3]));
    d4[1] = make_float4(__uint_as_float(r.v[CF32 ? 1 : 0][0]), __uint_as_float(r.v[CF32 ? 1 : 0][1]),
                        __uint_as_float(r.v[CF32 ? 1 : 0][2]), __uint_as_float(r.v[CF32 ? 1 : 0][3]));
  } else {
    const u32x4 w = r.v[0];
    d4[0] = make_float4(__uint_as_float(w[0] << 16), __uint_as_float(w[0] & 0xffff0000u), __uint_as_float(w[1] << 16),
                        __uint_as_float(w[1] & 0xffff0000u));
    d4[1] = make_float4(__uint_as_float(w[2] << 16), __uint_as_float(w[2] & 0xffff0000u), __uint_as_float(w[3] << 16),
                        __uint_as_float(w[3] & 0xffff0000u));
  }
}

template <bool CF32, bool AF32>
__global__ __launch_bounds__(256) void attn_tile_kernel(
    const float* __restrict__ q, const void* __restrict__ kc, const void* __restrict__ vc,
    const int32_t* __restrict__ block_tables, int MB, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ positions, void* __restrict__ out, int H, int G, int D, int Dv, int BS, float scale,
    int chunk, int window, int k_ld, int v_ld, float softcap, int sink, int vh0, int nvh, int o_ld, int o_col0) {
  extern __shared__ float lds[];
  const int b = blockIdx.z, h = blockIdx.y;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  const int row0 = q0 + blockIdx.x * 64;
  if (row0 >= q1) return;                                   // the same for the whole block
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lr = lane & 15, lk = lane >> 4;
  const int g = h / (H / G);
  const int ncols = nvh * Dv;                               // value columns of the block: nvh heads side by side
  const int DS = lds_stride(D, 4), VS = lds_stride(ncols, 16);
  float* Qs = lds;                                          // [4][16][DS]
  float* Ks = Qs + 64 * DS;                                 // [16][DS]
  float* Vs = Ks + 16 * DS;                                 // [16][VS]
  float* Ps = Vs + 16 * VS + wave * 16 * 17;                // [4][16][17]
  const int nt = ncols / 16;
  const int32_t* table = block_tables + static_cast<size_t>(b) * MB;
  // queries of the block's rows, scaled (rows past the portion: zero)
  for (int i = threadIdx.x; i < 64 * D; i += 256) {
    const int r = i / D, d = i - r * D;
    Qs[r * DS + d] = row0 + r < q1 ? q[(static_cast<size_t>(row0 + r) * H + h) * D + d] * scale : 0.f;
  }
  const int p0 = positions[row0];                           // rows of a portion are consecutive positions
  const int nrows = min(64, q1 - row0);
  auto first_key = [&](int p) {
    int lo = 0;
    if (chunk > 0) lo = (p / chunk) * chunk;
    if (window > 0) lo = max(lo, p - window + 1);
    return lo;
  };
  const int hi = p0 + nrows - 1;
  const int pw0 = p0 + 16 * wave;                           // position of this wave's first row
  const int wave_rows = max(0, min(16, nrows - 16 * wave));
  const int wave_lo = first_key(pw0), wave_hi = pw0 + wave_rows - 1;
  // staging: a tile is 16 keys x D (x Dv) elements = 2 D (2 Dv) units of 8; a thread owns up to two of each
  constexpr int NVU = kTileMaxVT / 8;                       // value units of 8 columns per thread (16 keys x ncols / 8 in all)
  const int ku = D / 8, vu = ncols / 8;
  int kkey[2], kcol[2], vkey[NVU], vcol[NVU], vhead[NVU], vin[NVU];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int u = threadIdx.x + 256 * i;
    kkey[i] = u < 16 * ku ? u / ku : -1;
    kcol[i] = (u % ku) * 8;
  }
#pragma unroll
  for (int i = 0; i < NVU; ++i) {
    const int u = threadIdx.x + 256 * i;
    vkey[i] = u < 16 * vu ? u / vu : -1;
    vcol[i] = (u % vu) * 8;                                 // column in the tile; inside its head: vin
    vhead[i] = vh0 < 0 ? g : vh0 + vcol[i] / Dv;
    vin[i] = vcol[i] % Dv;
  }
  Raw8<CF32> kr[2], vr[NVU];
  auto fetch = [&](int j0) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int jk = j0 + kkey[i];
      const bool kon = kkey[i] >= 0 && jk <= hi;
      const size_t krow = kon ? (static_cast<size_t>(table[jk / BS]) * G + g) * BS + jk % BS : 0;
      kr[i] = load_raw8<CF32>(kc, krow * k_ld + kcol[i], kon);
    }
#pragma unroll
    for (int i = 0; i < NVU; ++i) {
      const int jv = j0 + vkey[i];
      const bool von = vkey[i] >= 0 && jv <= hi;
      const size_t vrow = von ? (static_cast<size_t>(table[jv / BS]) * G + vhead[i]) * BS + jv % BS : 0;
      vr[i] = load_raw8<CF32>(vc, vrow * v_ld + vin[i], von);
    }
  };
  float m[4], l[4];
  f32x4 o[kTileMaxVT];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m[r] = sink ? 0.f : -INFINITY;
    l[r] = sink ? 1.f : 0.f;
  }
#pragma unroll
  for (int t = 0; t < kTileMaxVT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float* Qw = Qs + wave * 16 * DS;
  int j0 = (first_key(p0) / 16) * 16;
  fetch(j0);
  for (; j0 <= hi; j0 += 16) {
    __syncthreads();                                        // the previous tile has been consumed
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (kkey[i] >= 0) store_raw8<CF32>(kr[i], Ks + kkey[i] * DS + kcol[i]);
#pragma unroll
    for (int i = 0; i < NVU; ++i)
      if (vkey[i] >= 0) store_raw8<CF32>(vr[i], Vs + vkey[i] * VS + vcol[i]);
    __syncthreads();
    if (j0 + 16 <= hi) fetch(j0 + 16);                      // in flight while this tile is computed
    const bool mine = wave_rows > 0 && j0 <= wave_hi && j0 + 15 >= wave_lo;     // wave-uniform
    if (!mine) continue;
    f32x4 sacc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};      // two chains keep the matrix pipe busy
    for (int d = 0; d < D; d += 8) {
      sacc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(Qw[lr * DS + d + lk], Ks[lr * DS + d + lk], sacc[0], 0, 0, 0);
      sacc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(Qw[lr * DS + d + 4 + lk], Ks[lr * DS + d + 4 + lk], sacc[1], 0, 0, 0);
    }
    const int j = j0 + lr;
    float corr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * lk + r;
      const int prow = pw0 + row;
      const bool valid = row < wave_rows && j <= prow && j >= first_key(prow);
      const float sraw = sacc[0][r] + sacc[1][r];
      const float sv = valid ? (softcap > 0.f ? softcap * tanhf(sraw / softcap) : sraw) : -INFINITY;
      float mt = sv;
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) mt = fmaxf(mt, __shfl_xor(mt, off, 64));
      const float mn = fmaxf(m[r], mt);
      const float base = mn == -INFINITY ? 0.f : mn;        // nothing visible yet: weights 0, no NaN
      const float pv = valid ? expf(sv - base) : 0.f;
      corr[r] = expf(m[r] - base);
      float ps = pv;
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) ps += __shfl_xor(ps, off, 64);
      l[r] = l[r] * corr[r] + ps;
      m[r] = mn;
      Ps[row * 17 + lr] = pv;
    }
    // P goes from the score layout to the operand layout through this wave's own LDS patch: the
    // wave's LDS accesses execute in order, the fences keep the compiler from moving them
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float pa[4];
#pragma unroll
    for (int j4 = 0; j4 < 4; ++j4) pa[j4] = Ps[lr * 17 + 4 * j4 + lk];
#pragma unroll
    for (int t = 0; t < kTileMaxVT; ++t) {
      if (t < nt) {
        f32x4 acc = o[t];
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] *= corr[r];
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[j4], Vs[(4 * j4 + lk) * VS + t * 16 + lr], acc, 0, 0, 0);
        o[t] = acc;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");     // P is read before the next tile overwrites it
    __builtin_amdgcn_wave_barrier();
  }
  typename Act<AF32>::type* dst = static_cast<typename Act<AF32>::type*>(out);
#pragma unroll
  for (int t = 0; t < kTileMaxVT; ++t) {
    if (t < nt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = 4 * lk + r;
        if (row < wave_rows)
          Act<AF32>::store(dst, (static_cast<size_t>(row0 + 16 * wave + row) * H + h) * o_ld + o_col0 + t * 16 + lr,
                           o[t][r] / l[r]);
      }
    }
  }
}

// ---------------------------------------------------------------- shape-agnostic GEMM
// C[M, N] = A[M, K] W[N, K]^T (+ bias) with fp32 accumulation on the vector ALUs: 64 x 64 tiles,
// 16-deep slabs in LDS, 4 x 4 outputs per thread. Any M, N, K; A, W and C each fp32 or bf16; A may be
// a column slice (row stride lda).
// epi 1: square of relu.
template <bool AF32, bool WF32, bool CF32>
__global__ __launch_bounds__(256) void gemm_any_kernel(const void* __restrict__ A, int lda, const void* __restrict__ W,
                                                       const void* __restrict__ bias, void* __restrict__ C, int M, int N,
                                                       int K, int epi) {
  __shared__ float As[16][64 + 4];
  __shared__ float Ws[16][64 + 4];
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const typename Act<AF32>::type* a = static_cast<const typename Act<AF32>::type*>(A);
  const typename Act<WF32>::type* w = static_cast<const typename Act<WF32>::type*>(W);
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int i = threadIdx.x; i < 64 * 16; i += 256) {
      const int r = i >> 4, k = i & 15;
      As[k][r] = (m0 + r < M && k0 + k < K) ? Act<AF32>::load(a, static_cast<size_t>(m0 + r) * lda + k0 + k) : 0.f;
      Ws[k][r] = (n0 + r < N && k0 + k < K) ? Act<WF32>::load(w, static_cast<size_t>(n0 + r) * K + k0 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = As[k][ty * 4 + i];
        wv[i] = Ws[k][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * wv[j];
    }
    __syncthreads();
  }
  typename Act<CF32>::type* c = static_cast<typename Act<CF32>::type*>(C);
  const typename Act<WF32>::type* bs = static_cast<const typename Act<WF32>::type*>(bias);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = m0 + ty * 4 + i;
    if (r >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= N) continue;
      float v = acc[i][j] + (bs != nullptr ? Act<WF32>::load(bs, col) : 0.f);
      if (epi == 1) {
        v = fmaxf(v, 0.f);
        v *= v;
      }
      Act<CF32>::store(c, static_cast<size_t>(r) * N + col, v);
    }
  }
}

// ---------------------------------------------------------------- per-head products
// C[m, h, :] = W[h] A[m, h, :] for H heads side by side: A [M, H*K] (row stride lda), W [H, N, K],
// C [M, H*N]. The tiling of gemm_any_kernel with the head as the third grid dimension. With
// ``gate`` [M, H] (row stride ld_gate) the head's outputs are scaled by sigmoid(gate[m, h]); ``gate_full``: the gate
// is [M, H*N], one logit per output. Head h's inputs start at column h * a_hs of A, its outputs at column h * c_hs
// of C (row stride c_ld): heads may be column blocks of wider per-head rows on either side.
// RPT rows per thread: a block covers 16 * RPT rows x 64 columns. Few rows (decode steps) take RPT = 1, which
// spreads the same products over four times as many waves.
template <bool AF32, bool WF32, bool CF32, int RPT>
__global__ __launch_bounds__(256) void head_linear_kernel(const void* __restrict__ A, int lda, const void* __restrict__ W,
                                                          void* __restrict__ C, const float* __restrict__ gate,
                                                          int ld_gate, int M, int H, int N, int K, int a_hs, int c_ld,
                                                          int c_hs, int gate_full) {
  constexpr int KS = 32;                            // slab depth: per-head depths are short, so few, deep slabs
  constexpr int TM = 16 * RPT;
  constexpr int NA = TM * KS / 256, NW = 64 * KS / 256;
  __shared__ float As[KS][TM + 4];
  __shared__ float Ws[KS][64 + 4];
  const int h = blockIdx.z;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const typename Act<AF32>::type* a = static_cast<const typename Act<AF32>::type*>(A) + static_cast<size_t>(h) * a_hs;
  const typename Act<WF32>::type* w = static_cast<const typename Act<WF32>::type*>(W) + static_cast<size_t>(h) * N * K;
  float acc[RPT][4] = {};
  // the next slab's elements are loaded into registers before the current one is multiplied, so the
  // loads' latency hides behind the products
  float ra[NA], rw[NW];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int j = 0; j < NA; ++j) {
      const int i = threadIdx.x + 256 * j;
      const int r = i / KS, k = i % KS;
      ra[j] = (m0 + r < M && k0 + k < K) ? Act<AF32>::load(a, static_cast<size_t>(m0 + r) * lda + k0 + k) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      const int i = threadIdx.x + 256 * j;
      const int r = i / KS, k = i % KS;
      rw[j] = (n0 + r < N && k0 + k < K) ? Act<WF32>::load(w, static_cast<size_t>(n0 + r) * K + k0 + k) : 0.f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += KS) {
#pragma unroll
    for (int j = 0; j < NA; ++j) {
      const int i = threadIdx.x + 256 * j;
      As[i % KS][i / KS] = ra[j];
    }
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      const int i = threadIdx.x + 256 * j;
      Ws[i % KS][i / KS] = rw[j];
    }
    __syncthreads();
    if (k0 + KS < K) fetch(k0 + KS);
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      float av[RPT], wv[4];
#pragma unroll
      for (int i = 0; i < RPT; ++i) av[i] = As[k][ty * RPT + i];
#pragma unroll
      for (int i = 0; i < 4; ++i) wv[i] = Ws[k][tx * 4 + i];
#pragma unroll
      for (int i = 0; i < RPT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * wv[j];
    }
    __syncthreads();
  }
  typename Act<CF32>::type* c = static_cast<typename Act<CF32>::type*>(C);
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = m0 + ty * RPT + i;
    if (r >= M) continue;
    const float g = gate != nullptr && !gate_full ? sigmoidf_(gate[static_cast<size_t>(r) * ld_gate + h]) : 1.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= N) continue;
      const float ge = gate_full ? sigmoidf_(gate[static_cast<size_t>(r) * ld_gate + h * N + col]) : g;
      Act<CF32>::store(c, static_cast<size_t>(r) * c_ld + static_cast<size_t>(h) * c_hs + col, acc[i][j] * ge);
    }
  }
}

}  // namespace

// ================================================================= launchers
LC_EXPORT int lc_embed_rows(const void* ids, const void* E, int e_f32, void* x, void* xa, int act_f32, int T, int d,
                            int vocab, const void* feed_tok, const void* feed_rows, float scale, const void* positions,
                            const void* inv_freq, hipStream_t st) {
  if (T <= 0) return 0;
  if (d <= 0 || vocab <= 0 || (inv_freq != nullptr && (positions == nullptr || (d & 1)))) return -1;
  const dim3 grid((T + 3) / 4), block(256);
#define LC_EMB(E32, A32)                                                                                      \
  embed_rows_kernel<E32, A32><<<grid, block, 0, st>>>(static_cast<const int32_t*>(ids), E, static_cast<float*>(x), \
                                                      xa, T, d, vocab, static_cast<const int32_t*>(feed_tok), \
                                                      static_cast<const int32_t*>(feed_rows), scale,          \
                                                      static_cast<const int32_t*>(positions),                 \
                                                      static_cast<const double*>(inv_freq))
  if (e_f32 && act_f32) LC_EMB(true, true);
  else if (e_f32) LC_EMB(true, false);
  else if (act_f32) LC_EMB(false, true);
  else LC_EMB(false, false);
#undef LC_EMB
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_scalar_norm_add(void* x, const void* y, const void* gain, float eps, void* xa, int act_f32, int T,
                                 int d, hipStream_t st) {
  if (T <= 0) return 0;
  if (d <= 0) return -1;
  const bool few = T <= 512;
  const dim3 grid(few ? T : (T + 3) / 4), block(256);
#define LC_SN(A32, WAVES)                                                                                       \
  scalar_norm_add_kernel<A32, WAVES><<<grid, block, 0, st>>>(static_cast<float*>(x), static_cast<const float*>(y), \
                                                             static_cast<const float*>(gain), eps, xa, T, d)
  if (act_f32 && few) LC_SN(true, 4);
  else if (act_f32) LC_SN(true, 1);
  else if (few) LC_SN(false, 4);
  else LC_SN(false, 1);
#undef LC_SN
  LC_RETURN_LAST_ERROR();
}

// y [T, >= cols] with row stride ld -> out [T, cols].
LC_EXPORT int lc_relu2(const void* y, void* out, int act_f32, int T, int cols, int ld, hipStream_t st) {
  if (T <= 0 || cols <= 0) return 0;
  if (ld < cols) return -1;
  const long long n = static_cast<long long>(T) * cols;
  const dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
  if (act_f32) relu2_kernel<true><<<grid, block, 0, st>>>(static_cast<const float*>(y), out, n, cols, ld);
  else relu2_kernel<false><<<grid, block, 0, st>>>(static_cast<const float*>(y), out, n, cols, ld);
  LC_RETURN_LAST_ERROR();
}

// ``max_len``: the longest portion of the step (host-known). Portions longer than two segments take
// the segmented passes; ``scratch`` then holds B * nseg * 2 * w floats (see lc_scan_scratch_floats).
// 32 rows: the pass that writes the outputs is a dependent chain per state column, so twice the waves of
// half the length finish sooner (2048-row prompt, 16 heads: 301 us with 64-row segments, 212 us with 32).
constexpr int kScanSegment = 32;

LC_EXPORT long long lc_scan_scratch_floats(int B, int max_len, long long state_floats, long long decay_floats) {
  if (max_len <= 2 * kScanSegment) return 0;
  const long long nseg = (max_len + kScanSegment - 1) / kScanSegment;
  return static_cast<long long>(B) * nseg * (state_floats + decay_floats);
}

LC_EXPORT int lc_mingru_scan(const void* zxg, void* state, const void* cu_q, const void* positions, const void* slots,
                             void* out, int act_f32, int B, int w, int max_len, void* scratch, hipStream_t st) {
  if (B <= 0) return 0;
  if (w <= 0) return -1;
  const bool segmented = max_len > 2 * kScanSegment;
  if (segmented && scratch == nullptr) return -1;
  const int nseg = segmented ? (max_len + kScanSegment - 1) / kScanSegment : 1;
  const dim3 grid((w + 127) / 128, B, nseg), block(128);
#define LC_GRU(A32, MODE)                                                                                           \
  mingru_scan_kernel<A32><<<grid, block, 0, st>>>(static_cast<const float*>(zxg), static_cast<float*>(state),       \
                                                  static_cast<const int32_t*>(cu_q),                                \
                                                  static_cast<const int32_t*>(positions),                           \
                                                  static_cast<const int32_t*>(slots), out, w, MODE, kScanSegment,   \
                                                  static_cast<float*>(scratch))
  if (segmented) {
    LC_GRU(true, 1);
    if (act_f32) LC_GRU(true, 2);
    else LC_GRU(false, 2);
  } else if (act_f32) {
    LC_GRU(true, 0);
  } else {
    LC_GRU(false, 0);
  }
#undef LC_GRU
  LC_RETURN_LAST_ERROR();
}

// The scan over prepared operands (``prep``: T * H * D float4, see the prepare kernels): per head
// S <- a S + k v^T over Dv value columns, the last ``ones`` of which read v = 1.
static int launch_linear_scan(const void* proj, int ld, const void* prep, void* state, long long state_stride,
                              const void* cu_q, const void* positions, const void* slots, void* out, int B, int H, int D,
                              int Dv, int ones, int max_len, void* scratch, hipStream_t st) {
  const bool segmented = max_len > 2 * kScanSegment;
  if (segmented && scratch == nullptr) return -1;
  const int nseg = segmented ? (max_len + kScanSegment - 1) / kScanSegment : 1;
  const dim3 grid((Dv + 63) / 64, H, B * nseg), block(64);
  float* cs = static_cast<float*>(scratch);
  float* ca = segmented ? cs + static_cast<size_t>(B) * nseg * H * D * Dv : nullptr;
#define LC_GLA(DMAX, MODE)                                                                                             \
  gla_scan_kernel<DMAX><<<grid, block, 0, st>>>(static_cast<const float*>(proj), ld, static_cast<const float4*>(prep), \
                                                static_cast<float*>(state), static_cast<const int32_t*>(cu_q),      \
                                                static_cast<const int32_t*>(positions),                             \
                                                static_cast<const int32_t*>(slots), static_cast<float*>(out), H, D, \
                                                Dv, MODE, nseg, kScanSegment, cs, state_stride, ones)
#define LC_GLA_D(MODE)          \
  if (D <= 32) LC_GLA(32, MODE);  \
  else if (D <= 64) LC_GLA(64, MODE); \
  else if (D <= 128) LC_GLA(128, MODE); \
  else LC_GLA(256, MODE)
  if (segmented) {
    static_assert(kScanSegment <= kSegRows, "a segment's rows are staged in LDS at once");
    const dim3 sgrid(((D + kSegD - 1) / kSegD) * ((Dv + kSegV - 1) / kSegV), H, B * nseg);
    scan_segment_state_kernel<<<sgrid, dim3(256), 0, st>>>(
        static_cast<const float*>(proj), ld, static_cast<const float4*>(prep), static_cast<const int32_t*>(cu_q),
        static_cast<const int32_t*>(slots), H, D, Dv, nseg, kScanSegment, cs, ca, ones);
    const size_t n = static_cast<size_t>(H) * D * Dv;
    gla_carry_kernel<<<dim3(static_cast<unsigned>((n + 255) / 256), B), dim3(256), 0, st>>>(
        cs, ca, static_cast<const float*>(state), static_cast<const int32_t*>(cu_q),
        static_cast<const int32_t*>(positions), static_cast<const int32_t*>(slots), H, D, Dv, nseg, kScanSegment,
        state_stride);
    LC_GLA_D(2);
  } else {
    LC_GLA_D(0);
  }
#undef LC_GLA_D
#undef LC_GLA
  LC_RETURN_LAST_ERROR();
}

// ``prep``: T * H * D float4 of scratch for the per-token operands (gla_prepare_kernel).
LC_EXPORT int lc_gla_scan(const void* proj, int ld, const void* decay, void* state, long long state_stride,
                          const void* cu_q, const void* positions, const void* slots, void* out, int T, int B, int H,
                          int D, int Dv, float tau, int max_len, void* scratch, void* prep, hipStream_t st) {
  if (B <= 0) return 0;
  if (H <= 0 || D <= 0 || Dv <= 0 || D > 256 || ld < 2 * H * D + H * Dv || !(tau > 0.f)) return -1;
  if (prep == nullptr || T <= 0 || state_stride < static_cast<long long>(H) * D * Dv) return -1;
  const long long n = static_cast<long long>(T) * H * D;
  gla_prepare_kernel<<<dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st>>>(
      static_cast<const float*>(proj), ld, static_cast<const float*>(decay), static_cast<float4*>(prep), n, H * D,
      1.f / tau, 1.f / sqrtf(static_cast<float>(D)));
  return launch_linear_scan(proj, ld, prep, state, state_stride, cu_q, positions, slots, out, B, H, D, Dv, 0, max_len,
                            scratch, st);
}

// mLSTM: gates and running maxima, prepared operands, then the scan over Dv + 1 value columns (the
// extra column, v = 1, is the normaliser). ``prep``: T * H * (4 D + 2) floats; ``out`` [T, H * (Dv + 1)];
// ``m_out`` [T, H]; a slot of ``state`` holds H * D * (Dv + 1) floats and then the H maxima.
LC_EXPORT int lc_mlstm_scan(const void* proj, int ld, void* state, long long state_stride, const void* cu_q,
                            const void* positions, const void* slots, void* out, void* m_out, int T, int B, int H, int D,
                            int Dv, float cap, int max_len, void* scratch, void* prep, hipStream_t st) {
  if (B <= 0 || T <= 0) return 0;
  if (H <= 0 || D <= 0 || Dv <= 0 || D > 256 || ld < 2 * H * D + 2 * H * Dv + 2 * H || cap < 0.f) return -1;
  const long long n_s = static_cast<long long>(H) * D * (Dv + 1);
  if (prep == nullptr || m_out == nullptr || state_stride < n_s + H) return -1;
  const long long n = static_cast<long long>(T) * H * D;
  float2* gates = reinterpret_cast<float2*>(static_cast<float4*>(prep) + n);
  mlstm_gates_kernel<<<dim3(H, B), dim3(64), 0, st>>>(
      static_cast<const float*>(proj), ld, 2 * H * D + 2 * H * Dv, static_cast<float*>(state), state_stride, n_s,
      static_cast<const int32_t*>(cu_q), static_cast<const int32_t*>(positions), static_cast<const int32_t*>(slots), gates,
      static_cast<float*>(m_out), H, cap);
  mlstm_prepare_kernel<<<dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st>>>(
      static_cast<const float*>(proj), ld, gates, static_cast<float4*>(prep), n, H, D, 1.f / sqrtf(static_cast<float>(D)));
  return launch_linear_scan(proj, ld, prep, state, state_stride, cu_q, positions, slots, out, B, H, D, Dv + 1, 1, max_len,
                            scratch, st);
}

LC_EXPORT int lc_add_rmsnorm(void* x, const void* y, const void* w, float eps, void* xa, int act_f32, int T, int d,
                             hipStream_t st) {
  if (T <= 0) return 0;
  if (d <= 0 || (w != nullptr && xa == nullptr)) return -1;
  const bool few = T <= 512;
  const dim3 grid(few ? T : (T + 3) / 4), block(256);
#define LC_AN(A32, WAVES)                                                                                          \
  add_rmsnorm_kernel<A32, WAVES><<<grid, block, 0, st>>>(static_cast<float*>(x), static_cast<const float*>(y),    \
                                                         static_cast<const float*>(w), eps, xa, T, d)
  if (act_f32 && few) LC_AN(true, 4);
  else if (act_f32) LC_AN(true, 1);
  else if (few) LC_AN(false, 4);
  else LC_AN(false, 1);
#undef LC_AN
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_glu(const void* y, void* out, int act_f32, int T, int n, int kind, hipStream_t st) {
  if (T <= 0 || n <= 0) return 0;
  const long long total = static_cast<long long>(T) * n;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256)), block(256);
  if (act_f32) glu_kernel<true><<<grid, block, 0, st>>>(static_cast<const float*>(y), out, total, n, kind);
  else glu_kernel<false><<<grid, block, 0, st>>>(static_cast<const float*>(y), out, total, n, kind);
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_add_dyt(void* x, const void* y, float mult, float alpha, const void* w, const void* b, void* out,
                         int act_f32, int ldo, int T, int d, hipStream_t st) {
  if (T <= 0) return 0;
  if (d <= 0 || (w != nullptr && (out == nullptr || b == nullptr)) || (out != nullptr && ldo < d)) return -1;
  if (y == nullptr && out == nullptr) return 0;
  const long long total = static_cast<long long>(T) * d;
  const bool v4 = d % 4 == 0 && ldo % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const long long threads = v4 ? total / 4 : total;
  const dim3 grid(static_cast<unsigned>((threads + 255) / 256)), block(256);
#define LC_AD(A32, V)                                                                                                  \
  add_dyt_kernel<A32, V><<<grid, block, 0, st>>>(static_cast<float*>(x), static_cast<const float*>(y), mult, alpha,   \
                                                 static_cast<const float*>(w), static_cast<const float*>(b), out, ldo, \
                                                 total, d)
  if (act_f32 && v4) LC_AD(true, 4);
  else if (act_f32) LC_AD(true, 1);
  else if (v4) LC_AD(false, 4);
  else LC_AD(false, 1);
#undef LC_AD
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_glu_clamped(const void* y, int ld, int col_gate, int col_up, int n, float limit, float slope, float shift,
                             const void* slot_of, const void* wts, void* out, int act_f32, int rows, hipStream_t st) {
  if (rows <= 0 || n <= 0) return 0;
  if (col_gate < 0 || col_up < 0 || ld < col_gate + n || ld < col_up + n || (wts != nullptr && slot_of == nullptr)) return -1;
  const long long total = static_cast<long long>(rows) * n;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256)), block(256);
  if (act_f32)
    glu_clamped_kernel<true><<<grid, block, 0, st>>>(static_cast<const float*>(y), ld, col_gate, col_up, n, limit, slope,
                                                     shift, static_cast<const int32_t*>(slot_of),
                                                     static_cast<const float*>(wts), out, total);
  else
    glu_clamped_kernel<false><<<grid, block, 0, st>>>(static_cast<const float*>(y), ld, col_gate, col_up, n, limit, slope,
                                                      shift, static_cast<const int32_t*>(slot_of),
                                                      static_cast<const float*>(wts), out, total);
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_rope_pairs_write(const void* qk, int ld, const void* inv_freq, const void* positions,
                                  const void* slot_mapping, void* kc, void* vc, int cache_f32, void* q_out, int T, int H,
                                  int G, int D, int BS, int rot_dims, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || D <= 0 || BS <= 0 || rot_dims < 0 || rot_dims > D || (rot_dims & 1)) return -1;
  if (ld < (H + G) * D || kc == nullptr || q_out == nullptr || (rot_dims > 0 && (vc == nullptr || inv_freq == nullptr)))
    return -1;
  const size_t lds = static_cast<size_t>(rot_dims > 0 ? rot_dims : 1) * sizeof(float);
  if (lds > 64 * 1024) return -1;
#define LC_RP(C32)                                                                                                \
  rope_pairs_write_kernel<C32><<<dim3(T), dim3(256), lds, st>>>(                                                  \
      static_cast<const float*>(qk), ld, static_cast<const double*>(inv_freq), static_cast<const int32_t*>(positions), \
      static_cast<const int32_t*>(slot_mapping), kc, vc, static_cast<float*>(q_out), H, G, D, BS, rot_dims)
  if (cache_f32) LC_RP(true);
  else LC_RP(false);
#undef LC_RP
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_latent_write(const void* proj, int ld, int col0, int R, const void* w, float eps, const void* slot_mapping,
                              void* cache, int cache_f32, int BS, int T, hipStream_t st) {
  if (T <= 0) return 0;
  if (R <= 0 || col0 < 0 || ld < col0 + R || BS <= 0) return -1;
  const dim3 grid((T + 3) / 4), block(256);
  if (cache_f32)
    latent_write_kernel<true><<<grid, block, 0, st>>>(static_cast<const float*>(proj), ld, col0, R,
                                                      static_cast<const float*>(w), eps,
                                                      static_cast<const int32_t*>(slot_mapping), cache, BS, T);
  else
    latent_write_kernel<false><<<grid, block, 0, st>>>(static_cast<const float*>(proj), ld, col0, R,
                                                       static_cast<const float*>(w), eps,
                                                       static_cast<const int32_t*>(slot_mapping), cache, BS, T);
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_head_linear(const void* A, int a_f32, int lda, const void* W, int w_f32, void* C, int c_f32,
                             const void* gate, int ld_gate, int M, int H, int N, int K, int a_hs, int c_ld, int c_hs,
                             int gate_full, hipStream_t st) {
  if (M <= 0 || N <= 0 || H <= 0) return 0;
  if (K <= 0 || a_hs < K || lda < (H - 1) * a_hs + K || H > 65535 || c_hs < N || c_ld < (H - 1) * c_hs + N) return -1;
  if (gate != nullptr && ld_gate < (gate_full ? H * N : H)) return -1;
  if (gate == nullptr && gate_full) return -1;
  const bool few = M <= 64;                          // decode steps: one row per thread, four times the blocks
  const dim3 grid((N + 63) / 64, few ? (M + 15) / 16 : (M + 63) / 64, H), block(256);
#define LC_HL(A32, W32, C32)                                                                                       \
  if (few)                                                                                                         \
    head_linear_kernel<A32, W32, C32, 1><<<grid, block, 0, st>>>(A, lda, W, C, static_cast<const float*>(gate), ld_gate, \
                                                                 M, H, N, K, a_hs, c_ld, c_hs, gate_full);         \
  else                                                                                                             \
    head_linear_kernel<A32, W32, C32, 4><<<grid, block, 0, st>>>(A, lda, W, C, static_cast<const float*>(gate), ld_gate, \
                                                                 M, H, N, K, a_hs, c_ld, c_hs, gate_full)
  const int sel = (a_f32 ? 4 : 0) | (w_f32 ? 2 : 0) | (c_f32 ? 1 : 0);
  switch (sel) {
    case 0: LC_HL(false, false, false); break;
    case 1: LC_HL(false, false, true); break;
    case 2: LC_HL(false, true, false); break;
    case 3: LC_HL(false, true, true); break;
    case 4: LC_HL(true, false, false); break;
    case 5: LC_HL(true, false, true); break;
    case 6: LC_HL(true, true, false); break;
    default: LC_HL(true, true, true); break;
  }
#undef LC_HL
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_headnorm_gate(const void* o, const void* w, const void* gate, int ld_gate, void* out, int act_f32,
                               int T, int H, int Dv, float eps, int ld_head, int w_stride, int gate_kind, const void* m,
                               hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || Dv <= 0 || ld_gate < H * Dv || ld_head < Dv || (m != nullptr && ld_head < Dv + 1)) return -1;
  const dim3 grid((T * H + 3) / 4), block(256);
  if (act_f32)
    headnorm_gate_kernel<true><<<grid, block, 0, st>>>(static_cast<const float*>(o), static_cast<const float*>(w),
                                                       static_cast<const float*>(gate), ld_gate, out, T, H, Dv, eps,
                                                       ld_head, w_stride, gate_kind, static_cast<const float*>(m));
  else
    headnorm_gate_kernel<false><<<grid, block, 0, st>>>(static_cast<const float*>(o), static_cast<const float*>(w),
                                                        static_cast<const float*>(gate), ld_gate, out, T, H, Dv, eps,
                                                        ld_head, w_stride, gate_kind, static_cast<const float*>(m));
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_qkv_prep(const void* qkv, int ld, const void* qn, const void* kn, const void* inv_freq,
                          const void* positions, const void* slot_mapping, void* kc, void* vc, int cache_f32,
                          void* q_out, int T, int H, int G, int D, int Dv, int BS, int rot_dims, float eps, int has_kv,
                          hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || D <= 0 || Dv <= 0 || BS <= 0 || rot_dims < 0 || rot_dims > D || (rot_dims & 1)) return -1;
  if (ld < H * D + (has_kv ? G * (D + Dv) : 0)) return -1;
  if (has_kv && (kc == nullptr || vc == nullptr || kn == nullptr)) return -1;
#define LC_PREP(C32)                                                                                              \
  qkv_prep_kernel<C32><<<dim3(T), dim3(256), 0, st>>>(                                                            \
      static_cast<const float*>(qkv), ld, static_cast<const float*>(qn), static_cast<const float*>(kn),           \
      static_cast<const float*>(inv_freq), static_cast<const int32_t*>(positions),                                \
      static_cast<const int32_t*>(slot_mapping), kc, vc, static_cast<float*>(q_out), H, G, D, Dv, BS, rot_dims, eps, \
      has_kv)
  if (cache_f32) LC_PREP(true);
  else LC_PREP(false);
#undef LC_PREP
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_attn_masked(const void* q, const void* kc, const void* vc, int cache_f32, const void* block_tables,
                             int MB, const void* row_seq, const void* positions, void* out, int act_f32, int T, int H,
                             int G, int D, int Dv, int BS, float scale, int chunk, int window, int k_ld, int v_ld,
                             float softcap, int sink, int vh0, int nvh, int o_ld, int o_col0, int vz, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || BS <= 0 || MB <= 0 || vz <= 0 || vz > 65535) return -1;
  // ``vz`` groups of nvh value heads each, one per block along z (vz = 1 unless value heads are named)
  if (nvh <= 0 || nvh * Dv > 64 * kMaxVCols || (vh0 < 0 && (nvh != 1 || vz != 1)) || (vh0 >= 0 && vh0 + vz * nvh > G)) return -1;
  if (k_ld < D || v_ld < Dv || o_col0 < 0 || o_ld < o_col0 + vz * nvh * Dv || softcap < 0.f) return -1;
  const size_t lds = 4 * static_cast<size_t>(D + 128) * sizeof(float);
  if (lds > 64 * 1024) return -1;
  const dim3 grid(T, (H + 3) / 4, vz), block(256);
#define LC_ATT(C32, A32)                                                                                        \
  attn_masked_kernel<C32, A32><<<grid, block, lds, st>>>(                                                       \
      static_cast<const float*>(q), kc, vc, static_cast<const int32_t*>(block_tables), MB,                      \
      static_cast<const int32_t*>(row_seq), static_cast<const int32_t*>(positions), out, H, G, D, Dv, BS, scale, \
      chunk, window, k_ld, v_ld, softcap, sink, vh0, nvh, o_ld, o_col0)
  if (cache_f32 && act_f32) LC_ATT(true, true);
  else if (cache_f32) LC_ATT(true, false);
  else if (act_f32) LC_ATT(false, true);
  else LC_ATT(false, false);
#undef LC_ATT
  LC_RETURN_LAST_ERROR();
}

// Prompt portions: sequences [0, n_seq) of cu_q, the longest of ``max_len`` rows. Returns -2 when
// the shape is not one the tile kernel takes (the caller then uses the row kernel for these rows too).
LC_EXPORT int lc_attn_tile(const void* q, const void* kc, const void* vc, int cache_f32, const void* block_tables,
                           int MB, const void* cu_q, const void* positions, void* out, int act_f32, int n_seq,
                           int max_len, int H, int G, int D, int Dv, int BS, float scale, int chunk, int window,
                           int k_ld, int v_ld, float softcap, int sink, int vh0, int nvh, int o_ld, int o_col0,
                           hipStream_t st) {
  if (n_seq <= 0 || max_len <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || BS <= 0 || MB <= 0) return -1;
  if (nvh <= 0 || (vh0 < 0 && nvh != 1) || (vh0 >= 0 && vh0 + nvh > G)) return -1;
  if (k_ld < D || v_ld < Dv || o_col0 < 0 || o_ld < o_col0 + nvh * Dv || softcap < 0.f) return -1;
  const int NC = nvh * Dv;
  // (16-byte loads of the staged tiles: rows and column blocks start on 16-byte borders)
  if (D % 8 || Dv % 8 || NC % 16 || NC > 16 * kTileMaxVT || D > 256 || k_ld % 8 || v_ld % 8) return -2;
  const int DS = D + ((4 - D % 32 + 32) % 32), VS = NC + ((16 - NC % 32 + 32) % 32);
  const size_t lds = (static_cast<size_t>(80) * DS + 16 * VS + 4 * 16 * 17) * sizeof(float);
  if (lds > static_cast<size_t>(kTileMaxLds)) return -2;
  const dim3 grid((max_len + 63) / 64, H, n_seq), block(256);
  static LcDeviceOnce attr_once;
  attr_once.run([&] {
#define LC_TILE_ATTR(C32, A32)                                                             \
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(attn_tile_kernel<C32, A32>),     \
                            hipFuncAttributeMaxDynamicSharedMemorySize, kTileMaxLds)
    LC_TILE_ATTR(true, true); LC_TILE_ATTR(true, false); LC_TILE_ATTR(false, true); LC_TILE_ATTR(false, false);
#undef LC_TILE_ATTR
  });
#define LC_TILE(C32, A32)                                                                                       \
  attn_tile_kernel<C32, A32><<<grid, block, lds, st>>>(                                                         \
      static_cast<const float*>(q), kc, vc, static_cast<const int32_t*>(block_tables), MB,                      \
      static_cast<const int32_t*>(cu_q), static_cast<const int32_t*>(positions), out, H, G, D, Dv, BS, scale,   \
      chunk, window, k_ld, v_ld, softcap, sink, vh0, nvh, o_ld, o_col0)
  if (cache_f32 && act_f32) LC_TILE(true, true);
  else if (cache_f32) LC_TILE(true, false);
  else if (act_f32) LC_TILE(false, true);
  else LC_TILE(false, false);
#undef LC_TILE
  LC_RETURN_LAST_ERROR();
}

// A may be a column slice of a wider matrix: ``lda`` is its row stride in elements.
LC_EXPORT int lc_gemm_any(const void* A, int a_f32, int lda, const void* W, int w_f32, const void* bias, void* C,
                          int c_f32, int M, int N, int K, int epi, hipStream_t st) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K) return -1;
  const dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
#define LC_GA(A32, W32, C32) gemm_any_kernel<A32, W32, C32><<<grid, block, 0, st>>>(A, lda, W, bias, C, M, N, K, epi)
  const int sel = (a_f32 ? 4 : 0) | (w_f32 ? 2 : 0) | (c_f32 ? 1 : 0);
  switch (sel) {
    case 0: LC_GA(false, false, false); break;
    case 1: LC_GA(false, false, true); break;
    case 2: LC_GA(false, true, false); break;
    case 3: LC_GA(false, true, true); break;
    case 4: LC_GA(true, false, false); break;
    case 5: LC_GA(true, false, true); break;
    case 6: LC_GA(true, true, false); break;
    default: LC_GA(true, true, true); break;
  }
#undef LC_GA
  LC_RETURN_LAST_ERROR();
}

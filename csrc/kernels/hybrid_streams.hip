// Kernels of hybrid decoder designs whose residual is several parallel streams (hyper-connections), and of
// attention variants around the shared attention kernels of hybrid.hip: rotary positions on queries, keys AND
// values in either pair layout with the paged cache write, the mix of the heads' softmax weights ("talking heads")
// applied behind the weighted sums, latent attention whose cached row carries a rotated key part shared by all
// heads, and the xIELU activation of a dense feed-forward.
//
// Hyper-connections: S streams x_1 .. x_S per token, fp32 [T, S, d]. A sublayer reads u = sum_s in[s] x_s through
// an RMS norm and writes, all streams at once from the old ones, x_t <- sum_s mix[s, t] x_s + out[t] y. The write
// of one sublayer, the read of the next and its norm are one launch; nothing but fp32 touches the streams.
//
// Angles are position * frequency formed in fp64 from fp64 frequencies and reduced to [-pi, pi] before the fp32
// sine / cosine; a token's table of them is built once per block in LDS.
#include "hybrid_common.h"

namespace {

constexpr int kMaxStreams = 8;

LC_DEVICE void angle_table(float* cs, int half, double pos, const double* __restrict__ inv_freq) {
  // cs[j] = cos, cs[half + j] = sin of pos * inv_freq[j]
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    constexpr double kTwoPi = 6.283185307179586476925286766559;
    double a = pos * inv_freq[j];
    a -= kTwoPi * rint(a / kTwoPi);
    float s, c;
    sincosf(static_cast<float>(a), &s, &c);
    cs[j] = c;
    cs[half + j] = s;
  }
}

// Coordinate i (< dims) of a head that starts at ``head`` after the turn by the table's angles times ``sign``.
// pairs = 0: i is paired with i +- dims / 2; pairs = 1: 2m with 2m + 1.
LC_DEVICE float turned(const float* __restrict__ head, int i, int dims, const float* cs, int pairs, float sign) {
  const int half = dims >> 1;
  const float a = head[i];
  if (pairs) {
    const float c = cs[i >> 1], s = sign * cs[half + (i >> 1)];
    const float other = head[i ^ 1];
    return (i & 1) ? a * c + other * s : a * c - other * s;
  }
  const int j = i < half ? i : i - half;
  const float c = cs[j], s = sign * cs[half + j];
  return i < half ? a * c - head[i + half] * s : a * c + head[i - half] * s;
}

// ---------------------------------------------------------------- streams: start
// xs[t, s, :] = x0[t] / sqrt(mean(x0[t]^2) + eps) * w for every stream s. WAVES = 1: a wave per row, four rows per
// block; WAVES = 4: a block per row (few rows).
template <int WAVES>
__global__ __launch_bounds__(256) void hc_init_kernel(const float* __restrict__ x0, const float* __restrict__ w,
                                                      float eps, float* __restrict__ xs, int T, int S, int d) {
  __shared__ float red[16];
  constexpr int LANES = 64 * WAVES;
  const int row = WAVES == 1 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  const int lane = WAVES == 1 ? (threadIdx.x & 63) : threadIdx.x;
  if (WAVES == 1 && row >= T) return;
  const float* xr = x0 + static_cast<size_t>(row) * d;
  float ss = 0.f;
  for (int c = lane; c < d; c += LANES) ss += xr[c] * xr[c];
  ss = WAVES == 1 ? wave_sum(ss) : block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / static_cast<float>(d) + eps);
  float* dst = xs + static_cast<size_t>(row) * S * d;
  for (int c = lane; c < d; c += LANES) {
    const float v = xr[c] * r * w[c];
    for (int s = 0; s < S; ++s) dst[static_cast<size_t>(s) * d + c] = v;
  }
}

// ---------------------------------------------------------------- streams: one sublayer's write, the next one's read
// With y: xs[t, j, :] <- sum_s mix[s * S + j] xs[t, s, :] + outw[j] y[t, :] (in place: a thread owns a coordinate of
// all streams). With inw: u = sum_s inw[s] xs[t, s, :] (of the new streams); u goes to ``u_out`` (fp32) when given,
// and u / sqrt(mean(u^2) + eps) * normw to ``xa`` in the activation type when a norm weight is given. SMAX: the
// register arrays' size (S <= SMAX). Rows of up to 8 coordinates per thread are handled in one unrolled sweep (all
// loads in flight together, u kept in registers for the norm); wider rows loop and form u again after the reduction.
template <int SMAX>
struct StreamCoef {
  const float* m;   // [S][S] from, to
  const float* o;   // [S]
  const float* i;   // [S]
};

template <int SMAX>
LC_DEVICE float hc_point(float* __restrict__ xr, const float* __restrict__ yr, const StreamCoef<SMAX>& k, int S, int d, int c,
                         bool read) {
  float v[SMAX];
#pragma unroll
  for (int s = 0; s < SMAX; ++s) v[s] = s < S ? xr[static_cast<size_t>(s) * d + c] : 0.f;
  if (yr != nullptr) {
    const float yv = yr[c];
    float n[SMAX];
#pragma unroll
    for (int j = 0; j < SMAX; ++j) {
      float a = 0.f;
      if (j < S) {
#pragma unroll
        for (int s = 0; s < SMAX; ++s)
          if (s < S) a += k.m[s * S + j] * v[s];
        a += k.o[j] * yv;
        xr[static_cast<size_t>(j) * d + c] = a;
      }
      n[j] = a;
    }
#pragma unroll
    for (int j = 0; j < SMAX; ++j) v[j] = n[j];
  }
  float u = 0.f;
  if (read) {
#pragma unroll
    for (int s = 0; s < SMAX; ++s)
      if (s < S) u += k.i[s] * v[s];
  }
  return u;
}

template <bool AF32, int WAVES, int SMAX>
__global__ __launch_bounds__(256) void hc_step_kernel(float* __restrict__ xs, const float* __restrict__ y,
                                                      const float* __restrict__ mix, const float* __restrict__ outw,
                                                      const float* __restrict__ inw, const float* __restrict__ normw,
                                                      float eps, float* __restrict__ u_out, void* __restrict__ xa, int T,
                                                      int S, int d) {
  __shared__ float red[16];
  __shared__ float coef[SMAX * SMAX + 2 * SMAX];
  constexpr int LANES = 64 * WAVES;
  constexpr int UMAX = 8;
  const int row = WAVES == 1 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  const int lane = WAVES == 1 ? (threadIdx.x & 63) : threadIdx.x;
  for (int i = threadIdx.x; i < S * S; i += blockDim.x) coef[i] = y != nullptr ? mix[i] : 0.f;
  for (int i = threadIdx.x; i < S; i += blockDim.x) {
    coef[SMAX * SMAX + i] = y != nullptr ? outw[i] : 0.f;
    coef[SMAX * SMAX + SMAX + i] = inw != nullptr ? inw[i] : 0.f;
  }
  __syncthreads();
  const StreamCoef<SMAX> k{coef, coef + SMAX * SMAX, coef + SMAX * SMAX + SMAX};
  const bool on = WAVES != 1 || row < T;             // (idle waves still take part in the barriers)
  float* xr = xs + static_cast<size_t>(on ? row : 0) * S * d;
  const float* yr = y != nullptr ? y + static_cast<size_t>(on ? row : 0) * d : nullptr;
  const bool read = inw != nullptr;
  const bool fits = d <= LANES * UMAX;               // the same for every thread
  float ss = 0.f;
  float u[UMAX];
  if (on && fits) {
#pragma unroll
    for (int e = 0; e < UMAX; ++e) {
      const int c = lane + e * LANES;
      u[e] = c < d ? hc_point<SMAX>(xr, yr, k, S, d, c, read) : 0.f;
      ss += u[e] * u[e];
      if (u_out != nullptr && c < d) u_out[static_cast<size_t>(row) * d + c] = u[e];
    }
  } else if (on) {
    for (int c = lane; c < d; c += LANES) {
      const float uv = hc_point<SMAX>(xr, yr, k, S, d, c, read);
      ss += uv * uv;
      if (u_out != nullptr) u_out[static_cast<size_t>(row) * d + c] = uv;
    }
  }
  if (normw == nullptr || !read) return;             // the same for every thread
  ss = WAVES == 1 ? wave_sum(ss) : block_sum(ss, red);
  if (!on) return;
  const float r = 1.f / sqrtf(ss / static_cast<float>(d) + eps);
  typename Act<AF32>::type* a = static_cast<typename Act<AF32>::type*>(xa);
  if (fits) {
#pragma unroll
    for (int e = 0; e < UMAX; ++e) {
      const int c = lane + e * LANES;
      if (c < d) Act<AF32>::store(a, static_cast<size_t>(row) * d + c, u[e] * r * normw[c]);
    }
  } else {
    for (int c = lane; c < d; c += LANES)            // the same sum in the same order as above, from the new streams
      Act<AF32>::store(a, static_cast<size_t>(row) * d + c, hc_point<SMAX>(xr, nullptr, k, S, d, c, true) * r * normw[c]);
  }
}

// ---------------------------------------------------------------- rotary positions on q, k and v; cache write
// One block per token. qkv [T, ld] fp32: q [H*D] | k [G*D] | v [G*Dv] (biases already added by the product). The
// first rot_dims coordinates of every query and key head turn by position * inv_freq[i] in the pair layout
// ``pairs`` (0: i with i + rot_dims / 2; 1: neighbours); with ``inv_freq_v`` every value head turns over its whole
// width by position * inv_freq_v[m] in the layout ``v_pairs``, and is cached so. Keys go to [blocks, G, BS, D],
// values to [blocks, G, BS, Dv] at the token's slot; the turned queries to q_out [T, H*D].
template <bool CF32>
__global__ __launch_bounds__(256) void rope_qkv_write_kernel(
    const float* __restrict__ qkv, int ld, const double* __restrict__ inv_freq, const double* __restrict__ inv_freq_v,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slot_mapping, void* __restrict__ kc,
    void* __restrict__ vc, float* __restrict__ q_out, int H, int G, int D, int Dv, int BS, int rot_dims, int pairs,
    int v_pairs) {
  extern __shared__ float cs_dyn[];                // [rot_dims] for q / k, then [Dv] for v
  const int t = blockIdx.x;
  const float* row = qkv + static_cast<size_t>(t) * ld;
  const double pos = static_cast<double>(positions[t]);
  float* cs_v = cs_dyn + rot_dims;
  angle_table(cs_dyn, rot_dims >> 1, pos, inv_freq);
  if (inv_freq_v != nullptr) angle_table(cs_v, Dv >> 1, pos, inv_freq_v);
  __syncthreads();
  const int nq = H * D, nk = G * D, nv = G * Dv;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    const int c = i % D;
    q_out[static_cast<size_t>(t) * nq + i] = c < rot_dims ? turned(row + i - c, c, rot_dims, cs_dyn, pairs, 1.f) : row[i];
  }
  const int slot = slot_mapping[t];
  if (slot < 0 || kc == nullptr) return;
  const size_t blk = slot / BS, off = slot % BS;
  typename Act<CF32>::type* kd = static_cast<typename Act<CF32>::type*>(kc);
  typename Act<CF32>::type* vd = static_cast<typename Act<CF32>::type*>(vc);
  const float* k = row + nq;
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int c = i % D;
    const float r = c < rot_dims ? turned(k + i - c, c, rot_dims, cs_dyn, pairs, 1.f) : k[i];
    Act<CF32>::store(kd, ((blk * G + i / D) * BS + off) * D + c, r);
  }
  const float* v = k + nk;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const int c = i % Dv;
    const float r = inv_freq_v != nullptr ? turned(v + i - c, c, Dv, cs_v, v_pairs, 1.f) : v[i];
    Act<CF32>::store(vd, ((blk * G + i / Dv) * BS + off) * Dv + c, r);
  }
}

// ---------------------------------------------------------------- mixed heads' weights behind the weighted sums
// One block per token. o [T, H, G, Dv] fp32: head g's softmax weights applied to the values of EVERY key/value head
// c. Mixing the weights of the heads by talk [H, H] before they meet the values is linear in them, so it is done
// on these sums: out[t, h, :] = sum_g talk[h, g] o[t, g, kv(h), :] with kv(h) = h / (H / G). With ``inv_freq_v``
// the result turns back by -position * inv_freq_v[m] over its whole width (values cached turned by their own
// position leave a sum that depends on position differences only).
template <bool AF32>
__global__ __launch_bounds__(256) void talk_mix_kernel(const float* __restrict__ o, const float* __restrict__ talk,
                                                       const int32_t* __restrict__ positions,
                                                       const double* __restrict__ inv_freq_v, void* __restrict__ out, int H,
                                                       int G, int Dv, int v_pairs) {
  extern __shared__ float lds_tm[];                // mixed [Dv], then cos / sin [Dv]
  const int t = blockIdx.x, h = blockIdx.y;        // a block per (token, head)
  float* mixed = lds_tm;
  float* cs = lds_tm + Dv;
  if (inv_freq_v != nullptr) angle_table(cs, Dv >> 1, static_cast<double>(positions[t]), inv_freq_v);
  const int kv = h / (H / G);
  const float* ot = o + (static_cast<size_t>(t) * H * G + kv) * Dv;
  for (int c = threadIdx.x; c < Dv; c += blockDim.x) {
    float a = 0.f;
    for (int g = 0; g < H; ++g) a += talk[h * H + g] * ot[static_cast<size_t>(g) * G * Dv + c];
    mixed[c] = a;
  }
  __syncthreads();
  typename Act<AF32>::type* dst = static_cast<typename Act<AF32>::type*>(out);
  for (int c = threadIdx.x; c < Dv; c += blockDim.x) {
    const float r = inv_freq_v != nullptr ? turned(mixed, c, Dv, cs, v_pairs, -1.f) : mixed[c];
    Act<AF32>::store(dst, (static_cast<size_t>(t) * H + h) * Dv + c, r);
  }
}

// ---------------------------------------------------------------- latent attention with a shared rotated key part
// One block per token. proj [T, ld] fp32 holds the queries from column 0, head by head [D plain | rd to turn], and
// (when the layer has a down-projection of its own) R + rd columns from ``col_c`` on: the compressed row and the key
// part all heads share. The cache row [R + rd] at the token's slot gets rms_norm(compressed) * w | turned key part;
// the turned query parts go to columns R .. R + rd - 1 of each head's block of qlat [T, H * (R + rd)], whose first R
// columns per head (the query in the compressed row's coordinates) another launch writes.
template <bool CF32>
__global__ __launch_bounds__(256) void latent_rope_write_kernel(
    const float* __restrict__ proj, int ld, int col_c, const float* __restrict__ w, float eps,
    const double* __restrict__ inv_freq, const int32_t* __restrict__ positions, const int32_t* __restrict__ slot_mapping,
    void* __restrict__ cache, float* __restrict__ qlat, int H, int D, int R, int rd, int BS, int pairs) {
  extern __shared__ float cs_lat[];                // cos / sin [rd]
  __shared__ float red[16];
  const int t = blockIdx.x;
  const float* row = proj + static_cast<size_t>(t) * ld;
  angle_table(cs_lat, rd >> 1, static_cast<double>(positions[t]), inv_freq);
  __syncthreads();
  const int W = R + rd;
  for (int i = threadIdx.x; i < H * rd; i += blockDim.x) {
    const int h = i / rd, c = i - h * rd;
    qlat[(static_cast<size_t>(t) * H + h) * W + R + c] = turned(row + h * (D + rd) + D, c, rd, cs_lat, pairs, 1.f);
  }
  if (cache == nullptr) return;                    // the same for every thread
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const float* c0 = row + col_c;
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += blockDim.x) ss += c0[c] * c0[c];
  const float r = 1.f / sqrtf(block_sum(ss, red) / static_cast<float>(R) + eps);
  typename Act<CF32>::type* dst = static_cast<typename Act<CF32>::type*>(cache);
  for (int c = threadIdx.x; c < R; c += blockDim.x) Act<CF32>::store(dst, static_cast<size_t>(slot) * W + c, c0[c] * r * w[c]);
  for (int c = threadIdx.x; c < rd; c += blockDim.x)
    Act<CF32>::store(dst, static_cast<size_t>(slot) * W + R + c, turned(c0 + R, c, rd, cs_lat, pairs, 1.f));
}

// ---------------------------------------------------------------- xIELU
// z > 0: ap z^2 + z / 2; z <= 0: an (exp(z) - 1 - z) + z / 2 (ap = softplus(p), an = 1/2 + softplus(q), made by the
// host). y fp32 [T, n] with row stride ld (a column block of a wider matrix); out [T, n] in the activation type.
template <bool AF32>
__global__ void xielu_kernel(const float* __restrict__ y, int ld, void* __restrict__ out, long long total, int n, float ap,
                             float an) {
  const long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long long t = i / n;
  const float z = y[t * ld + (i - t * n)];
  const float r = z > 0.f ? ap * z * z + 0.5f * z : an * (expm1f(z) - z) + 0.5f * z;
  Act<AF32>::store(static_cast<typename Act<AF32>::type*>(out), i, r);
}

}  // namespace

// ================================================================= launchers
LC_EXPORT int lc_hc_init(const void* x0, const void* w, float eps, void* xs, int T, int S, int d, hipStream_t st) {
  if (T <= 0) return 0;
  if (d <= 0 || S <= 0 || x0 == nullptr || w == nullptr || xs == nullptr) return -1;
  const bool few = T <= 512;
  const dim3 grid(few ? T : (T + 3) / 4), block(256);
  if (few)
    hc_init_kernel<4><<<grid, block, 0, st>>>(static_cast<const float*>(x0), static_cast<const float*>(w), eps,
                                              static_cast<float*>(xs), T, S, d);
  else
    hc_init_kernel<1><<<grid, block, 0, st>>>(static_cast<const float*>(x0), static_cast<const float*>(w), eps,
                                              static_cast<float*>(xs), T, S, d);
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_hc_step(void* xs, const void* y, const void* mix, const void* outw, const void* inw, const void* normw,
                         float eps, void* u_out, void* xa, int act_f32, int T, int S, int d, hipStream_t st) {
  if (T <= 0) return 0;
  if (d <= 0 || S <= 0 || S > kMaxStreams || xs == nullptr) return -1;
  if (y != nullptr && (mix == nullptr || outw == nullptr)) return -1;
  if (normw != nullptr && (inw == nullptr || xa == nullptr)) return -1;
  if (u_out != nullptr && inw == nullptr) return -1;
  const bool few = T <= 512;
  const dim3 grid(few ? T : (T + 3) / 4), block(256);
#define LC_HC(A32, WAVES, SMAX)                                                                                    \
  hc_step_kernel<A32, WAVES, SMAX><<<grid, block, 0, st>>>(                                                        \
      static_cast<float*>(xs), static_cast<const float*>(y), static_cast<const float*>(mix),                       \
      static_cast<const float*>(outw), static_cast<const float*>(inw), static_cast<const float*>(normw), eps,      \
      static_cast<float*>(u_out), xa, T, S, d)
#define LC_HC_S(A32, WAVES)               \
  if (S <= 2) LC_HC(A32, WAVES, 2);       \
  else if (S <= 4) LC_HC(A32, WAVES, 4);  \
  else LC_HC(A32, WAVES, kMaxStreams)
  if (act_f32 && few) { LC_HC_S(true, 4); }
  else if (act_f32) { LC_HC_S(true, 1); }
  else if (few) { LC_HC_S(false, 4); }
  else { LC_HC_S(false, 1); }
#undef LC_HC_S
#undef LC_HC
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_rope_qkv_write(const void* qkv, int ld, const void* inv_freq, const void* inv_freq_v,
                                const void* positions, const void* slot_mapping, void* kc, void* vc, int cache_f32,
                                void* q_out, int T, int H, int G, int D, int Dv, int BS, int rot_dims, int pairs,
                                int v_pairs, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || D <= 0 || Dv <= 0 || BS <= 0 || rot_dims < 0 || rot_dims > D || (rot_dims & 1)) return -1;
  if (ld < H * D + G * (D + Dv) || q_out == nullptr || (kc == nullptr) != (vc == nullptr)) return -1;
  if ((rot_dims > 0 && inv_freq == nullptr) || (inv_freq_v != nullptr && (Dv & 1))) return -1;
  const size_t lds = static_cast<size_t>(rot_dims + Dv + 1) * sizeof(float);
  if (lds > 64 * 1024) return -1;
#define LC_RQ(C32)                                                                                                   \
  rope_qkv_write_kernel<C32><<<dim3(T), dim3(256), lds, st>>>(                                                       \
      static_cast<const float*>(qkv), ld, static_cast<const double*>(inv_freq), static_cast<const double*>(inv_freq_v), \
      static_cast<const int32_t*>(positions), static_cast<const int32_t*>(slot_mapping), kc, vc,                     \
      static_cast<float*>(q_out), H, G, D, Dv, BS, rot_dims, pairs, v_pairs)
  if (cache_f32) LC_RQ(true);
  else LC_RQ(false);
#undef LC_RQ
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_talk_mix(const void* o, const void* talk, const void* positions, const void* inv_freq_v, void* out,
                          int act_f32, int T, int H, int G, int Dv, int v_pairs, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || Dv <= 0 || o == nullptr || talk == nullptr || out == nullptr) return -1;
  if (inv_freq_v != nullptr && ((Dv & 1) || positions == nullptr)) return -1;
  const size_t lds = static_cast<size_t>(2 * Dv + 1) * sizeof(float);
  if (lds > 64 * 1024 || H > 65535) return -1;
  const int threads = Dv <= 64 ? 64 : (Dv <= 128 ? 128 : 256);
#define LC_TM(A32)                                                                                               \
  talk_mix_kernel<A32><<<dim3(T, H), dim3(threads), lds, st>>>(static_cast<const float*>(o), static_cast<const float*>(talk), \
                                                        static_cast<const int32_t*>(positions),                  \
                                                        static_cast<const double*>(inv_freq_v), out, H, G, Dv, v_pairs)
  if (act_f32) LC_TM(true);
  else LC_TM(false);
#undef LC_TM
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_latent_rope_write(const void* proj, int ld, int col_c, const void* w, float eps, const void* inv_freq,
                                   const void* positions, const void* slot_mapping, void* cache, int cache_f32, void* qlat,
                                   int T, int H, int D, int R, int rd, int BS, int pairs, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || D < 0 || R <= 0 || rd < 0 || (rd & 1) || BS <= 0 || qlat == nullptr || ld < H * (D + rd)) return -1;
  if (rd > 0 && (inv_freq == nullptr || positions == nullptr)) return -1;
  if (cache != nullptr && (w == nullptr || slot_mapping == nullptr || col_c < H * (D + rd) || ld < col_c + R + rd)) return -1;
  const size_t lds = static_cast<size_t>(rd + 1) * sizeof(float);
  if (lds > 64 * 1024) return -1;
#define LC_LR(C32)                                                                                                  \
  latent_rope_write_kernel<C32><<<dim3(T), dim3(256), lds, st>>>(                                                   \
      static_cast<const float*>(proj), ld, col_c, static_cast<const float*>(w), eps, static_cast<const double*>(inv_freq), \
      static_cast<const int32_t*>(positions), static_cast<const int32_t*>(slot_mapping), cache,                     \
      static_cast<float*>(qlat), H, D, R, rd, BS, pairs)
  if (cache_f32) LC_LR(true);
  else LC_LR(false);
#undef LC_LR
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_xielu(const void* y, int ld, void* out, int act_f32, int T, int n, float ap, float an, hipStream_t st) {
  if (T <= 0 || n <= 0) return 0;
  if (ld < n) return -1;
  const long long total = static_cast<long long>(T) * n;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256)), block(256);
  if (act_f32)
    xielu_kernel<true><<<grid, block, 0, st>>>(static_cast<const float*>(y), ld, out, total, n, ap, an);
  else
    xielu_kernel<false><<<grid, block, 0, st>>>(static_cast<const float*>(y), ld, out, total, n, ap, an);
  LC_RETURN_LAST_ERROR();
}

// Routed feed-forwards of hybrid decoder designs: a softmax or sigmoid router with a bias-corrected,
// group-limited top-k choice, a counting sort of the (token, choice) pairs by expert for any number
// of experts, per-expert products of any shape and type over the sorted rows (fp32 accumulation on
// the vector ALUs, like the shape-agnostic GEMM), and the fp32 mix of the chosen experts' outputs,
// in which experts without tensors ("identity experts") return their input.
#include "hybrid_common.h"

namespace {

constexpr int kMaxTop = 32;
constexpr int kMaxGroups = 64;

// ---------------------------------------------------------------- routing
// One wave per token. z [T, n] fp32 router logits (row stride ld). s = softmax(z) (score_fn 0) or sigmoid(z), each
// output on its own (score_fn 1); choice = s + correction (no correction given: s); the n
// outputs form ``groups`` runs of n / groups neighbours, a run's score is its largest choice, the
// ``keep`` best runs stay eligible (ties: the lower index); the ``top`` largest eligible choices are
// taken (ties: the lower index) with weights s * scale.
__global__ __launch_bounds__(256) void route_grouped_kernel(const float* __restrict__ z, int ld,
                                                            const float* __restrict__ corr, int T, int n, int top,
                                                            int groups, int keep, float scale, int score_fn,
                                                            int32_t* __restrict__ ids, float* __restrict__ wts) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;                               // no block-wide barrier below
  float* sc = lds + static_cast<size_t>(wave) * (2 * n + 2 * kMaxGroups);   // softmax scores
  float* ch = sc + n;                               // choice scores (-inf once taken or not eligible)
  float* gs = ch + n;                               // group scores
  float* ok = gs + kMaxGroups;                      // 1: the group is eligible
  const float* zr = z + static_cast<size_t>(t) * ld;
  float inv = 1.f;
  if (score_fn == 1) {
    for (int e = lane; e < n; e += 64) sc[e] = sigmoidf_(zr[e]);
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < n; e += 64) mx = fmaxf(mx, zr[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < n; e += 64) {
      const float p = expf(zr[e] - mx);
      sc[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    inv = 1.f / sum;
  }
  for (int e = lane; e < n; e += 64) {
    const float s = sc[e] * inv;
    sc[e] = s;
    ch[e] = corr != nullptr ? s + corr[e] : s;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (keep < groups) {
    const int gsz = n / groups;
    for (int g = lane; g < groups; g += 64) {
      float m = -INFINITY;
      for (int j = 0; j < gsz; ++j) m = fmaxf(m, ch[g * gsz + j]);
      gs[g] = m;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int g = lane; g < groups; g += 64) {
      int rank = 0;
      const float mine = gs[g];
      for (int j = 0; j < groups; ++j) rank += (gs[j] > mine || (gs[j] == mine && j < g)) ? 1 : 0;
      ok[g] = rank < keep ? 1.f : 0.f;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int e = lane; e < n; e += 64)
      if (ok[e / gsz] == 0.f) ch[e] = -INFINITY;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < n; e += 64) {
      const float v = ch[e];
      if (v > best) {                               // a lane walks its outputs in rising order: ties keep the lower one
        best = v;
        at = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oa = __shfl_xor(at, off, 64);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (at >= n) at = k < n ? k : 0;                // nothing eligible is left (NaN logits): still a valid expert
    if (lane == 0) {
      ids[static_cast<size_t>(t) * top + k] = at;
      wts[static_cast<size_t>(t) * top + k] = sc[at] * scale;
      ch[at] = -INFINITY;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// ---------------------------------------------------------------- sort of the pairs by expert
// One block. ids [A] (A = T * top, pair a = token a / top). offsets [n + 1]: first sorted position of
// every expert; sorted_src [A]: token of every sorted position; slot_of [A]: sorted position of pair a;
// with ``wts`` [A] also sorted_wts [A]: the pair's weight at its sorted position.
// The order inside an expert is whatever the atomics give; every row is computed on its own, so
// the values do not depend on it.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int32_t* __restrict__ ids, int A, int top, int n,
                                                        int32_t* __restrict__ offsets, int32_t* __restrict__ sorted_src,
                                                        int32_t* __restrict__ slot_of, const float* __restrict__ wts,
                                                        float* __restrict__ sorted_wts) {
  extern __shared__ int cnt[];                      // [n] counts, then [n] cursors
  int* cur = cnt + n;
  for (int e = threadIdx.x; e < n; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int a = threadIdx.x; a < A; a += blockDim.x) {
    const int e = ids[a];
    if (e >= 0 && e < n) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < n; ++e) {
      offsets[e] = run;
      cur[e] = run;
      run += cnt[e];
    }
    offsets[n] = run;
  }
  __syncthreads();
  for (int a = threadIdx.x; a < A; a += blockDim.x) {
    const int e = ids[a];
    if (e < 0 || e >= n) {
      slot_of[a] = 0;
      continue;
    }
    const int p = atomicAdd(&cur[e], 1);
    sorted_src[p] = a / top;
    slot_of[a] = p;
    if (wts != nullptr) sorted_wts[p] = wts[a];
  }
}

// ---------------------------------------------------------------- per-expert products over sorted rows
// Sorted position p in [offsets[e], offsets[e + 1]) gives C[p] = W[e] A[row_index[p]] (A[p] without
// an index); W [E, N, K]. Tiles of 64 positions x 64 columns as in the shape-agnostic GEMM; tile
// blockIdx.y belongs to the expert whose run of tiles it falls into (experts are walked in order;
// at most ceil(rows / 64) + E tiles exist). epi 1: square of relu.
template <bool AF32, bool WF32, bool CF32>
__global__ __launch_bounds__(256) void gemm_any_grouped_kernel(const void* __restrict__ A, int lda,
                                                               const int32_t* __restrict__ row_index,
                                                               const int32_t* __restrict__ offsets,
                                                               const void* __restrict__ W, void* __restrict__ C, int E,
                                                               int N, int K, int epi) {
  __shared__ float As[16][64 + 4];
  __shared__ float Ws[16][64 + 4];
  __shared__ int rows[64];
  int e = 0, tile = blockIdx.y, lo = 0, hi = 0;
  for (; e < E; ++e) {
    lo = offsets[e];
    hi = offsets[e + 1];
    const int nt = (hi - lo + 63) >> 6;
    if (tile < nt) break;
    tile -= nt;
  }
  if (e >= E) return;                                // the same for the whole block
  const int p0 = lo + tile * 64;
  const int M = min(64, hi - p0);
  const int n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  if (threadIdx.x < 64) rows[threadIdx.x] = threadIdx.x < M ? (row_index != nullptr ? row_index[p0 + threadIdx.x] : p0 + threadIdx.x) : 0;
  __syncthreads();
  const typename Act<AF32>::type* a = static_cast<const typename Act<AF32>::type*>(A);
  const typename Act<WF32>::type* w = static_cast<const typename Act<WF32>::type*>(W) + static_cast<size_t>(e) * N * K;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int i = threadIdx.x; i < 64 * 16; i += 256) {
      const int r = i >> 4, k = i & 15;
      As[k][r] = (r < M && k0 + k < K) ? Act<AF32>::load(a, static_cast<size_t>(rows[r]) * lda + k0 + k) : 0.f;
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
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= N) continue;
      float v = acc[i][j];
      if (epi == 1) {
        v = fmaxf(v, 0.f);
        v *= v;
      }
      Act<CF32>::store(c, static_cast<size_t>(p0 + r) * N + col, v);
    }
  }
}

// ---------------------------------------------------------------- mix of the chosen experts
// out[t] = sum_k wts[t, k] * (ye[slot_of[t, k]] if ids[t, k] < E else h[t]) (+ shared[t]), fp32. One block per token.
// No weights given: 1 (designs whose weight went into the expert's input). ``shared_gate`` (one logit per token,
// row stride ld_gate): the shared expert's row is scaled by its sigmoid.
template <bool HF32>
__global__ __launch_bounds__(256) void moe_mix_kernel(const float* __restrict__ ye, const int32_t* __restrict__ slot_of,
                                                      const int32_t* __restrict__ ids, const float* __restrict__ wts,
                                                      const void* __restrict__ h, const float* __restrict__ shared,
                                                      const float* __restrict__ shared_gate, int ld_gate,
                                                      float* __restrict__ out, int d, int top, int E) {
  __shared__ int src[kMaxTop];
  __shared__ float wk[kMaxTop];
  const int t = blockIdx.x;
  if (threadIdx.x < top) {
    const int a = t * top + threadIdx.x;
    src[threadIdx.x] = ids[a] < E ? slot_of[a] : -1;
    wk[threadIdx.x] = wts != nullptr ? wts[a] : 1.f;
  }
  __syncthreads();
  const float sg = shared_gate != nullptr ? sigmoidf_(shared_gate[static_cast<size_t>(t) * ld_gate]) : 1.f;
  const typename Act<HF32>::type* hr = static_cast<const typename Act<HF32>::type*>(h) + static_cast<size_t>(t) * d;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    float acc = shared != nullptr ? sg * shared[static_cast<size_t>(t) * d + c] : 0.f;
    for (int k = 0; k < top; ++k)
      acc += wk[k] * (src[k] >= 0 ? ye[static_cast<size_t>(src[k]) * d + c] : Act<HF32>::load(hr, c));
    out[static_cast<size_t>(t) * d + c] = acc;
  }
}

}  // namespace

// ================================================================= launchers
LC_EXPORT int lc_route_grouped(const void* z, int ld, const void* corr, int T, int n, int top, int groups, int keep,
                               float scale, int score_fn, void* ids, void* wts, hipStream_t st) {
  if (T <= 0) return 0;
  if (ld < n) return -1;
  if (n <= 0 || top <= 0 || top > kMaxTop || top > n || groups <= 0 || groups > kMaxGroups || n % groups || keep < 1 ||
      keep > groups || top > keep * (n / groups) || score_fn < 0 || score_fn > 1)
    return -1;
  const size_t lds = 4 * static_cast<size_t>(2 * n + 2 * kMaxGroups) * sizeof(float);
  if (lds > 64 * 1024) return -1;
  route_grouped_kernel<<<dim3((T + 3) / 4), dim3(256), lds, st>>>(static_cast<const float*>(z), ld,
                                                                 static_cast<const float*>(corr), T, n, top, groups, keep,
                                                                 scale, score_fn, static_cast<int32_t*>(ids),
                                                                 static_cast<float*>(wts));
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_moe_sort(const void* ids, int T, int top, int n, void* offsets, void* sorted_src, void* slot_of,
                          const void* wts, void* sorted_wts, hipStream_t st) {
  if (T <= 0) return 0;
  if (top <= 0 || n <= 0 || n > 4096 || (wts != nullptr && sorted_wts == nullptr)) return -1;
  moe_sort_kernel<<<dim3(1), dim3(1024), 2 * static_cast<size_t>(n) * sizeof(int), st>>>(
      static_cast<const int32_t*>(ids), T * top, top, n, static_cast<int32_t*>(offsets), static_cast<int32_t*>(sorted_src),
      static_cast<int32_t*>(slot_of), static_cast<const float*>(wts), static_cast<float*>(sorted_wts));
  LC_RETURN_LAST_ERROR();
}

// ``rows``: an upper bound of offsets[E] known to the host (tokens x choices).
LC_EXPORT int lc_gemm_any_grouped(const void* A, int a_f32, int lda, const void* row_index, const void* offsets,
                                  const void* W, int w_f32, void* C, int c_f32, int rows, int E, int N, int K, int epi,
                                  hipStream_t st) {
  if (rows <= 0 || N <= 0 || E <= 0) return 0;
  if (K <= 0 || lda < K) return -1;
  const int tiles = (rows + 63) / 64 + E;
  if (tiles > 65535) return -1;
  const dim3 grid((N + 63) / 64, tiles), block(256);
#define LC_GG(A32, W32, C32)                                                                                     \
  gemm_any_grouped_kernel<A32, W32, C32><<<grid, block, 0, st>>>(A, lda, static_cast<const int32_t*>(row_index), \
                                                                 static_cast<const int32_t*>(offsets), W, C, E, N, K, epi)
  const int sel = (a_f32 ? 4 : 0) | (w_f32 ? 2 : 0) | (c_f32 ? 1 : 0);
  switch (sel) {
    case 0: LC_GG(false, false, false); break;
    case 1: LC_GG(false, false, true); break;
    case 2: LC_GG(false, true, false); break;
    case 3: LC_GG(false, true, true); break;
    case 4: LC_GG(true, false, false); break;
    case 5: LC_GG(true, false, true); break;
    case 6: LC_GG(true, true, false); break;
    default: LC_GG(true, true, true); break;
  }
#undef LC_GG
  LC_RETURN_LAST_ERROR();
}

LC_EXPORT int lc_moe_mix(const void* ye, const void* slot_of, const void* ids, const void* wts, const void* h, int h_f32,
                         const void* shared, const void* shared_gate, int ld_gate, void* out, int T, int d, int top, int E,
                         hipStream_t st) {
  if (T <= 0) return 0;
  if (d <= 0 || top <= 0 || top > kMaxTop || (shared_gate != nullptr && (shared == nullptr || ld_gate < 1))) return -1;
  if (h_f32)
    moe_mix_kernel<true><<<dim3(T), dim3(256), 0, st>>>(static_cast<const float*>(ye), static_cast<const int32_t*>(slot_of),
                                                        static_cast<const int32_t*>(ids), static_cast<const float*>(wts), h,
                                                        static_cast<const float*>(shared),
                                                        static_cast<const float*>(shared_gate), ld_gate,
                                                        static_cast<float*>(out), d, top, E);
  else
    moe_mix_kernel<false><<<dim3(T), dim3(256), 0, st>>>(static_cast<const float*>(ye), static_cast<const int32_t*>(slot_of),
                                                         static_cast<const int32_t*>(ids), static_cast<const float*>(wts), h,
                                                         static_cast<const float*>(shared),
                                                         static_cast<const float*>(shared_gate), ld_gate,
                                                         static_cast<float*>(out), d, top, E);
  LC_RETURN_LAST_ERROR();
}

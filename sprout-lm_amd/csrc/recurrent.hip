// Mixers that keep a state of fixed size per request instead of cached keys: a gated linear recurrence over channels
// behind a short causal convolution, and retention (linear attention with a fixed decay per head).  Decays, gates,
// step sizes, unit norms and the states themselves are float32 whatever the storage type; only loads of projections
// and weights and the store of the result see it.  A step's tokens lie flat, request after request; q_start / q_len /
// state_slots (one entry per request of the step) say where a request's tokens are and which row of the state tensors
// is its own.  A kernel reads the state as the step before left it and leaves it for the next one.
#include "common.h"
#include "mfma.h"
#include "sprout_hip.h"

namespace sprout {

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

// Kernels that take a block per chunk number the chunks of a step's requests without gaps to speak of: chunk ci of request
// r is number q_start[r] / C + r + ci (a request of n tokens has at most n / C + 1 chunks, so the numbers of two requests
// never meet), and T / C + requests blocks cover them all, however unequal the requests' portions are.  Which request and
// chunk a number means: the last request whose first number is not above it (the requests' few descriptors are the same for
// the whole block).  False: the number is one of the few that no chunk has.
__device__ __forceinline__ bool chunk_of_block(const int32_t* q_start, const int32_t* q_len, int n_seqs, int C, int number,
                                               int& request, int& chunk) {
  int lo = 0, hi = n_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] / C + mid <= number) lo = mid;
    else hi = mid - 1;
  }
  request = lo;
  chunk = number - (q_start[lo] / C + lo);
  return chunk * C < q_len[lo];
}

// ------------------------------------------------------------------------------------------------ gated linear recurrence
struct LruArgs {
  const void* proj;            // [T, stride]: the gate branch (before its activation) at y_off, the recurrent branch at x_off
  long long stride;
  int y_off, x_off;
  int width, blocks, taps;
  const void* conv_w;          // [width, taps], the last column is the current token's
  const void* conv_b;          // [width]
  const void* wa;              // [blocks, n(in), n(out)], n = width / blocks: the recurrence gate's matrices, input-major
  const void* ba;              // [blocks, n]
  const void* wi;              // the input gate's, likewise
  const void* bi;
  const void* lam;             // [width]
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* seq_of_token;
  const int32_t* state_slots;
  float* state;                // [slots, width]
  float* tail;                 // [slots, taps - 1, width]: the convolution's inputs of the tokens before the step, oldest first
  float* decay;                // [T, width] scratch: a_t
  float* drive;                // [T, width] scratch: sqrt(1 - a_t^2) i_t u_t
  void* out;                   // [T, width]: S_t * gelu(y_t)
  int T;
};

// The convolution outputs of TT tokens from t0 on, channels c0 .. c0 + n - 1, into u_s [TT][ld].  Where a token lies in its
// request's share of the step and which state row is its request's is looked up once per token, not once per channel, so
// that the channels' loads do not each wait behind that chain.
template <typename T, int TT>
__device__ __forceinline__ void conv_outputs(const LruArgs& a, float* u_s, int t0, int c0, int n, int ld) {
  __shared__ int place[TT], row[TT];
  if (threadIdx.x < TT) {
    const int t = t0 + threadIdx.x;
    int j = 0, slot = 0;
    if (t < a.T) {
      const int s = a.seq_of_token[t];
      j = t - a.q_start[s];
      slot = a.state_slots[s];
    }
    place[threadIdx.x] = j;
    row[threadIdx.x] = slot;
  }
  __syncthreads();
  const T* proj = (const T*)a.proj;
  const int keep = a.taps - 1;
#pragma unroll 4
  for (int e = threadIdx.x; e < TT * n; e += blockDim.x) {
    const int tt = e / n, c = c0 + e % n, t = t0 + tt;
    float u = 0.f;
    if (t < a.T) {
      const int j = place[tt];
      u = to_float(((const T*)a.conv_b)[c]);
      if (j >= keep) {      // every tap's input is a token of this step: loads at addresses that are valid whatever the tap, so
        // that they are asked for together (under a condition each would wait on its own), the sum in the taps' order
#pragma unroll
        for (int tap = 0; tap < 8; ++tap) {
          const int tp = min(tap, keep);
          const float w = to_float(((const T*)a.conv_w)[size_t(c) * a.taps + tp]);
          const float x = to_float(proj[size_t(t - (keep - tp)) * a.stride + a.x_off + c]);
          if (tap < a.taps) u = fmaf(w, x, u);
        }
        for (int tap = 8; tap < a.taps; ++tap)
          u = fmaf(to_float(((const T*)a.conv_w)[size_t(c) * a.taps + tap]),
                   to_float(proj[size_t(t - (keep - tap)) * a.stride + a.x_off + c]), u);
      } else {
        const float* tail = a.tail + size_t(row[tt]) * keep * a.width;
        for (int tap = 0; tap < a.taps; ++tap) {
          const int back = keep - tap;
          const float x = j - back >= 0 ? to_float(proj[size_t(t - back) * a.stride + a.x_off + c])
                                        : tail[size_t(keep + j - back) * a.width + c];
          u = fmaf(to_float(((const T*)a.conv_w)[size_t(c) * a.taps + tap]), x, u);
        }
      }
    }
    u_s[tt * ld + e % n] = u;
  }
  __syncthreads();
}

// A block takes TT tokens of one diagonal block of channels: their convolution outputs wait in LDS; then a thread owns
// an output channel of both gates and one of `slices` equal shares of the block's inputs (256 threads = lanes x slices),
// walks its share once for all TT tokens, and the slices' sums meet in LDS.
template <typename T, int TT>
__global__ __launch_bounds__(256) void rglru_gates_kernel(LruArgs a, int lanes) {
  extern __shared__ float u_s[];      // [TT][n], then the slices' sums [slices - 1][TT][2][lanes]
  const int n = a.width / a.blocks, b = blockIdx.y, t0 = blockIdx.x * TT, c0 = b * n;
  const int slices = blockDim.x / lanes, lane = threadIdx.x % lanes, slice = threadIdx.x / lanes;
  float* sums = u_s + TT * n;
  conv_outputs<T, TT>(a, u_s, t0, c0, n, n);
  const int share = (n + slices - 1) / slices, k_first = slice * share, k_end = min(n, k_first + share);
  for (int o0 = 0; o0 < n; o0 += lanes) {
    const int o = o0 + lane;
    const bool live = o < n;
    float ra[TT], ri[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) ra[tt] = ri[tt] = 0.f;
    if (live) {
      const T* wa = (const T*)a.wa + size_t(b) * n * n + o;
      const T* wi = (const T*)a.wi + size_t(b) * n * n + o;
      int k = k_first;
      if ((n & 3) == 0 && (k_first & 3) == 0) {      // four inputs at a time: a token's four convolution outputs in one LDS read
#pragma unroll 2
        for (; k + 4 <= k_end; k += 4) {
          float va[4], vi[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            va[j] = to_float(wa[size_t(k + j) * n]);
            vi[j] = to_float(wi[size_t(k + j) * n]);
          }
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
            const float4 u = *reinterpret_cast<const float4*>(u_s + tt * n + k);
            ra[tt] = fmaf(va[3], u.w, fmaf(va[2], u.z, fmaf(va[1], u.y, fmaf(va[0], u.x, ra[tt]))));
            ri[tt] = fmaf(vi[3], u.w, fmaf(vi[2], u.z, fmaf(vi[1], u.y, fmaf(vi[0], u.x, ri[tt]))));
          }
        }
      }
      for (; k < k_end; ++k) {
        const float va = to_float(wa[size_t(k) * n]), vi = to_float(wi[size_t(k) * n]);
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          const float u = u_s[tt * n + k];
          ra[tt] = fmaf(va, u, ra[tt]);
          ri[tt] = fmaf(vi, u, ri[tt]);
        }
      }
    }
    if (slices > 1) {
      if (o0) __syncthreads();      // the sums of the channels before have been read
      if (slice) {
        float* mine = sums + size_t(slice - 1) * TT * 2 * lanes + lane;
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          mine[(2 * tt) * lanes] = ra[tt];
          mine[(2 * tt + 1) * lanes] = ri[tt];
        }
      }
      __syncthreads();
    }
    if (slice || !live) continue;
    for (int other = 1; other < slices; ++other) {
      const float* theirs = sums + size_t(other - 1) * TT * 2 * lanes + lane;
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        ra[tt] += theirs[(2 * tt) * lanes];
        ri[tt] += theirs[(2 * tt + 1) * lanes];
      }
    }
    const float bias_a = to_float(((const T*)a.ba)[c0 + o]), bias_i = to_float(((const T*)a.bi)[c0 + o]);
    const float rate = 8.0f * softplus(to_float(((const T*)a.lam)[c0 + o]));
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      const int t = t0 + tt;
      if (t >= a.T) break;
      const float log_a = -rate * sigmoid(ra[tt] + bias_a);
      a.decay[size_t(t) * a.width + c0 + o] = expf(log_a);
      a.drive[size_t(t) * a.width + c0 + o] = sqrtf(-expm1f(2.0f * log_a)) * sigmoid(ri[tt] + bias_i) * u_s[tt * n + o];
    }
  }
}

// The gates of a few tokens (a decode step) in bfloat16 storage: what counts is how soon the block's two matrices have
// come from memory.  A thread asks for eight neighbouring outputs of an input at a time (16 bytes), n / 8 threads cover an
// input's row, the block's threads beyond that share the inputs in slices; a thread's loads do not wait for each other.
template <int TT>
__global__ __launch_bounds__(256) void rglru_gates_few_kernel(LruArgs a, int slices) {
  extern __shared__ float u_s[];      // [TT][n], then the slices' sums [slices][TT][2][n]
  using T = bf16_t;
  constexpr int KB = 8;               // inputs whose rows a thread asks for at once
  const int n = a.width / a.blocks, b = blockIdx.y, t0 = blockIdx.x * TT, c0 = b * n, cols = n / 8;
  float* sums = u_s + TT * n;
  const int col = threadIdx.x % cols, slice = threadIdx.x / cols;
  const int share = (n + slices - 1) / slices, k_first = slice * share, k_end = slice < slices ? min(n, k_first + share) : 0;
  const T* wa = (const T*)a.wa + size_t(b) * n * n + col * 8;
  const T* wi = (const T*)a.wi + size_t(b) * n * n + col * 8;
  uint4 pa[KB], pi[KB];
#pragma unroll
  for (int j = 0; j < KB; ++j) {      // the first rows are on their way while the convolution is taken
    const bool in = k_first + j < k_end;
    pa[j] = in ? *reinterpret_cast<const uint4*>(wa + size_t(k_first + j) * n) : uint4{0, 0, 0, 0};
    pi[j] = in ? *reinterpret_cast<const uint4*>(wi + size_t(k_first + j) * n) : uint4{0, 0, 0, 0};
  }
  // what the first output of this thread in the last stage needs, likewise
  const int o_first = threadIdx.x % n;
  const bool ends = threadIdx.x < TT * n;
  const float bias_a0 = ends ? to_float(((const T*)a.ba)[c0 + o_first]) : 0.f;
  const float bias_i0 = ends ? to_float(((const T*)a.bi)[c0 + o_first]) : 0.f;
  const float lam0 = ends ? to_float(((const T*)a.lam)[c0 + o_first]) : 0.f;
  conv_outputs<T, TT>(a, u_s, t0, c0, n, n);
  if (slice < slices) {
    float ra[TT][8], ri[TT][8];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
      for (int j = 0; j < 8; ++j) ra[tt][j] = ri[tt][j] = 0.f;
    for (int kb = k_first; kb < k_end; kb += KB) {
      if (kb != k_first) {
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          const bool in = kb + j < k_end;
          pa[j] = in ? *reinterpret_cast<const uint4*>(wa + size_t(kb + j) * n) : uint4{0, 0, 0, 0};
          pi[j] = in ? *reinterpret_cast<const uint4*>(wi + size_t(kb + j) * n) : uint4{0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int j = 0; j < KB; ++j) {
        const int k = min(kb + j, n - 1);      // rows past the share hold zeros
        const uint32_t wa2[4] = {pa[j].x, pa[j].y, pa[j].z, pa[j].w}, wi2[4] = {pi[j].x, pi[j].y, pi[j].z, pi[j].w};
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          const float u = u_s[tt * n + k];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            ra[tt][2 * q] = fmaf(__uint_as_float(wa2[q] << 16), u, ra[tt][2 * q]);
            ra[tt][2 * q + 1] = fmaf(__uint_as_float(wa2[q] & 0xffff0000u), u, ra[tt][2 * q + 1]);
            ri[tt][2 * q] = fmaf(__uint_as_float(wi2[q] << 16), u, ri[tt][2 * q]);
            ri[tt][2 * q + 1] = fmaf(__uint_as_float(wi2[q] & 0xffff0000u), u, ri[tt][2 * q + 1]);
          }
        }
      }
    }
    float* mine = sums + size_t(slice) * TT * 2 * n + col * 8;
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        mine[(2 * tt) * n + j] = ra[tt][j];
        mine[(2 * tt + 1) * n + j] = ri[tt][j];
      }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < TT * n; e += blockDim.x) {
    const int tt = e / n, o = e % n, t = t0 + tt;
    if (t >= a.T) continue;
    const bool first = e == threadIdx.x;
    float ra = first ? bias_a0 : to_float(((const T*)a.ba)[c0 + o]), ri = first ? bias_i0 : to_float(((const T*)a.bi)[c0 + o]);
    for (int other = 0; other < slices; ++other) {
      ra += sums[(size_t(other) * TT * 2 + 2 * tt) * n + o];
      ri += sums[(size_t(other) * TT * 2 + 2 * tt + 1) * n + o];
    }
    const float rate = 8.0f * softplus(first ? lam0 : to_float(((const T*)a.lam)[c0 + o]));
    const float log_a = -rate * sigmoid(ra);
    a.decay[size_t(t) * a.width + c0 + o] = expf(log_a);
    a.drive[size_t(t) * a.width + c0 + o] = sqrtf(-expm1f(2.0f * log_a)) * sigmoid(ri) * u_s[tt * n + o];
  }
}

// A thread owns one channel of one request and walks the request's tokens; then it leaves the convolution's last inputs.
template <typename T>
__global__ __launch_bounds__(256) void rglru_scan_kernel(LruArgs a) {
  const int s = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= a.width) return;
  const int start = a.q_start[s], n = a.q_len[s], slot = a.state_slots[s], end = start + n;
  const T* proj = (const T*)a.proj;
  T* out = (T*)a.out;
  float S = a.state[size_t(slot) * a.width + c];
  int t = start;
  for (; t + 4 <= end; t += 4) {       // the loads of four tokens are asked for before the chain of sums
    float d[4], g[4], y[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      d[j] = a.decay[size_t(t + j) * a.width + c];
      g[j] = a.drive[size_t(t + j) * a.width + c];
      y[j] = to_float(proj[size_t(t + j) * a.stride + a.y_off + c]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      S = fmaf(d[j], S, g[j]);
      out[size_t(t + j) * a.width + c] = from_float<T>(S * gelu_tanh(y[j]));
    }
  }
  for (; t < end; ++t) {
    S = fmaf(a.decay[size_t(t) * a.width + c], S, a.drive[size_t(t) * a.width + c]);
    out[size_t(t) * a.width + c] = from_float<T>(S * gelu_tanh(to_float(proj[size_t(t) * a.stride + a.y_off + c])));
  }
  a.state[size_t(slot) * a.width + c] = S;
  const int keep = a.taps - 1;
  float* tail = a.tail + size_t(slot) * keep * a.width;
  for (int p = 0; p < keep; ++p) {       // ascending: an entry that moves down is read before its place is written
    const int j = n - keep + p;
    tail[size_t(p) * a.width + c] = j >= 0 ? to_float(proj[size_t(start + j) * a.stride + a.x_off + c])
                                           : tail[size_t(p + n) * a.width + c];
  }
}

// The same walk for long portions, in three passes over chunks of kScanChunk tokens so that a request's tokens are shared
// out over the chip: every chunk's own product of decays and its sum from zero; per channel the few chunks one after the
// other, which leaves every chunk the state it starts from (and the request its new state and convolution inputs); then
// every chunk again from that state, writing the output.  carry_a, carry_b: float32 [T / kScanChunk + requests, width]; chunk ci
// of request s has row q_start[s] / kScanChunk + s + ci, which keeps unequal requests' rows apart without gaps to speak of.
constexpr int kScanChunk = 64;

__global__ __launch_bounds__(256) void rglru_chunk_local_kernel(LruArgs a, float* __restrict__ carry_a,
                                                                float* __restrict__ carry_b, int n_seqs) {
  int s, ci;
  if (!chunk_of_block(a.q_start, a.q_len, n_seqs, kScanChunk, blockIdx.x, s, ci)) return;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= a.width) return;
  const int first = a.q_start[s] + ci * kScanChunk, end = min(first + kScanChunk, a.q_start[s] + a.q_len[s]);
  if (first >= end) return;
  float A = 1.f, B = 0.f;
  int t = first;
  for (; t + 8 <= end; t += 8) {
    float d[8], g[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      d[j] = a.decay[size_t(t + j) * a.width + c];
      g[j] = a.drive[size_t(t + j) * a.width + c];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      B = fmaf(d[j], B, g[j]);
      A *= d[j];
    }
  }
  for (; t < end; ++t) {
    const float d = a.decay[size_t(t) * a.width + c];
    B = fmaf(d, B, a.drive[size_t(t) * a.width + c]);
    A *= d;
  }
  const size_t at = size_t(a.q_start[s] / kScanChunk + s + ci) * a.width + c;
  carry_a[at] = A;
  carry_b[at] = B;
}

template <typename T>
__global__ __launch_bounds__(256) void rglru_chunk_carry_kernel(LruArgs a, const float* __restrict__ carry_a,
                                                                float* __restrict__ carry_b, int chunks) {
  const int s = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= a.width) return;
  const int start = a.q_start[s], n = a.q_len[s], slot = a.state_slots[s];
  const int used = (n + kScanChunk - 1) / kScanChunk;
  float S = a.state[size_t(slot) * a.width + c];
  const size_t base = size_t(start / kScanChunk + s) * a.width + c;
  for (int ci = 0; ci < used; ci += 8) {      // eight chunks' products and sums are asked for together
    float A[8], B[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const size_t at = base + size_t(min(ci + j, used - 1)) * a.width;
      A[j] = carry_a[at];
      B[j] = carry_b[at];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (ci + j < used) {
        carry_b[base + size_t(ci + j) * a.width] = S;          // what the chunk starts from
        S = fmaf(A[j], S, B[j]);
      }
    }
  }
  a.state[size_t(slot) * a.width + c] = S;
  const T* proj = (const T*)a.proj;
  const int keep = a.taps - 1;
  float* tail = a.tail + size_t(slot) * keep * a.width;
  for (int p = 0; p < keep; ++p) {
    const int j = n - keep + p;
    tail[size_t(p) * a.width + c] = j >= 0 ? to_float(proj[size_t(start + j) * a.stride + a.x_off + c])
                                           : tail[size_t(p + n) * a.width + c];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rglru_chunk_apply_kernel(LruArgs a, const float* __restrict__ carry_b, int n_seqs) {
  int s, ci;
  if (!chunk_of_block(a.q_start, a.q_len, n_seqs, kScanChunk, blockIdx.x, s, ci)) return;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= a.width) return;
  const int first = a.q_start[s] + ci * kScanChunk, end = min(first + kScanChunk, a.q_start[s] + a.q_len[s]);
  if (first >= end) return;
  const T* proj = (const T*)a.proj;
  T* out = (T*)a.out;
  float S = carry_b[size_t(a.q_start[s] / kScanChunk + s + ci) * a.width + c];
  int t = first;
  for (; t + 8 <= end; t += 8) {
    float d[8], g[8], y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      d[j] = a.decay[size_t(t + j) * a.width + c];
      g[j] = a.drive[size_t(t + j) * a.width + c];
      y[j] = to_float(proj[size_t(t + j) * a.stride + a.y_off + c]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      S = fmaf(d[j], S, g[j]);
      out[size_t(t + j) * a.width + c] = from_float<T>(S * gelu_tanh(y[j]));
    }
  }
  for (; t < end; ++t) {
    S = fmaf(a.decay[size_t(t) * a.width + c], S, a.drive[size_t(t) * a.width + c]);
    out[size_t(t) * a.width + c] = from_float<T>(S * gelu_tanh(to_float(proj[size_t(t) * a.stride + a.y_off + c])));
  }
}

// ------------------------------------------------------------------------------------------------ retention
struct RetentionArgs {
  const void* proj;            // [T, stride]: q and k (heads * dim each), v and the gate (heads * vdim each) at their offsets
  long long stride;
  int q_off, k_off, v_off, g_off;
  int heads, dim, vdim, rotary_dim;
  const float* cos_sin;        // [T, rotary_dim / 2, 2]: (cosine, sine) of every token's angles
  const float* decay;          // [heads]
  float eps;
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* state_slots;
  float* state;                // [slots, heads, dim, vdim]
  void* out;                   // [T, heads * vdim]
  int groups;                  // row groups of a block: thread = group * vdim + column
};

// One block per (request, head), token after token: S <- decay S + k v^T in registers (a thread owns one column of the
// state and every `groups`-th row), o = S^T q summed over the row groups in LDS, then the head's unit norm and gate.
template <typename T, int ROWS>
__global__ __launch_bounds__(256) void retention_kernel(RetentionArgs a) {
  extern __shared__ float lds[];      // q [dim], k [dim], partial sums [groups][vdim]
  __shared__ float scratch[16];
  const int s = blockIdx.x, h = blockIdx.y, D = a.dim, V = a.vdim, half = a.rotary_dim / 2, R = a.groups;
  float* qs = lds;
  float* ks = lds + D;
  float* part = lds + 2 * D;
  const int v = threadIdx.x % V, dr = threadIdx.x / V;
  const bool active = dr < R;
  const int start = a.q_start[s], n = a.q_len[s], slot = a.state_slots[s];
  float* kept = a.state + (size_t(slot) * a.heads + h) * D * V;
  float S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = dr + r * R;
    S[r] = active && d < D ? kept[size_t(d) * V + v] : 0.f;
  }
  const float gamma = a.decay[h], k_scale = 1.0f / sqrtf(float(D));
  const T* proj = (const T*)a.proj;
  T* out = (T*)a.out;
  for (int t = start; t < start + n; ++t) {
    const T* row = proj + size_t(t) * a.stride;
    // the value and the gate are asked for here, before the waits on the block: their way from memory is not waited for twice
    const float value_v = active ? to_float(row[a.v_off + h * V + v]) : 0.f;
    const float g = threadIdx.x < V ? to_float(row[a.g_off + h * V + threadIdx.x]) : 0.f;
    for (int i = threadIdx.x; i < 2 * D; i += blockDim.x) {
      const bool is_k = i >= D;
      const int d = is_k ? i - D : i;
      const T* src = row + (is_k ? a.k_off : a.q_off) + h * D;
      float value;
      if (d < 2 * half) {
        const int p = d < half ? d : d - half;
        const float2 cs = reinterpret_cast<const float2*>(a.cos_sin)[size_t(t) * half + p];
        const float x = to_float(src[p]), y = to_float(src[p + half]);
        value = d < half ? x * cs.x - y * cs.y : y * cs.x + x * cs.y;
      } else {
        value = to_float(src[d]);
      }
      if (is_k) ks[d] = value * k_scale;
      else qs[d] = value;
    }
    __syncthreads();
    float partial = 0.f;
    if (active) {
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int d = dr + r * R;
        if (d < D) {
          S[r] = fmaf(gamma, S[r], ks[d] * value_v);
          partial = fmaf(S[r], qs[d], partial);
        }
      }
      part[dr * V + v] = partial;
    }
    __syncthreads();
    float o = 0.f;
    if (threadIdx.x < V)
      for (int j = 0; j < R; ++j) o += part[j * V + threadIdx.x];
    const float squares = block_sum(o * o, scratch);
    if (threadIdx.x < V) {
      const float unit = 1.0f / sqrtf(squares / float(V) + a.eps);
      out[(size_t(t) * a.heads + h) * V + threadIdx.x] = from_float<T>((o * unit) * (g * sigmoid(g)));
    }
  }
  if (active) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int d = dr + r * R;
      if (d < D) kept[size_t(d) * V + v] = S[r];
    }
  }
}

// The same sums for long portions, chunk by chunk, in three passes so that a request's tokens are shared out over the chip.
// With a chunk's tokens 0 .. n-1, its state before them S0 and decay g:
//   o_i = g^(i+1) S0^T q_i + sum_(j<=i) g^(i-j) (q_i . k_j) v_j        S_n = g^n S0 + sum_j g^(n-1-j) k_j v_j^T
// Only powers of g with exponents >= 0 appear (nothing is divided by a power), so a small decay loses nothing.
// First every chunk's own sum U = sum_j g^(n-1-j) k_j v_j^T; then per state element the chunks one after the other, which
// leaves in U's place the state each chunk starts from; then every chunk's outputs.  scratch: float32
// [T / C + requests, heads, dim, vdim]: chunk ci of request s has row q_start[s] / C + s + ci, which keeps the requests'
// rows apart (a request of n tokens has at most n / C + 1 chunks) however unequal their portions are.  A thread block is 8
// rows of 32 threads.
template <typename T>
__device__ __forceinline__ float turned(const T* src, const float* cos_sin, size_t t, int d, int half) {
  if (d < 2 * half) {
    const int p = d < half ? d : d - half;
    const float2 cs = reinterpret_cast<const float2*>(cos_sin)[t * half + p];
    const float x = to_float(src[p]), y = to_float(src[p + half]);
    return d < half ? x * cs.x - y * cs.y : y * cs.x + x * cs.y;
  }
  return to_float(src[d]);
}

// Heads too large for the registers of one block: the state stays in memory.  A thread owns columns v, v + 256, ... of the
// head's state, walks their rows for every token (S <- decay S + k v^T and the column's sum S^T q in one pass), and the
// head's unit norm needs the columns' sums only.  Any dim and vdim; slow, for sizes the other kernel does not take.
template <typename T>
__global__ __launch_bounds__(256) void retention_general_kernel(RetentionArgs a) {
  extern __shared__ float lds[];      // q [dim], k [dim], the columns' sums [vdim]
  __shared__ float scratch[16];
  const int s = blockIdx.x, h = blockIdx.y, D = a.dim, V = a.vdim, half = a.rotary_dim / 2;
  float* qs = lds;
  float* ks = lds + D;
  float* o_row = lds + 2 * D;
  const int start = a.q_start[s], n = a.q_len[s], slot = a.state_slots[s];
  float* kept = a.state + (size_t(slot) * a.heads + h) * D * V;
  const float gamma = a.decay[h], k_scale = 1.0f / sqrtf(float(D));
  const T* proj = (const T*)a.proj;
  T* out = (T*)a.out;
  for (int t = start; t < start + n; ++t) {
    const T* row = proj + size_t(t) * a.stride;
    for (int i = threadIdx.x; i < 2 * D; i += blockDim.x) {
      const bool is_k = i >= D;
      const int d = is_k ? i - D : i;
      const float value = turned(row + (is_k ? a.k_off : a.q_off) + h * D, a.cos_sin, size_t(t), d, half);
      if (is_k) ks[d] = value * k_scale;
      else qs[d] = value;
    }
    __syncthreads();
    float squares = 0.f;
    for (int v = threadIdx.x; v < V; v += blockDim.x) {
      const float value = to_float(row[a.v_off + h * V + v]);
      float o = 0.f;
      for (int d = 0; d < D; ++d) {
        const float S = fmaf(gamma, kept[size_t(d) * V + v], ks[d] * value);
        kept[size_t(d) * V + v] = S;
        o = fmaf(S, qs[d], o);
      }
      o_row[v] = o;
      squares = fmaf(o, o, squares);
    }
    squares = block_sum(squares, scratch);
    const float unit = 1.0f / sqrtf(squares / float(V) + a.eps);
    for (int v = threadIdx.x; v < V; v += blockDim.x) {      // a thread reads back what it wrote itself
      const float g = to_float(row[a.g_off + h * V + v]);
      out[(size_t(t) * a.heads + h) * V + v] = from_float<T>((o_row[v] * unit) * (g * sigmoid(g)));
    }
    __syncthreads();
  }
}

template <typename T, int CV>
__global__ __launch_bounds__(256) void retention_chunk_local_kernel(RetentionArgs a, float* __restrict__ scratch, int n_seqs, int C) {
  extern __shared__ float lds[];      // k [C][D + 1] (times its power of the decay), v [C][V]
  int s, ci;
  if (!chunk_of_block(a.q_start, a.q_len, n_seqs, C, blockIdx.x, s, ci)) return;
  const int h = blockIdx.y;
  const int D = a.dim, V = a.vdim, half = a.rotary_dim / 2, DP = D + 1;
  const int first = a.q_start[s] + ci * C, len = min(C, a.q_start[s] + a.q_len[s] - first);
  if (len <= 0) return;
  float* ks = lds;
  float* vs = lds + C * DP;
  const float gamma = a.decay[h], k_scale = 1.0f / sqrtf(float(D));
  const T* proj = (const T*)a.proj;
  for (int e = threadIdx.x; e < len * D; e += blockDim.x) {
    const int j = e / D, d = e % D;
    const T* src = proj + size_t(first + j) * a.stride + a.k_off + h * D;
    ks[j * DP + d] = (turned(src, a.cos_sin, size_t(first + j), d, half) * k_scale) * powf(gamma, float(len - 1 - j));
  }
  for (int e = threadIdx.x; e < len * V; e += blockDim.x) {
    const int j = e / V, v = e % V;
    vs[e] = to_float(proj[size_t(first + j) * a.stride + a.v_off + h * V + v]);
  }
  __syncthreads();
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  float* U = scratch + (size_t(a.q_start[s] / C + s + ci) * a.heads + h) * D * V;
  for (int d0 = 0; d0 < D; d0 += 32) {
    float acc[4][CV];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int c = 0; c < CV; ++c) acc[r][c] = 0.f;
    for (int j = 0; j < len; ++j) {
      float kk[4], vv[CV];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int d = d0 + ty + 8 * r;
        kk[r] = d < D ? ks[j * DP + d] : 0.f;
      }
#pragma unroll
      for (int c = 0; c < CV; ++c) {
        const int v = tx + 32 * c;
        vv[c] = v < V ? vs[j * V + v] : 0.f;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < CV; ++c) acc[r][c] = fmaf(kk[r], vv[c], acc[r][c]);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int d = d0 + ty + 8 * r;
#pragma unroll
      for (int c = 0; c < CV; ++c) {
        const int v = tx + 32 * c;
        if (d < D && v < V) U[size_t(d) * V + v] = acc[r][c];
      }
    }
  }
}

__global__ __launch_bounds__(256) void retention_chunk_carry_kernel(RetentionArgs a, float* __restrict__ scratch, int chunks, int C) {
  const int s = blockIdx.x, h = blockIdx.y, DV = a.dim * a.vdim, e = blockIdx.z * blockDim.x + threadIdx.x;
  if (e >= DV) return;
  const int n = a.q_len[s], slot = a.state_slots[s], used = (n + C - 1) / C;
  const float gamma = a.decay[h];
  float* kept = a.state + (size_t(slot) * a.heads + h) * DV + e;
  float S = *kept;
  const size_t step = size_t(a.heads) * DV;
  float* at = scratch + (size_t(a.q_start[s] / C + s) * a.heads + h) * DV + e;
  const float whole = powf(gamma, float(C)), last = powf(gamma, float(n - (used - 1) * C));
  for (int ci = 0; ci < used; ci += 8) {      // eight chunks' sums are asked for together (past the last: the last one's again)
    float U[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) U[j] = at[size_t(min(ci + j, used - 1)) * step];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (ci + j < used) {
        at[size_t(ci + j) * step] = S;          // what the chunk starts from
        S = fmaf(ci + j == used - 1 ? last : whole, S, U[j]);
      }
    }
  }
  *kept = S;
}

template <typename T, int C, int CV>
__global__ __launch_bounds__(256) void retention_chunk_apply_kernel(RetentionArgs a, const float* __restrict__ scratch, int n_seqs) {
  extern __shared__ float lds[];      // q, k [C][D + 1], v [C][V], weights [C][C + 1], powers of the decay [C + 1]
  constexpr int RPT = C / 8, JC = (C + 31) / 32, CP = C + 1;
  int s, ci;
  if (!chunk_of_block(a.q_start, a.q_len, n_seqs, C, blockIdx.x, s, ci)) return;
  const int h = blockIdx.y;
  const int D = a.dim, V = a.vdim, half = a.rotary_dim / 2, DP = D + 1;
  const int first = a.q_start[s] + ci * C, len = min(C, a.q_start[s] + a.q_len[s] - first);
  if (len <= 0) return;
  float* qs = lds;
  float* ks = qs + C * DP;
  float* vs = ks + C * DP;
  float* ps = vs + C * V;
  float* pw = ps + C * CP;
  const float gamma = a.decay[h], k_scale = 1.0f / sqrtf(float(D));
  const T* proj = (const T*)a.proj;
  T* out = (T*)a.out;
  for (int e = threadIdx.x; e < 2 * C * D; e += blockDim.x) {
    const bool is_k = e >= C * D;
    const int r = is_k ? e - C * D : e, j = r / D, d = r % D;
    float value = 0.f;
    if (j < len) {
      const T* src = proj + size_t(first + j) * a.stride + (is_k ? a.k_off : a.q_off) + h * D;
      value = turned(src, a.cos_sin, size_t(first + j), d, half);
      if (is_k) value *= k_scale;
    }
    (is_k ? ks : qs)[j * DP + d] = value;
  }
  for (int e = threadIdx.x; e < C * V; e += blockDim.x) {
    const int j = e / V, v = e % V;
    vs[e] = j < len ? to_float(proj[size_t(first + j) * a.stride + a.v_off + h * V + v]) : 0.f;
  }
  for (int e = threadIdx.x; e <= C; e += blockDim.x) pw[e] = powf(gamma, float(e));
  __syncthreads();
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  {
    float acc[RPT][JC];
#pragma unroll
    for (int r = 0; r < RPT; ++r)
#pragma unroll
      for (int c = 0; c < JC; ++c) acc[r][c] = 0.f;
    for (int d = 0; d < D; ++d) {
      float qq[RPT], kk[JC];
#pragma unroll
      for (int r = 0; r < RPT; ++r) qq[r] = qs[(ty + 8 * r) * DP + d];
#pragma unroll
      for (int c = 0; c < JC; ++c) {
        const int j = tx + 32 * c;
        kk[c] = j < C ? ks[j * DP + d] : 0.f;
      }
#pragma unroll
      for (int r = 0; r < RPT; ++r)
#pragma unroll
        for (int c = 0; c < JC; ++c) acc[r][c] = fmaf(qq[r], kk[c], acc[r][c]);
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r)
#pragma unroll
      for (int c = 0; c < JC; ++c) {
        const int i = ty + 8 * r, j = tx + 32 * c;
        if (j < C) ps[i * CP + j] = j <= i ? acc[r][c] * pw[i - j] : 0.f;
      }
  }
  __syncthreads();
  float o[RPT][CV];
#pragma unroll
  for (int r = 0; r < RPT; ++r)
#pragma unroll
    for (int c = 0; c < CV; ++c) o[r][c] = 0.f;
  const float* S0 = scratch + (size_t(a.q_start[s] / C + s + ci) * a.heads + h) * D * V;
  for (int d = 0; d < D; ++d) {      // what the tokens before the chunk left
    float qq[RPT], ss[CV];
#pragma unroll
    for (int r = 0; r < RPT; ++r) qq[r] = qs[(ty + 8 * r) * DP + d];
#pragma unroll
    for (int c = 0; c < CV; ++c) {
      const int v = tx + 32 * c;
      ss[c] = v < V ? S0[size_t(d) * V + v] : 0.f;
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r)
#pragma unroll
      for (int c = 0; c < CV; ++c) o[r][c] = fmaf(qq[r], ss[c], o[r][c]);
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r)
#pragma unroll
    for (int c = 0; c < CV; ++c) o[r][c] *= pw[ty + 8 * r + 1];
  for (int j = 0; j < len; ++j) {      // the chunk's own tokens
    float pp[RPT], vv[CV];
#pragma unroll
    for (int r = 0; r < RPT; ++r) pp[r] = ps[(ty + 8 * r) * CP + j];
#pragma unroll
    for (int c = 0; c < CV; ++c) {
      const int v = tx + 32 * c;
      vv[c] = v < V ? vs[j * V + v] : 0.f;
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r)
#pragma unroll
      for (int c = 0; c < CV; ++c) o[r][c] = fmaf(pp[r], vv[c], o[r][c]);
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int i = ty + 8 * r;
    float squares = 0.f;
#pragma unroll
    for (int c = 0; c < CV; ++c) squares = fmaf(o[r][c], o[r][c], squares);      // columns past V hold zeros
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) squares += __shfl_xor(squares, off);
    if (i >= len) continue;
    const float unit = 1.0f / sqrtf(squares / float(V) + a.eps);
    const T* row = proj + size_t(first + i) * a.stride;
#pragma unroll
    for (int c = 0; c < CV; ++c) {
      const int v = tx + 32 * c;
      if (v < V) {
        const float g = to_float(row[a.g_off + h * V + v]);
        out[(size_t(first + i) * a.heads + h) * V + v] = from_float<T>((o[r][c] * unit) * (g * sigmoid(g)));
      }
    }
  }
}

// Rows of q or k of a chunk into LDS [C][DP], turned, times `scale` and (where given) a weight per row; rows from `len` on
// are zeros.  An item is a pair that turns together (one cosine and sine for both numbers) or a number that does not turn;
// a thread's items are independent, so their loads are asked for together.
template <typename T>
__device__ __forceinline__ void load_turned_rows(float* dst, int DP, const T* rows, long long stride, const float* cos_sin,
                                                 int first, int len, int C, int D, int half, float scale,
                                                 const float* row_weight) {
  // every load has an address that is valid whatever the item (rows past the end read the last row, and the result is dropped):
  // loads under a condition would each wait on their own
  const int W = D - half;
  if (half > 0) {
#pragma unroll 4
    for (int e = threadIdx.x; e < C * W; e += blockDim.x) {
      const int j = e / W, i = e % W, jj = min(j, len - 1);
      const bool turns = i < half;
      const T* src = rows + size_t(jj) * stride;
      const float2 cs = reinterpret_cast<const float2*>(cos_sin)[size_t(first + jj) * half + (turns ? i : 0)];
      const float x = to_float(src[turns ? i : i + half]), y = to_float(src[i + half]);
      const float w = j < len ? (row_weight ? scale * row_weight[jj] : scale) : 0.f;
      float* row = dst + j * DP;
      if (turns) row[i] = (x * cs.x - y * cs.y) * w;
      row[i + half] = turns ? (y * cs.x + x * cs.y) * w : y * w;
    }
  } else {
#pragma unroll 4
    for (int e = threadIdx.x; e < C * D; e += blockDim.x) {
      const int j = e / D, i = e % D, jj = min(j, len - 1);
      const float y = to_float(rows[size_t(jj) * stride + i]);
      dst[j * DP + i] = j < len ? y * (row_weight ? scale * row_weight[jj] : scale) : 0.f;
    }
  }
}

template <typename T>
__device__ __forceinline__ void load_value_rows(float* dst, const T* rows, long long stride, int len, int C, int V) {
#pragma unroll 4
  for (int e = threadIdx.x; e < C * V; e += blockDim.x) {
    const int j = e / V, v = e % V;
    const float value = to_float(rows[size_t(min(j, len - 1)) * stride + v]);
    dst[e] = j < len ? value : 0.f;
  }
}

// The chunk's rows in one go, for bfloat16 rows whose sizes and offsets are all in eights (16-byte loads) and small enough
// that a thread has at most one group of eight of q, one of k and four of v: every load of a thread is asked for before
// the first is used, so a block waits for memory once.  q_dst may be null (only k and v are wanted).
__device__ __forceinline__ void unpack8(const uint4& p, float* f) {
  const uint32_t w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    f[2 * q] = __uint_as_float(w[q] << 16);
    f[2 * q + 1] = __uint_as_float(w[q] & 0xffff0000u);
  }
}

__device__ __forceinline__ void load_chunk_wide(const RetentionArgs& a, int h, int first, int len, int C, float* q_dst, float* k_dst,
                                                float* v_dst, float k_scale, const float* k_weight) {
  const int D = a.dim, V = a.vdim, half = a.rotary_dim / 2, DP = D + 1;
  const bf16_t* proj = (const bf16_t*)a.proj;
  const int groups = (D - half) / 8, items = C * groups, turning = half / 8;
  const int tid = threadIdx.x, j = min(tid / groups, C - 1), g = tid % groups, jj = min(j, len - 1);
  const bool turns = g < turning;
  const int lo_at = turns ? 8 * g : 2 * half + 8 * (g - turning), hi_at = turns ? lo_at + half : lo_at;
  const bf16_t* row = proj + size_t(first + jj) * a.stride;
  const uint4 kx = ldg128(row + a.k_off + h * D + lo_at), ky = ldg128(row + a.k_off + h * D + hi_at);
  uint4 qx = kx, qy = ky;
  if (q_dst) {
    qx = ldg128(row + a.q_off + h * D + lo_at);
    qy = ldg128(row + a.q_off + h * D + hi_at);
  }
  float4 cs[4] = {};
  if (half > 0) {
    const float4* at = reinterpret_cast<const float4*>(a.cos_sin + (size_t(first + jj) * half + (turns ? 8 * g : 0)) * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) cs[i] = at[i];
  }
  const int v_groups = V / 8, v_items = C * v_groups;
  uint4 vv[4];
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int e = min(tid + 256 * it, v_items - 1), vj = min(e / v_groups, len - 1);
    vv[it] = ldg128(proj + size_t(first + vj) * a.stride + a.v_off + h * V + 8 * (e % v_groups));
  }
  if (tid < items) {
    const bool in = j < len;
    const float wk = in ? (k_weight ? k_scale * k_weight[jj] : k_scale) : 0.f, wq = in ? 1.f : 0.f;
    float x[8], y[8];
    const float c[16] = {cs[0].x, cs[0].y, cs[0].z, cs[0].w, cs[1].x, cs[1].y, cs[1].z, cs[1].w,
                         cs[2].x, cs[2].y, cs[2].z, cs[2].w, cs[3].x, cs[3].y, cs[3].z, cs[3].w};
    unpack8(kx, x);
    unpack8(ky, y);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (turns) {
        k_dst[j * DP + lo_at + i] = (x[i] * c[2 * i] - y[i] * c[2 * i + 1]) * wk;
        k_dst[j * DP + hi_at + i] = (y[i] * c[2 * i] + x[i] * c[2 * i + 1]) * wk;
      } else {
        k_dst[j * DP + lo_at + i] = x[i] * wk;
      }
    }
    if (q_dst) {
      unpack8(qx, x);
      unpack8(qy, y);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (turns) {
          q_dst[j * DP + lo_at + i] = (x[i] * c[2 * i] - y[i] * c[2 * i + 1]) * wq;
          q_dst[j * DP + hi_at + i] = (y[i] * c[2 * i] + x[i] * c[2 * i + 1]) * wq;
        } else {
          q_dst[j * DP + lo_at + i] = x[i] * wq;
        }
      }
    }
  }
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int e = tid + 256 * it;
    if (e >= v_items) break;
    float f[8];
    unpack8(vv[it], f);
    const int vj = e / v_groups;
    float* dst = v_dst + vj * V + 8 * (e % v_groups);
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = vj < len ? f[i] : 0.f;
  }
}

// Whether load_chunk_wide takes the rows (decided on the host).
static bool retention_wide_rows(int dtype, const RetentionArgs& a, int C) {
  const int half = a.rotary_dim / 2;
  const bool eights = a.dim % 8 == 0 && half % 8 == 0 && a.vdim % 8 == 0 && a.stride % 8 == 0 && a.q_off % 8 == 0 && a.k_off % 8 == 0 &&
                      a.v_off % 8 == 0;
  return dtype == kBF16 && eights && a.dim > half && C * ((a.dim - half) / 8) <= 256 && C * (a.vdim / 8) <= 1024 &&
         (reinterpret_cast<uintptr_t>(a.proj) % 16) == 0 && (reinterpret_cast<uintptr_t>(a.cos_sin) % 16) == 0;
}

// The same three passes with the products on the matrix cores' float32 instruction (32x32x2: float32 operands and sums, no
// reduced precision), chunks of 32 tokens, a block of four waves per (chunk, head).  Lane l of a wave gives the instruction
// A[l % 32][l / 32] and B[l / 32][l % 32] and holds D[8 (r / 4) + 4 (l / 32) + r % 4][l % 32] in element r.
constexpr int kMfmaChunk = 32;

// U [dim][vdim] = sum_j (g^(n-1-j) k_j) v_j^T: a wave a tile of 32 x 32, the chunk's tokens two at a time.
template <typename T>
__global__ __launch_bounds__(256) void retention_mfma_local_kernel(RetentionArgs a, float* __restrict__ scratch, int n_seqs, int wide) {
  extern __shared__ float lds[];      // k [C][D + 1] (times its power of the decay), v [C][V]; rows past the chunk's end are zeros
  constexpr int C = kMfmaChunk;
  int s, ci;
  if (!chunk_of_block(a.q_start, a.q_len, n_seqs, C, blockIdx.x, s, ci)) return;
  const int h = blockIdx.y;
  const int D = a.dim, V = a.vdim, half = a.rotary_dim / 2, DP = D + 1;
  const int first = a.q_start[s] + ci * C, len = min(C, a.q_start[s] + a.q_len[s] - first);
  if (len <= 0) return;
  float* ks = lds;
  float* vs = lds + C * DP;
  __shared__ float weight[C];      // g^(n-1-j)
  const float gamma = a.decay[h], k_scale = 1.0f / sqrtf(float(D));
  const T* proj = (const T*)a.proj;
  if (threadIdx.x < C) weight[threadIdx.x] = threadIdx.x < len ? powf(gamma, float(len - 1 - threadIdx.x)) : 0.f;
  if (!wide) load_value_rows(vs, proj + size_t(first) * a.stride + a.v_off + h * V, a.stride, len, C, V);
  __syncthreads();
  if (wide) load_chunk_wide(a, h, first, len, C, nullptr, ks, vs, k_scale, weight);
  else load_turned_rows(ks, DP, proj + size_t(first) * a.stride + a.k_off + h * D, a.stride, a.cos_sin, first, len, C, D, half, k_scale,
                        weight);
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 31, hi = lane >> 5;
  const int tiles_v = (V + 31) / 32, tiles = ((D + 31) / 32) * tiles_v;
  float* U = scratch + (size_t(a.q_start[s] / C + s + ci) * a.heads + h) * D * V;
  for (int tile = wave; tile < tiles; tile += 4) {
    const int d0 = (tile / tiles_v) * 32, v0 = (tile % tiles_v) * 32, d = d0 + col, v = v0 + col;
    floatx16 acc = {0};
#pragma unroll
    for (int kk = 0; kk < C / 2; ++kk) {
      const int j = 2 * kk + hi;
      acc = mfma32_f32(d < D ? ks[j * DP + d] : 0.f, v < V ? vs[j * V + v] : 0.f, acc);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = d0 + 8 * (r / 4) + 4 * hi + r % 4;
      if (row < D && v < V) U[size_t(row) * V + v] = acc[r];
    }
  }
}

// The chunk's outputs.  Scores: the four waves share the key dimension and wave 0 sums, masks and weighs them; then a wave a
// tile of 32 value columns (NT tiles a wave): g^(i+1) q_i S0 over dim, the weighted scores times the values over the chunk's
// tokens, in one accumulator; the heads' unit norm over all columns through LDS; the gate; the store.
template <typename T, int NT>
__global__ __launch_bounds__(256) void retention_mfma_apply_kernel(RetentionArgs a, const float* __restrict__ scratch, int n_seqs, int wide) {
  extern __shared__ float lds[];      // q, k [C][D + 1], v [C][V], weights [C][C + 1], powers [C + 1], three partial score tiles, row sums [4][C]
  constexpr int C = kMfmaChunk, CP = C + 1;
  int s, ci;
  if (!chunk_of_block(a.q_start, a.q_len, n_seqs, C, blockIdx.x, s, ci)) return;
  const int h = blockIdx.y;
  const int D = a.dim, V = a.vdim, half = a.rotary_dim / 2, DP = D + 1;
  const int first = a.q_start[s] + ci * C, len = min(C, a.q_start[s] + a.q_len[s] - first);
  if (len <= 0) return;
  float* qs = lds;
  float* ks = qs + C * DP;
  float* vs = ks + C * DP;
  float* ps = vs + C * V;
  float* pw = ps + C * CP;
  float* parts = pw + CP;             // [3][C][CP]
  float* squares = parts + 3 * C * CP;   // [4][C]
  const float gamma = a.decay[h], k_scale = 1.0f / sqrtf(float(D));
  const T* proj = (const T*)a.proj;
  T* out = (T*)a.out;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, col = lane & 31, hi = lane >> 5;
  const float* S0 = scratch + (size_t(a.q_start[s] / C + s + ci) * a.heads + h) * D * V;
  // what the wave's first tile needs from memory later is asked for now, with the chunk's rows: the state before the chunk
  // (its first 2 PRE rows) and the gates; addresses are valid whatever the lane, what is not needed is dropped
  constexpr int PRE = 32;
  float kept0[PRE], gate0[16];
  {
    const int vc = min(wave * 32 + col, V - 1);
#pragma unroll
    for (int kk = 0; kk < PRE; ++kk) kept0[kk] = S0[size_t(min(2 * kk + hi, D - 1)) * V + vc];
#pragma unroll
    for (int r = 0; r < 16; ++r)
      gate0[r] = to_float(proj[size_t(first + min(8 * (r / 4) + 4 * hi + r % 4, len - 1)) * a.stride + a.g_off + h * V + vc]);
  }
  if (wide) {
    load_chunk_wide(a, h, first, len, C, qs, ks, vs, k_scale, nullptr);
  } else {
    load_turned_rows(qs, DP, proj + size_t(first) * a.stride + a.q_off + h * D, a.stride, a.cos_sin, first, len, C, D, half, 1.0f,
                     (const float*)nullptr);
    load_turned_rows(ks, DP, proj + size_t(first) * a.stride + a.k_off + h * D, a.stride, a.cos_sin, first, len, C, D, half, k_scale,
                     (const float*)nullptr);
    load_value_rows(vs, proj + size_t(first) * a.stride + a.v_off + h * V, a.stride, len, C, V);
  }
  for (int e = threadIdx.x; e <= C; e += blockDim.x) pw[e] = powf(gamma, float(e));
  __syncthreads();
  {
    const int steps = (D + 1) / 2, share = (steps + 3) / 4, kk_end = min(steps, (wave + 1) * share);
    floatx16 acc = {0};
    for (int kk = wave * share; kk < kk_end; ++kk) {
      const int d = 2 * kk + hi;
      const bool in = d < D;
      acc = mfma32_f32(in ? qs[col * DP + d] : 0.f, in ? ks[col * DP + d] : 0.f, acc);
    }
    if (wave) {
#pragma unroll
      for (int r = 0; r < 16; ++r) parts[((wave - 1) * C + 8 * (r / 4) + 4 * hi + r % 4) * CP + col] = acc[r];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r / 4) + 4 * hi + r % 4, j = col;
        const float sum = ((acc[r] + parts[i * CP + j]) + parts[(C + i) * CP + j]) + parts[(2 * C + i) * CP + j];
        ps[i * CP + j] = j <= i ? sum * pw[i - j] : 0.f;
      }
    }
    __syncthreads();
  }
  const int tiles_v = (V + 31) / 32;
  floatx16 o[NT];
  float sq[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) sq[r] = 0.f;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    o[t] = floatx16{0};
    const int tile = wave + 4 * t;
    if (tile >= tiles_v) continue;
    const int v = tile * 32 + col;
    const bool live = v < V;
    const float weight = pw[col + 1];
    const int steps = (D + 1) / 2;
    int kk0 = 0;
    if (t == 0) {      // what the tokens before the chunk left: first from the rows asked for at the start
#pragma unroll
      for (int kk = 0; kk < PRE; ++kk) {
        const int d = 2 * kk + hi;
        const bool in = d < D;
        if (kk < steps) o[t] = mfma32_f32(in ? qs[col * DP + d] * weight : 0.f, in && live ? kept0[kk] : 0.f, o[t]);
      }
      kk0 = PRE;
    }
#pragma unroll 8
    for (int kk = kk0; kk < steps; ++kk) {
      const int d = 2 * kk + hi;
      const bool in = d < D;
      const float kept = S0[size_t(min(d, D - 1)) * V + min(v, V - 1)];      // always a valid address: the loads do not wait on each other
      o[t] = mfma32_f32(in ? qs[col * DP + d] * weight : 0.f, in && live ? kept : 0.f, o[t]);
    }
#pragma unroll
    for (int kk = 0; kk < C / 2; ++kk) {      // the chunk's own tokens
      const int j = 2 * kk + hi;
      o[t] = mfma32_f32(ps[col * CP + j], live ? vs[j * V + v] : 0.f, o[t]);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) sq[r] = fmaf(o[t][r], o[t][r], sq[r]);      // columns past V hold zeros
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float total = sq[r];
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) total += __shfl_xor(total, off);
    if (col == 0) squares[wave * C + 8 * (r / 4) + 4 * hi + r % 4] = total;
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int tile = wave + 4 * t, v = tile * 32 + col;
    if (tile >= tiles_v || v >= V) continue;
    float g[16];
#pragma unroll
    for (int r = 0; r < 16; ++r)
      g[r] = t == 0 ? gate0[r]
                    : to_float(proj[size_t(first + min(8 * (r / 4) + 4 * hi + r % 4, len - 1)) * a.stride + a.g_off + h * V + v]);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 8 * (r / 4) + 4 * hi + r % 4;
      if (i >= len) continue;
      const float total = ((squares[i] + squares[C + i]) + squares[2 * C + i]) + squares[3 * C + i];
      const float unit = 1.0f / sqrtf(total / float(V) + a.eps);
      out[(size_t(first + i) * a.heads + h) * V + v] = from_float<T>((o[t][r] * unit) * (g[r] * sigmoid(g[r])));
    }
  }
}

static size_t retention_mfma_lds(int dim, int vdim) {
  constexpr int C = kMfmaChunk;
  return sizeof(float) * (size_t(2) * C * (dim + 1) + size_t(C) * vdim + size_t(4) * C * (C + 1) + (C + 1) + 4 * C);
}
static bool retention_mfma_fits(int dim, int vdim) { return vdim <= 256 && retention_mfma_lds(dim, vdim) <= 64 * 1024; }

constexpr int kRetentionLongPortion = 8;      // a step whose longest portion has more tokens takes the chunks

static size_t retention_chunk_lds(int C, int dim, int vdim) {
  return sizeof(float) * (size_t(2) * C * (dim + 1) + size_t(C) * vdim + size_t(C) * (C + 1) + C + 1);
}
// Tokens per chunk: the most whose tiles fit 64 KB of LDS (0: none do).
static int retention_chunk_tokens(int dim, int vdim) {
  if (retention_mfma_fits(dim, vdim)) return kMfmaChunk;      // the matrix cores' kernels
  for (int C : {64, 32, 16})
    if (retention_chunk_lds(C, dim, vdim) <= 64 * 1024) return C;
  return 0;
}

template <typename T, int CV>
static int launch_retention_chunks(hipStream_t s, const RetentionArgs& a, int n_seqs, int max_q_len, int T_tokens, float* scratch) {
  const int C = retention_chunk_tokens(a.dim, a.vdim), chunks = (max_q_len + C - 1) / C, DV = a.dim * a.vdim;
  SP_REQUIRE((long long)n_seqs * chunks < (1 << 30), "sp_retention: too many chunks");
  const dim3 grid(T_tokens / C + n_seqs, a.heads);      // a block per chunk number (chunk_of_block)
  const size_t local_lds = sizeof(float) * (size_t(C) * (a.dim + 1) + size_t(C) * a.vdim);
  if (retention_mfma_fits(a.dim, a.vdim)) {
    const int wide = retention_wide_rows(sizeof(T) == 2 ? kBF16 : kF32, a, C);
    retention_mfma_local_kernel<T><<<grid, 256, local_lds, s>>>(a, scratch, n_seqs, wide);
    retention_chunk_carry_kernel<<<dim3(n_seqs, a.heads, (DV + 255) / 256), 256, 0, s>>>(a, scratch, chunks, C);
    const size_t mfma_lds = retention_mfma_lds(a.dim, a.vdim);
    if (a.vdim <= 128) retention_mfma_apply_kernel<T, 1><<<grid, 256, mfma_lds, s>>>(a, scratch, n_seqs, wide);
    else retention_mfma_apply_kernel<T, 2><<<grid, 256, mfma_lds, s>>>(a, scratch, n_seqs, wide);
    return check_launch("sp_retention (chunks on the matrix cores)");
  }
  retention_chunk_local_kernel<T, CV><<<grid, 256, local_lds, s>>>(a, scratch, n_seqs, C);
  retention_chunk_carry_kernel<<<dim3(n_seqs, a.heads, (DV + 255) / 256), 256, 0, s>>>(a, scratch, chunks, C);
  const size_t lds = retention_chunk_lds(C, a.dim, a.vdim);
  if (C == 64) retention_chunk_apply_kernel<T, 64, CV><<<grid, 256, lds, s>>>(a, scratch, n_seqs);
  else if (C == 32) retention_chunk_apply_kernel<T, 32, CV><<<grid, 256, lds, s>>>(a, scratch, n_seqs);
  else retention_chunk_apply_kernel<T, 16, CV><<<grid, 256, lds, s>>>(a, scratch, n_seqs);
  return check_launch("sp_retention (chunks)");
}

template <typename T>
static int launch_retention_chunks(hipStream_t s, const RetentionArgs& a, int n_seqs, int max_q_len, int T_tokens, float* scratch) {
  const int cv = (a.vdim + 31) / 32;
  if (cv <= 1) return launch_retention_chunks<T, 1>(s, a, n_seqs, max_q_len, T_tokens, scratch);
  if (cv <= 2) return launch_retention_chunks<T, 2>(s, a, n_seqs, max_q_len, T_tokens, scratch);
  if (cv <= 4) return launch_retention_chunks<T, 4>(s, a, n_seqs, max_q_len, T_tokens, scratch);
  return launch_retention_chunks<T, 8>(s, a, n_seqs, max_q_len, T_tokens, scratch);
}

template <typename T>
static int launch_retention(hipStream_t s, const RetentionArgs& a, int n_seqs, int rows, int threads, size_t lds) {
  const dim3 grid(n_seqs, a.heads);
  if (rows <= 8) retention_kernel<T, 8><<<grid, threads, lds, s>>>(a);
  else if (rows <= 16) retention_kernel<T, 16><<<grid, threads, lds, s>>>(a);
  else if (rows <= 32) retention_kernel<T, 32><<<grid, threads, lds, s>>>(a);
  else retention_kernel<T, 64><<<grid, threads, lds, s>>>(a);
  return check_launch("sp_retention");
}

}  // namespace sprout

using namespace sprout;

// float32 numbers of the scratch that a step whose longest portion has max_q_len tokens needs for its scan in chunks
// (0: the scan walks each request in one go and needs none).
extern "C" long long sp_rglru_carry_floats(int width, int n_seqs, int max_q_len, int T) {
  if (max_q_len <= 2 * kScanChunk) return 0;
  return 2LL * (T / kScanChunk + n_seqs) * width;
}

extern "C" int sp_rglru_takes(int width, int blocks, int taps) {
  return width > 0 && blocks > 0 && width % blocks == 0 && taps >= 1 && taps <= 64 && width / blocks <= 2048;
}

extern "C" int sp_rglru(void* stream, int dtype, const void* proj, long long stride, int y_off, int x_off, int width, int blocks,
                        int taps, const void* conv_w, const void* conv_b, const void* wa, const void* ba, const void* wi,
                        const void* bi, const void* lam, const int32_t* q_start, const int32_t* q_len,
                        const int32_t* seq_of_token, const int32_t* state_slots, float* state, float* tail, float* decay,
                        float* drive, void* out, int T, int n_seqs, int max_q_len, float* carry) {
  SP_REQUIRE(sp_rglru_takes(width, blocks, taps), "sp_rglru: no kernel for width=%d blocks=%d taps=%d", width, blocks, taps);
  SP_REQUIRE(T >= 0 && n_seqs >= 0 && y_off >= 0 && x_off >= 0 && stride >= y_off + width && stride >= x_off + width,
             "sp_rglru: rows of %lld numbers do not hold both branches", stride);
  SP_REQUIRE(proj && conv_w && conv_b && wa && ba && wi && bi && lam && q_start && q_len && seq_of_token && state_slots && state &&
             decay && drive && out && (tail || taps == 1), "sp_rglru: null operand");
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_rglru: unsupported dtype %d", dtype);
  if (T == 0 || n_seqs == 0) return 0;
  LruArgs a = {proj, stride, y_off, x_off, width, blocks, taps, conv_w, conv_b, wa, ba, wi, bi, lam, q_start, q_len, seq_of_token,
               state_slots, state, tail, decay, drive, out, T};
  hipStream_t s = (hipStream_t)stream;
  const int n = width / blocks;
  // few tokens: a block each, so that the chip has blocks enough; a tile's convolution outputs and sums stay within 40 KB of LDS
  const int tt = T <= 16 ? 1 : (T <= 64 || n > 512) ? 4 : 16;
  bool wide = false;
  if (dtype == kBF16 && tt <= 4 && n % 8 == 0 && n / 8 <= 256) {      // few tokens: the matrices sixteen bytes at a time
    const int cols = n / 8, few_slices = min(256 / cols, tt == 1 ? 16 : 8);
    const size_t few_lds = (size_t(tt) * n + size_t(few_slices) * tt * 2 * n) * sizeof(float);
    if (few_lds <= 48 * 1024) {
      const dim3 few_grid((T + tt - 1) / tt, blocks);
      if (tt == 1) rglru_gates_few_kernel<1><<<few_grid, 256, few_lds, s>>>(a, few_slices);
      else rglru_gates_few_kernel<4><<<few_grid, 256, few_lds, s>>>(a, few_slices);
      wide = true;
    }
  }
  if (!wide) {
  // many tokens: a thread an output, all of the block's inputs; fewer: the inputs in slices over 256 threads
  const int lanes = n >= 256 ? 256 : tt == 16 ? (n + 63) / 64 * 64 : n > 64 ? 128 : 64, slices = tt == 16 ? 1 : 256 / lanes;
  const int threads = lanes * slices;
  const dim3 grid((T + tt - 1) / tt, blocks);
  const size_t lds = (size_t(tt) * n + size_t(slices - 1) * tt * 2 * lanes) * sizeof(float);
#define SP_GATES(TYPE)                                                                        \
  do {                                                                                        \
    if (tt == 1) rglru_gates_kernel<TYPE, 1><<<grid, threads, lds, s>>>(a, lanes);              \
    else if (tt == 4) rglru_gates_kernel<TYPE, 4><<<grid, threads, lds, s>>>(a, lanes);          \
    else rglru_gates_kernel<TYPE, 16><<<grid, threads, lds, s>>>(a, lanes);                      \
  } while (0)
  if (dtype == kF32) SP_GATES(float);
  else SP_GATES(bf16_t);
#undef SP_GATES
  }
  if (check_launch("sp_rglru (gates)")) return 1;
  const int scan_threads = width >= 256 ? 256 : (width + 63) / 64 * 64;
  const dim3 scan_grid(n_seqs, (width + scan_threads - 1) / scan_threads);
  if (carry && max_q_len > 2 * kScanChunk) {      // a long portion: its chunks side by side
    const int chunks = (max_q_len + kScanChunk - 1) / kScanChunk;
    SP_REQUIRE((long long)n_seqs * chunks < (1 << 30), "sp_rglru: too many chunks");
    float* carry_a = carry;
    float* carry_b = carry + size_t(T / kScanChunk + n_seqs) * width;
    const dim3 chunk_grid(T / kScanChunk + n_seqs, scan_grid.y);      // a block per chunk number (chunk_of_block)
    rglru_chunk_local_kernel<<<chunk_grid, scan_threads, 0, s>>>(a, carry_a, carry_b, n_seqs);
    if (dtype == kF32) {
      rglru_chunk_carry_kernel<float><<<scan_grid, scan_threads, 0, s>>>(a, carry_a, carry_b, chunks);
      rglru_chunk_apply_kernel<float><<<chunk_grid, scan_threads, 0, s>>>(a, carry_b, n_seqs);
    } else {
      rglru_chunk_carry_kernel<bf16_t><<<scan_grid, scan_threads, 0, s>>>(a, carry_a, carry_b, chunks);
      rglru_chunk_apply_kernel<bf16_t><<<chunk_grid, scan_threads, 0, s>>>(a, carry_b, n_seqs);
    }
    return check_launch("sp_rglru (scan in chunks)");
  }
  if (dtype == kF32) rglru_scan_kernel<float><<<scan_grid, scan_threads, 0, s>>>(a);
  else rglru_scan_kernel<bf16_t><<<scan_grid, scan_threads, 0, s>>>(a);
  return check_launch("sp_rglru (scan)");
}

// Whether a head's state fits the registers of one block (a thread: one column, at most 64 rows).
static bool retention_in_registers(int dim, int vdim) {
  if (vdim > 256) return false;
  const int groups = 256 / vdim;
  return (dim + groups - 1) / groups <= 64;
}

extern "C" int sp_retention_takes(int dim, int vdim) {
  return dim > 0 && vdim > 0 && (retention_in_registers(dim, vdim) || size_t(2 * dim + vdim) * sizeof(float) <= 64 * 1024);
}

// float32 numbers of the scratch that a step whose longest portion has max_q_len tokens needs for its walk in chunks
// (0: every request's tokens are walked one after the other and none is needed).
extern "C" long long sp_retention_scratch_floats(int heads, int dim, int vdim, int n_seqs, int max_q_len, int T) {
  if (max_q_len <= kRetentionLongPortion || heads <= 0 || dim <= 0 || vdim <= 0 || vdim > 256) return 0;
  const int C = retention_chunk_tokens(dim, vdim);
  if (C == 0) return 0;
  return ((long long)T / C + n_seqs) * heads * dim * vdim;
}

extern "C" int sp_retention(void* stream, int dtype, const void* proj, long long stride, int q_off, int k_off, int v_off, int g_off,
                            int heads, int dim, int vdim, int rotary_dim, const float* cos_sin, const float* decay, float eps,
                            const int32_t* q_start, const int32_t* q_len, const int32_t* state_slots, float* state, void* out,
                            int T, int n_seqs, int max_q_len, float* scratch) {
  SP_REQUIRE(heads > 0 && sp_retention_takes(dim, vdim), "sp_retention: no kernel for heads of %d and %d numbers", dim, vdim);
  SP_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= dim && (rotary_dim == 0 || cos_sin),
             "sp_retention: %d numbers cannot turn in a head of %d", rotary_dim, dim);
  const long long qk = (long long)heads * dim, vg = (long long)heads * vdim;
  SP_REQUIRE(T >= 0 && n_seqs >= 0 && q_off >= 0 && k_off >= 0 && v_off >= 0 && g_off >= 0 && stride >= q_off + qk &&
             stride >= k_off + qk && stride >= v_off + vg && stride >= g_off + vg,
             "sp_retention: rows of %lld numbers do not hold q, k, v and the gate", stride);
  SP_REQUIRE(proj && decay && q_start && q_len && state_slots && state && out, "sp_retention: null operand");
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_retention: unsupported dtype %d", dtype);
  if (T == 0 || n_seqs == 0) return 0;
  const int groups = vdim <= 256 ? 256 / vdim : 1, rows = (dim + groups - 1) / groups;
  RetentionArgs a = {proj, stride, q_off, k_off, v_off, g_off, heads, dim, vdim, rotary_dim, cos_sin, decay, eps, q_start, q_len,
                     state_slots, state, out, groups};
  if (scratch && sp_retention_scratch_floats(heads, dim, vdim, n_seqs, max_q_len, T) > 0) {      // a long portion: its chunks side by side
    if (dtype == kF32) return launch_retention_chunks<float>((hipStream_t)stream, a, n_seqs, max_q_len, T, scratch);
    return launch_retention_chunks<bf16_t>((hipStream_t)stream, a, n_seqs, max_q_len, T, scratch);
  }
  if (!retention_in_registers(dim, vdim)) {
    const size_t general_lds = size_t(2 * dim + vdim) * sizeof(float);
    const dim3 grid(n_seqs, heads);
    if (dtype == kF32) retention_general_kernel<float><<<grid, 256, general_lds, (hipStream_t)stream>>>(a);
    else retention_general_kernel<bf16_t><<<grid, 256, general_lds, (hipStream_t)stream>>>(a);
    return check_launch("sp_retention (state in memory)");
  }
  const int threads = (groups * vdim + 63) / 64 * 64;
  const size_t lds = size_t(2 * dim + groups * vdim) * sizeof(float);
  if (dtype == kF32) return launch_retention<float>((hipStream_t)stream, a, n_seqs, rows, threads, lds);
  return launch_retention<bf16_t>((hipStream_t)stream, a, n_seqs, rows, threads, lds);
}

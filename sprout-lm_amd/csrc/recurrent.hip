// Mixers that keep a state of fixed size per request instead of cached keys: a gated linear recurrence over channels
// behind a short causal convolution, and retention (linear attention with a fixed decay per head).  Decays, gates,
// step sizes, unit norms and the states themselves are float32 whatever the storage type; only loads of projections
// and weights and the store of the result see it.  A step's tokens lie flat, request after request; q_start / q_len /
// state_slots (one entry per request of the step) say where a request's tokens are and which row of the state tensors
// is its own.  A kernel reads the state as the step before left it and leaves it for the next one.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

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

// A block takes TT tokens of one diagonal block of channels: their convolution outputs wait in LDS, then every thread
// owns output channels of both gates and walks the block's inputs once for all TT tokens.
template <typename T, int TT>
__global__ __launch_bounds__(256) void rglru_gates_kernel(LruArgs a) {
  extern __shared__ float u_s[];      // [TT][n]
  const int n = a.width / a.blocks, b = blockIdx.y, t0 = blockIdx.x * TT, c0 = b * n;
  const T* proj = (const T*)a.proj;
  const int keep = a.taps - 1;
  for (int e = threadIdx.x; e < TT * n; e += blockDim.x) {
    const int tt = e / n, c = c0 + e % n, t = t0 + tt;
    float u = 0.f;
    if (t < a.T) {
      const int s = a.seq_of_token[t];
      const int j = t - a.q_start[s];      // the token's place in its request's share of the step
      const float* tail = a.tail + size_t(a.state_slots[s]) * keep * a.width;
      u = to_float(((const T*)a.conv_b)[c]);
      for (int tap = 0; tap < a.taps; ++tap) {
        const int back = keep - tap;
        const float x = j - back >= 0 ? to_float(proj[size_t(t - back) * a.stride + a.x_off + c])
                                      : tail[size_t(keep + j - back) * a.width + c];
        u = fmaf(to_float(((const T*)a.conv_w)[size_t(c) * a.taps + tap]), x, u);
      }
    }
    u_s[e] = u;
  }
  __syncthreads();
  for (int o = threadIdx.x; o < n; o += blockDim.x) {
    float ra[TT], ri[TT];
    const float bias_a = to_float(((const T*)a.ba)[c0 + o]), bias_i = to_float(((const T*)a.bi)[c0 + o]);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) { ra[tt] = bias_a; ri[tt] = bias_i; }
    const T* wa = (const T*)a.wa + size_t(b) * n * n + o;
    const T* wi = (const T*)a.wi + size_t(b) * n * n + o;
    for (int k = 0; k < n; ++k) {
      const float va = to_float(wa[size_t(k) * n]), vi = to_float(wi[size_t(k) * n]);
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        const float u = u_s[tt * n + k];
        ra[tt] = fmaf(va, u, ra[tt]);
        ri[tt] = fmaf(vi, u, ri[tt]);
      }
    }
    const float rate = 8.0f * softplus(to_float(((const T*)a.lam)[c0 + o]));
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      const int t = t0 + tt;
      if (t >= a.T) break;
      const float log_a = -rate * sigmoid(ra[tt]);
      a.decay[size_t(t) * a.width + c0 + o] = expf(log_a);
      a.drive[size_t(t) * a.width + c0 + o] = sqrtf(-expm1f(2.0f * log_a)) * sigmoid(ri[tt]) * u_s[tt * n + o];
    }
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
      const float value = to_float(row[a.v_off + h * V + v]);
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int d = dr + r * R;
        if (d < D) {
          S[r] = fmaf(gamma, S[r], ks[d] * value);
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
      const float g = to_float(row[a.g_off + h * V + threadIdx.x]);
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

extern "C" int sp_rglru_takes(int width, int blocks, int taps) {
  return width > 0 && blocks > 0 && width % blocks == 0 && taps >= 1 && taps <= 64 && width / blocks <= 2048;
}

extern "C" int sp_rglru(void* stream, int dtype, const void* proj, long long stride, int y_off, int x_off, int width, int blocks,
                        int taps, const void* conv_w, const void* conv_b, const void* wa, const void* ba, const void* wi,
                        const void* bi, const void* lam, const int32_t* q_start, const int32_t* q_len,
                        const int32_t* seq_of_token, const int32_t* state_slots, float* state, float* tail, float* decay,
                        float* drive, void* out, int T, int n_seqs) {
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
  const int tt = T <= 1 ? 1 : (T <= 8 || n > 512) ? 4 : 16;      // a tile's convolution outputs stay within 32 KB of LDS
  const int threads = n >= 256 ? 256 : (n + 63) / 64 * 64;
  const dim3 grid((T + tt - 1) / tt, blocks);
  const size_t lds = size_t(tt) * n * sizeof(float);
#define SP_GATES(TYPE)                                                                        \
  do {                                                                                        \
    if (tt == 1) rglru_gates_kernel<TYPE, 1><<<grid, threads, lds, s>>>(a);                   \
    else if (tt == 4) rglru_gates_kernel<TYPE, 4><<<grid, threads, lds, s>>>(a);              \
    else rglru_gates_kernel<TYPE, 16><<<grid, threads, lds, s>>>(a);                          \
  } while (0)
  if (dtype == kF32) SP_GATES(float);
  else SP_GATES(bf16_t);
#undef SP_GATES
  if (check_launch("sp_rglru (gates)")) return 1;
  const int scan_threads = width >= 256 ? 256 : (width + 63) / 64 * 64;
  const dim3 scan_grid(n_seqs, (width + scan_threads - 1) / scan_threads);
  if (dtype == kF32) rglru_scan_kernel<float><<<scan_grid, scan_threads, 0, s>>>(a);
  else rglru_scan_kernel<bf16_t><<<scan_grid, scan_threads, 0, s>>>(a);
  return check_launch("sp_rglru (scan)");
}

extern "C" int sp_retention_takes(int dim, int vdim) {
  if (dim <= 0 || vdim <= 0 || vdim > 256) return 0;
  const int groups = 256 / vdim;
  return (dim + groups - 1) / groups <= 64;
}

extern "C" int sp_retention(void* stream, int dtype, const void* proj, long long stride, int q_off, int k_off, int v_off, int g_off,
                            int heads, int dim, int vdim, int rotary_dim, const float* cos_sin, const float* decay, float eps,
                            const int32_t* q_start, const int32_t* q_len, const int32_t* state_slots, float* state, void* out,
                            int T, int n_seqs) {
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
  const int groups = 256 / vdim, rows = (dim + groups - 1) / groups;
  RetentionArgs a = {proj, stride, q_off, k_off, v_off, g_off, heads, dim, vdim, rotary_dim, cos_sin, decay, eps, q_start, q_len,
                     state_slots, state, out, groups};
  const int threads = (groups * vdim + 63) / 64 * 64;
  const size_t lds = size_t(2 * dim + groups * vdim) * sizeof(float);
  if (dtype == kF32) return launch_retention<float>((hipStream_t)stream, a, n_seqs, rows, threads, lds);
  return launch_retention<bf16_t>((hipStream_t)stream, a, n_seqs, rows, threads, lds);
}

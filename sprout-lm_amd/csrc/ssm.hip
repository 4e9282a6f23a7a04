// Short causal convolutions with per-request state, the scans of two state-space mixers (the state-space-duality form
// with one decay per head and token, and the selective scan with one decay per channel, state and token), and what
// attention with weights mixed between heads after the softmax needs around the attention kernels.  Step sizes, decays,
// their exponentials, the states and all norms are float32 whatever the storage type; only loads of projections and
// weights and the stores of results see it.  A step's tokens lie flat, request after request; q_start / q_len /
// state_slots (one entry per request of the step) say where a request's tokens are and which row of the state tensors is
// its own.  A kernel reads the state as the step before left it and leaves it for the next one, so a portion of a prompt
// and a single decoded token are the same call.
#include <type_traits>

#include "common.h"
#include "sprout_hip.h"

namespace sprout {

__device__ __forceinline__ float softplus_of(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float silu_of(float z) { return z / (1.0f + expf(-z)); }

// ------------------------------------------------------------------------------------------------ short convolution
struct ConvArgs {
  const void* x;
  long long x_stride;
  int x_off, channels, taps;
  const void* w;
  const void* bias;
  int act, add_input;
  void* out;
  long long out_stride;
  int out_off;
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* seq_of_token;
  const int32_t* state_slots;
  float* state;
};

// A thread a (token, channel): the taps in their order, inputs before the request's share of the step from its state rows.
// The weights lie tap-major, [taps][channels].
template <typename T, typename TW>
__global__ __launch_bounds__(256) void short_conv_kernel(ConvArgs a) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.channels) return;
  const int s = a.seq_of_token[t];
  const int j = t - a.q_start[s], keep = a.taps - 1;
  const T* x = (const T*)a.x + a.x_off + c;
  const TW* w = (const TW*)a.w + c;
  const float* rows = keep ? a.state + size_t(a.state_slots[s]) * keep * a.channels + c : nullptr;
  float acc = a.bias ? to_float(((const TW*)a.bias)[c]) : 0.f;
  for (int tap = 0; tap < a.taps; ++tap) {
    const int back = keep - tap;
    const float v = j - back >= 0 ? to_float(x[size_t(t - back) * a.x_stride]) : rows[size_t(keep + j - back) * a.channels];
    acc = fmaf(to_float(w[size_t(tap) * a.channels]), v, acc);
  }
  if (a.act == 1) acc = silu_of(acc);
  if (a.add_input) acc += to_float(x[size_t(t) * a.x_stride]);
  ((T*)a.out)[size_t(t) * a.out_stride + a.out_off + c] = from_float<T>(acc);
}

__device__ __forceinline__ void unpack8(const uint4& raw, float (&v)[8]) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// The same for bfloat16 rows and weights whose channels come in whole eights at 16 bytes: a thread eight neighbouring
// channels of a token, sixteen bytes a load.  The sums run in the taps' order, as above.
__global__ __launch_bounds__(256) void short_conv_eights_kernel(ConvArgs a) {
  const int t = blockIdx.x, c = 8 * (blockIdx.y * 256 + threadIdx.x);
  if (c >= a.channels) return;
  const int s = a.seq_of_token[t];
  const int j = t - a.q_start[s], keep = a.taps - 1;
  const bf16_t* x = (const bf16_t*)a.x + a.x_off + c;
  const bf16_t* w = (const bf16_t*)a.w + c;
  const float* rows = keep ? a.state + size_t(a.state_slots[s]) * keep * a.channels + c : nullptr;
  float acc[8], v[8], wt[8];
  if (a.bias) unpack8(*reinterpret_cast<const uint4*>((const bf16_t*)a.bias + c), acc);
  else {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  }
  for (int tap = 0; tap < a.taps; ++tap) {
    const int back = keep - tap;
    if (j - back >= 0) {
      unpack8(*reinterpret_cast<const uint4*>(x + size_t(t - back) * a.x_stride), v);
    } else {
      const float4* r = reinterpret_cast<const float4*>(rows + size_t(keep + j - back) * a.channels);
      const float4 lo = r[0], hi = r[1];
      v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    }
    unpack8(*reinterpret_cast<const uint4*>(w + size_t(tap) * a.channels), wt);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = fmaf(wt[i], v[i], acc[i]);
  }
  if (a.act == 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = silu_of(acc[i]);
  }
  if (a.add_input) {
    unpack8(*reinterpret_cast<const uint4*>(x + size_t(t) * a.x_stride), v);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += v[i];
  }
  uint4 packed;
  packed.x = uint32_t(f32_to_bf16_bits(acc[0])) | uint32_t(f32_to_bf16_bits(acc[1])) << 16;
  packed.y = uint32_t(f32_to_bf16_bits(acc[2])) | uint32_t(f32_to_bf16_bits(acc[3])) << 16;
  packed.z = uint32_t(f32_to_bf16_bits(acc[4])) | uint32_t(f32_to_bf16_bits(acc[5])) << 16;
  packed.w = uint32_t(f32_to_bf16_bits(acc[6])) | uint32_t(f32_to_bf16_bits(acc[7])) << 16;
  *reinterpret_cast<uint4*>((bf16_t*)a.out + size_t(t) * a.out_stride + a.out_off + c) = packed;
}

// A step in which every request brings one token: the thread that owns a (request, channel) convolves and moves the
// state rows up itself, in one launch.  The sum runs in the taps' order, as above.
template <typename T, typename TW>
__global__ __launch_bounds__(256) void short_conv_single_kernel(ConvArgs a) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.channels) return;
  const int s = a.seq_of_token[t], keep = a.taps - 1;
  const float x = to_float(((const T*)a.x)[size_t(t) * a.x_stride + a.x_off + c]);
  const TW* w = (const TW*)a.w + c;
  float* rows = a.state + size_t(a.state_slots[s]) * keep * a.channels + c;
  float acc = a.bias ? to_float(((const TW*)a.bias)[c]) : 0.f;
  for (int tap = 0; tap < keep; ++tap) {
    const float v = rows[size_t(tap) * a.channels];
    acc = fmaf(to_float(w[size_t(tap) * a.channels]), v, acc);
    if (tap > 0) rows[size_t(tap - 1) * a.channels] = v;
  }
  rows[size_t(keep - 1) * a.channels] = x;
  acc = fmaf(to_float(w[size_t(keep) * a.channels]), x, acc);
  if (a.act == 1) acc = silu_of(acc);
  if (a.add_input) acc += x;
  ((T*)a.out)[size_t(t) * a.out_stride + a.out_off + c] = from_float<T>(acc);
}

// A thread a (request, channel): the state rows become the last taps - 1 inputs, older ones moved up from the rows
// themselves where the request brought fewer tokens than that.  Rows are written oldest first and read at or behind
// the row being written, by the one thread that owns the channel.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_state_kernel(ConvArgs a) {
  const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.channels) return;
  const int L = a.q_len[s], keep = a.taps - 1;
  if (L <= 0) return;
  const T* x = (const T*)a.x + size_t(a.q_start[s]) * a.x_stride + a.x_off + c;
  float* rows = a.state + size_t(a.state_slots[s]) * keep * a.channels + c;
  for (int j = 0; j < keep; ++j) {
    const int src = L - keep + j;
    rows[size_t(j) * a.channels] = src >= 0 ? to_float(x[size_t(src) * a.x_stride]) : rows[size_t(j + L) * a.channels];
  }
}

// ------------------------------------------------------------------------------------------------ small kernels
template <typename TW, typename TO>
__global__ __launch_bounds__(256) void group_rmsnorm_kernel(const float* __restrict__ x, const TW* __restrict__ w, float eps,
                                                            TO* __restrict__ out, int parts, int size) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  const int part = int(row % parts);
  const float* xr = x + row * size;
  float ss = 0.f;
  for (int i = threadIdx.x; i < size; i += 256) ss = fmaf(xr[i], xr[i], ss);
  const float r = 1.0f / sqrtf(block_sum(ss, scratch) / float(size) + eps);
  for (int i = threadIdx.x; i < size; i += 256)
    out[row * size + i] = from_float<TO>(xr[i] * r * to_float(w[size_t(part) * size + i]));
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_erf_kernel(T* __restrict__ x, long long n) {
  for (long long i = blockIdx.x * 256ll + threadIdx.x; i < n; i += 256ll * gridDim.x) {
    const float v = to_float(x[i]);
    x[i] = from_float<T>(0.5f * v * (1.0f + erff(v * 0.70710678118654752f)));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void scale_rows_kernel(const T* __restrict__ x, const float* __restrict__ weights, int top,
                                                         T* __restrict__ out, int H) {
  const size_t p = blockIdx.x;
  const float w = weights[p];
  const T* src = x + (p / top) * H;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < H; i += 256 * gridDim.y) out[p * H + i] = from_float<T>(to_float(src[i]) * w);
}

// ------------------------------------------------------------------------------------------------ state-space duality scan
struct SsdArgs {
  const void* proj;
  long long proj_stride;
  int z_off, dt_off;
  const void* xbc;
  long long xbc_stride;
  int heads, vdim, state_size, groups;
  const float* dt_bias;
  const float* a_log;
  const float* skip;
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* state_slots;
  float* state;
  float* out;
  int chunk, chunks;           // tokens a chunk, chunks a request (the longest portion's), where portions are walked in chunks
  float* scratch;              // [requests * chunks, heads, state, vdim]; by_column: [requests * chunks, heads, vdim, state]
  float* step_sums;            // [requests * chunks, heads]
  int by_column;               // the scratch holds a column's state rows together (what a lane of the LDS kernels owns)
};

// A block per request and 32 columns of the heads' values; a column's state rows are shared out over 8 neighbouring lanes
// (lane rg holds rows rg, rg + 8, ...: KPT of them), so a token's output is a sum over those lanes alone and the walk along
// the request's tokens needs no barrier.  Columns are independent of each other: S[:, p] takes B and u_p only.
//
// Long portions are walked in chunks of `chunk` tokens side by side, in three passes over the same recurrence:
//   MODE 1  every chunk from a state of zeros: what it adds, U_c, and the sum of its step sizes (the chunk's decay is
//           exp(-rate * sum)) go to the scratch;
//   carry   per state element the chunks in turn, S <- decay_c S + U_c, leaving in U_c's place the state chunk c starts
//           from, and in the request's state rows the state after its last token;
//   MODE 2  every chunk again, from the state it starts from, with the outputs.
// MODE 0 walks a request's tokens in one go (short portions, single tokens).  blockIdx.y: the request (MODE 0), or
// request * chunks_per_request + chunk.
// CP: the neighbouring columns a lane holds (2 where a head's values are an even number: a row's numbers are then read
// and written eight bytes a lane, 64 bytes a run, and B and C are fetched once for both).
template <typename T, int KPT, int MODE, int CP>
__global__ __launch_bounds__(256) void ssd_scan_kernel(SsdArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rg = lane & 7, pc = lane >> 3;
  const int inner = a.heads * a.vdim, N = a.state_size;
  const int s = MODE == 0 ? blockIdx.y : blockIdx.y / a.chunks;
  const int ci = MODE == 0 ? 0 : blockIdx.y % a.chunks;
  int col = (blockIdx.x * 32 + wave * 8 + pc) * CP;
  const bool live = col < inner;
  if (!live) col = inner - CP;      // the lane stays for its neighbours' sums and stores nothing
  const int n = col / a.vdim, p = col % a.vdim, g = n / (a.heads / a.groups);
  int q0 = a.q_start[s], L = a.q_len[s];
  if (MODE != 0) {
    q0 += ci * a.chunk;
    L = min(a.chunk, L - ci * a.chunk);
  }
  if (L <= 0) return;
  // the state rows of these columns: the request's own (MODE 0), or the chunk's place in the scratch
  float* S = MODE == 0 ? a.state + ((size_t(a.state_slots[s]) * a.heads + n) * N) * a.vdim + p
                       : a.scratch + ((size_t(blockIdx.y) * a.heads + n) * N) * a.vdim + p;
  float st[KPT][CP];
#pragma unroll
  for (int k = 0; k < KPT; ++k) {
    const int r = rg + 8 * k;
#pragma unroll
    for (int j = 0; j < CP; ++j) st[k][j] = 0.f;
    if (MODE != 1 && r < N) {
      if (CP == 2) {
        const float2 v = *reinterpret_cast<const float2*>(S + size_t(r) * a.vdim);
        st[k][0] = v.x;
        st[k][CP - 1] = v.y;
      } else {
        st[k][0] = S[size_t(r) * a.vdim];
      }
    }
  }
  const float rate = expf(a.a_log[n]), bias = a.dt_bias[n], skip = a.skip[n];
  const T* proj = (const T*)a.proj;
  const T* xbc = (const T*)a.xbc;
  const int b_off = inner + g * N, c_off = inner + a.groups * N + g * N;
  float steps = 0.f;
  for (int t = q0; t < q0 + L; ++t) {
    const T* pr = proj + size_t(t) * a.proj_stride;
    const T* xr = xbc + size_t(t) * a.xbc_stride;
    const float d = softplus_of(to_float(pr[a.dt_off + n]) + bias);
    const float decay = expf(-rate * d);
    float u[CP], du[CP], y[CP];
#pragma unroll
    for (int j = 0; j < CP; ++j) {
      u[j] = to_float(xr[col + j]);
      du[j] = d * u[j];
      y[j] = 0.f;
    }
    steps += d;
#pragma unroll
    for (int k = 0; k < KPT; ++k) {
      const int r = rg + 8 * k;
      if (r < N) {
        const float b = to_float(xr[b_off + r]);
        const float c = MODE != 1 ? to_float(xr[c_off + r]) : 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j) {
          st[k][j] = fmaf(decay, st[k][j], du[j] * b);
          if (MODE != 1) y[j] = fmaf(st[k][j], c, y[j]);
        }
      }
    }
    if (MODE != 1) {
#pragma unroll
      for (int j = 0; j < CP; ++j) {
        y[j] += __shfl_xor(y[j], 1, 64);
        y[j] += __shfl_xor(y[j], 2, 64);
        y[j] += __shfl_xor(y[j], 4, 64);
      }
      if (rg == 0 && live) {
#pragma unroll
        for (int j = 0; j < CP; ++j)
          a.out[size_t(t) * inner + col + j] = fmaf(skip, u[j], y[j]) * silu_of(to_float(pr[a.z_off + col + j]));
      }
    }
  }
  if (MODE == 2) return;
  if (live) {
#pragma unroll
    for (int k = 0; k < KPT; ++k) {
      const int r = rg + 8 * k;
      if (r < N) {
        if (CP == 2) *reinterpret_cast<float2*>(S + size_t(r) * a.vdim) = make_float2(st[k][0], st[k][CP - 1]);
        else S[size_t(r) * a.vdim] = st[k][0];
      }
    }
    if (MODE == 1 && p == 0 && rg == 0) a.step_sums[size_t(blockIdx.y) * a.heads + n] = steps;
  }
}

// K numbers of a row in LDS as floats, eight or sixteen bytes at a time (the row starts at a multiple of 16 bytes).
template <int K>
__device__ __forceinline__ void lds_row(const bf16_t* p, float (&v)[K]) {
#pragma unroll
  for (int i = 0; i < K; i += 4) {
    const uint2 w = *reinterpret_cast<const uint2*>(p + i);
    v[i] = __uint_as_float(w.x << 16);
    v[i + 1] = __uint_as_float(w.x & 0xffff0000u);
    v[i + 2] = __uint_as_float(w.y << 16);
    v[i + 3] = __uint_as_float(w.y & 0xffff0000u);
  }
}
template <int K>
__device__ __forceinline__ void lds_row(const float* p, float (&v)[K]) {
#pragma unroll
  for (int i = 0; i < K; i += 4) {
    const float4 w = *reinterpret_cast<const float4*>(p + i);
    v[i] = w.x; v[i + 1] = w.y; v[i + 2] = w.z; v[i + 3] = w.w;
  }
}

constexpr int kScanChunk = 64;      // tokens of a chunk where long portions are walked in chunks

// MODE 1 and MODE 2 of the scan above for heads whose values come in whole 32s, so that a block's 32 columns lie in one
// head: what the chunk's tokens share (B and C as floats, the step sizes and decays, computed once per token and not once
// per lane) and the block's columns of u and z are brought into LDS first, rows 8 * KPT wide with zeros behind the
// state's rows, and the walk along the tokens reads LDS alone; lane rg holds the KPT neighbouring rows from rg * KPT on.
// The kernels are bound by their vector instructions (a multiply-add per state element and token is what the design
// asks for), so MODE 1 does not walk the recurrence: what a chunk adds to a state of zeros is
// sum_t w_t u_t B_t with w_t = d_t exp(-rate * (the step sizes after t)), one multiply-add per element and token.
template <typename T, int KPT, int MODE>
__global__ __launch_bounds__(256) void ssd_chunk_kernel(SsdArgs a) {
  constexpr int L = kScanChunk, NP = 8 * KPT;
  extern __shared__ float4 lds_raw[];
  // B and C in LDS: floats for MODE 1, whose one multiply-add per element leaves no room for conversions; as they are
  // stored for MODE 2, which waits for LDS more than for its arithmetic when the rows are twice as long
  using TL = typename std::conditional<MODE == 1, float, T>::type;
  float* Ds = reinterpret_cast<float*>(lds_raw);      // [L] step sizes, [L] decays (MODE 2) or weights w_t (MODE 1)
  TL* Bs = reinterpret_cast<TL*>(Ds + 2 * L);         // [L][NP]
  TL* Cs = Bs + L * NP;                               // [L][NP], MODE 2 only
  T* Us = reinterpret_cast<T*>(MODE == 2 ? Cs + L * NP : Cs);      // [L][32]
  T* Zs = Us + L * 32;                                // [L][32], MODE 2 only
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rg = lane & 7, pc = lane >> 3;
  const int inner = a.heads * a.vdim, N = a.state_size;
  const int s = blockIdx.y / a.chunks, ci = blockIdx.y % a.chunks;
  const int col0 = blockIdx.x * 32, mine = wave * 8 + pc, col = col0 + mine;
  const int n = col0 / a.vdim, p = col % a.vdim, g = n / (a.heads / a.groups);
  const int q0 = a.q_start[s] + ci * L, len = min(L, a.q_len[s] - ci * L);
  if (len <= 0) return;
  const float rate = expf(a.a_log[n]), bias = a.dt_bias[n], skip = a.skip[n];
  const T* proj = (const T*)a.proj;
  const T* xbc = (const T*)a.xbc;
  const int b_off = inner + g * N, c_off = inner + a.groups * N + g * N;
  if (sizeof(T) == 2 && N == NP && (a.xbc_stride & 7) == 0 && (b_off & 7) == 0 && (c_off & 7) == 0 &&
      (reinterpret_cast<uintptr_t>(xbc) & 15) == 0) {
    // rows of whole eights at 16 bytes: eight numbers a load
    for (int i = threadIdx.x; i < len * (NP / 8); i += 256) {
      const int tt = i / (NP / 8), r = 8 * (i % (NP / 8));
      const T* xr = xbc + size_t(q0 + tt) * a.xbc_stride;
      if (MODE == 1) {
        float v[8];
        unpack8(*reinterpret_cast<const uint4*>(xr + b_off + r), v);
        float4* to = reinterpret_cast<float4*>(Bs + tt * NP + r);
        to[0] = make_float4(v[0], v[1], v[2], v[3]);
        to[1] = make_float4(v[4], v[5], v[6], v[7]);
      } else {
        *reinterpret_cast<uint4*>(Bs + tt * NP + r) = *reinterpret_cast<const uint4*>(xr + b_off + r);
        *reinterpret_cast<uint4*>(Cs + tt * NP + r) = *reinterpret_cast<const uint4*>(xr + c_off + r);
      }
    }
  } else {
    for (int i = threadIdx.x; i < len * NP; i += 256) {
      const int tt = i / NP, r = i % NP;
      const T* xr = xbc + size_t(q0 + tt) * a.xbc_stride;
      Bs[i] = from_float<TL>(r < N ? to_float(xr[b_off + r]) : 0.f);
      if (MODE == 2) Cs[i] = from_float<TL>(r < N ? to_float(xr[c_off + r]) : 0.f);
    }
  }
  for (int i = threadIdx.x; i < len * 32; i += 256) {
    const int tt = i >> 5, j = i & 31;
    Us[i] = xbc[size_t(q0 + tt) * a.xbc_stride + col0 + j];
    if (MODE == 2) Zs[i] = proj[size_t(q0 + tt) * a.proj_stride + a.z_off + col0 + j];
  }
  if (int(threadIdx.x) < len) {
    const float d = softplus_of(to_float(proj[size_t(q0 + threadIdx.x) * a.proj_stride + a.dt_off + n]) + bias);
    Ds[threadIdx.x] = d;
    if (MODE == 2) Ds[L + threadIdx.x] = expf(-rate * d);
  }
  // a column's state rows lie together in the scratch: a lane's KPT rows are one run of memory
  float* S = a.scratch + ((size_t(blockIdx.y) * a.heads + n) * a.vdim + p) * N + rg * KPT;
  float st[KPT];
#pragma unroll
  for (int k = 0; k < KPT; ++k) st[k] = 0.f;
  if (MODE == 2) {
    if (N == NP) {
#pragma unroll
      for (int k = 0; k < KPT; k += 4) {
        const float4 v = *reinterpret_cast<const float4*>(S + k);
        st[k] = v.x; st[k + 1] = v.y; st[k + 2] = v.z; st[k + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int k = 0; k < KPT; ++k)
        if (rg * KPT + k < N) st[k] = S[k];
    }
  }
  __syncthreads();
  if (MODE == 1) {
    // w_t = d_t exp(-rate * (d_(t+1) + ... + d_(len-1))): every token's weight in the chunk's last state
    if (int(threadIdx.x) < len) {
      float after = 0.f;
      for (int t2 = len - 1; t2 > int(threadIdx.x); --t2) after += Ds[t2];
      Ds[L + threadIdx.x] = Ds[threadIdx.x] * expf(-rate * after);
      if (threadIdx.x == 0 && blockIdx.x * 32 == n * a.vdim) a.step_sums[size_t(blockIdx.y) * a.heads + n] = after + Ds[0];
    }
    __syncthreads();
    for (int tt = 0; tt < len; ++tt) {
      const float wu = Ds[L + tt] * to_float(Us[tt * 32 + mine]);
      float b[KPT];
      lds_row<KPT>(Bs + tt * NP + rg * KPT, b);
#pragma unroll
      for (int k = 0; k < KPT; ++k) st[k] = fmaf(wu, b[k], st[k]);
    }
  } else {
    // eight tokens at a time: a lane's share of each token's output, then the eight lanes of a column exchange them so that
    // lane rg ends with the whole sum of token rg (three exchanges of 4, 2 and 1 numbers instead of three of 8), and
    // every lane finishes and stores one token's output
    for (int t0 = 0; t0 < len; t0 += 8) {
      float part[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int tt = min(t0 + i, len - 1);
        const bool real = t0 + i < len;
        const float d = Ds[tt], decay = real ? Ds[L + tt] : 1.f;
        const float du = real ? d * to_float(Us[tt * 32 + mine]) : 0.f;
        float b[KPT], c[KPT];
        lds_row<KPT>(Bs + tt * NP + rg * KPT, b);
        lds_row<KPT>(Cs + tt * NP + rg * KPT, c);
        float y = 0.f;
#pragma unroll
        for (int k = 0; k < KPT; ++k) {
          st[k] = fmaf(decay, st[k], du * b[k]);
          y = fmaf(st[k], c[k], y);
        }
        part[i] = y;
      }
      float four[4], two[2];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float keep = (rg & 4) ? part[i + 4] : part[i], give = (rg & 4) ? part[i] : part[i + 4];
        four[i] = keep + __shfl_xor(give, 4, 64);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const float keep = (rg & 2) ? four[i + 2] : four[i], give = (rg & 2) ? four[i] : four[i + 2];
        two[i] = keep + __shfl_xor(give, 2, 64);
      }
      const float keep = (rg & 1) ? two[1] : two[0], give = (rg & 1) ? two[0] : two[1];
      const float y = keep + __shfl_xor(give, 1, 64);
      const int tt = t0 + rg;
      if (tt < len)
        a.out[size_t(q0 + tt) * inner + col] = fmaf(skip, to_float(Us[tt * 32 + mine]), y) * silu_of(to_float(Zs[tt * 32 + mine]));
    }
    return;
  }
  if (N == NP) {
#pragma unroll
    for (int k = 0; k < KPT; k += 4) *reinterpret_cast<float4*>(S + k) = make_float4(st[k], st[k + 1], st[k + 2], st[k + 3]);
  } else {
#pragma unroll
    for (int k = 0; k < KPT; ++k)
      if (rg * KPT + k < N) S[k] = st[k];
  }
}

// A thread a state element of a request: the chunks in turn.
__global__ __launch_bounds__(256) void ssd_carry_kernel(SsdArgs a) {
  const int s = blockIdx.y;
  const size_t per_head = size_t(a.state_size) * a.vdim, per_request = per_head * a.heads;
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e >= per_request) return;
  const int L = a.q_len[s];
  if (L <= 0) return;
  const int n = int(e / per_head), used = (L + a.chunk - 1) / a.chunk;
  const float rate = expf(a.a_log[n]);
  // e counts the scratch's elements; the request's own rows lie [head][state][vdim]
  size_t own = e;
  if (a.by_column) {
    const size_t in_head = e % per_head;
    own = size_t(n) * per_head + (in_head % a.state_size) * a.vdim + in_head / a.state_size;
  }
  float* mine = a.state + size_t(a.state_slots[s]) * per_request + own;
  float S = *mine;
  for (int c = 0; c < used; ++c) {
    const size_t number = size_t(s) * a.chunks + c;
    float* at = a.scratch + number * per_request + e;
    const float added = *at;
    *at = S;
    S = fmaf(expf(-rate * a.step_sums[number * a.heads + n]), S, added);
  }
  *mine = S;
}

// ------------------------------------------------------------------------------------------------ selective scan
struct SelArgs {
  const void* u;
  long long u_stride;
  int u_off;
  const void* z;
  long long z_stride;
  int z_off;
  const float* dt;
  const void* bc;
  long long bc_stride;
  int bc_off, inner, state_size;
  const float* a;
  const float* skip;
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* state_slots;
  float* state;
  void* out;
  int chunk, chunks;
  float* scratch;              // [requests * chunks, inner, state]
  float* step_sums;            // [requests * chunks, inner]
};

// A block per request and 64 channels; a channel's states are shared out over 4 neighbouring lanes (lane ng holds states ng,
// ng + 4, ...: KPT of them).  MODE as for the duality scan: long portions in chunks side by side, three passes; a chunk's
// decay of state (c, n) is exp(rate[c, n] * the sum of the channel's step sizes).
template <typename T, int KPT, int MODE>
__global__ __launch_bounds__(256) void selective_scan_kernel(SelArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ng = lane & 3, cc = lane >> 2;
  const int N = a.state_size;
  const int s = MODE == 0 ? blockIdx.y : blockIdx.y / a.chunks;
  const int ci = MODE == 0 ? 0 : blockIdx.y % a.chunks;
  int c = blockIdx.x * 64 + wave * 16 + cc;
  const bool live = c < a.inner;
  if (!live) c = a.inner - 1;
  int q0 = a.q_start[s], L = a.q_len[s];
  if (MODE != 0) {
    q0 += ci * a.chunk;
    L = min(a.chunk, L - ci * a.chunk);
  }
  if (L <= 0) return;
  float* S = MODE == 0 ? a.state + (size_t(a.state_slots[s]) * a.inner + c) * N
                       : a.scratch + (size_t(blockIdx.y) * a.inner + c) * N;
  float st[KPT], ak[KPT];
#pragma unroll
  for (int k = 0; k < KPT; ++k) {
    const int n = ng + 4 * k;
    st[k] = (MODE != 1 && n < N) ? S[n] : 0.f;
    ak[k] = n < N ? a.a[size_t(c) * N + n] : 0.f;
  }
  const float skip = a.skip[c];
  const T* up = (const T*)a.u + a.u_off + c;
  const T* zp = (const T*)a.z + a.z_off + c;
  const T* bc = (const T*)a.bc + a.bc_off;
  float steps = 0.f;
  for (int t = q0; t < q0 + L; ++t) {
    const float d = softplus_of(a.dt[size_t(t) * a.inner + c]);
    const float u = to_float(up[size_t(t) * a.u_stride]);
    const T* row = bc + size_t(t) * a.bc_stride;
    const float du = d * u;
    steps += d;
    float y = 0.f;
#pragma unroll
    for (int k = 0; k < KPT; ++k) {
      const int n = ng + 4 * k;
      if (n < N) {
        st[k] = fmaf(expf(d * ak[k]), st[k], du * to_float(row[n]));
        if (MODE != 1) y = fmaf(st[k], to_float(row[N + n]), y);
      }
    }
    if (MODE != 1) {
      y += __shfl_xor(y, 1, 64);
      y += __shfl_xor(y, 2, 64);
      if (ng == 0 && live)
        ((T*)a.out)[size_t(t) * a.inner + c] = from_float<T>(fmaf(skip, u, y) * silu_of(to_float(zp[size_t(t) * a.z_stride])));
    }
  }
  if (MODE == 2) return;
  if (live) {
#pragma unroll
    for (int k = 0; k < KPT; ++k) {
      const int n = ng + 4 * k;
      if (n < N) S[n] = st[k];
    }
    if (MODE == 1 && ng == 0) a.step_sums[size_t(blockIdx.y) * a.inner + c] = steps;
  }
}

// MODE 1 and MODE 2 of the scan above with the chunk in LDS: the step sizes (their softplus taken once per token and
// channel, not once per lane), the block's columns of u and z, and B and C as floats in rows 4 * KPT wide with zeros behind
// the state's numbers; lane ng holds the KPT neighbouring states from ng * KPT on.
template <typename T, int KPT, int MODE>
__global__ __launch_bounds__(256) void selective_chunk_kernel(SelArgs a) {
  constexpr int L = kScanChunk, NP = 4 * KPT;
  extern __shared__ float4 lds_raw[];
  float* Ds = reinterpret_cast<float*>(lds_raw);      // [L][64]
  float* BCs = Ds + L * 64;                           // [L][2][NP]
  T* Us = reinterpret_cast<T*>(BCs + L * 2 * NP);     // [L][64]
  T* Zs = Us + L * 64;                                // [L][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ng = lane & 3, cc = lane >> 2, mine = wave * 16 + cc;
  const int N = a.state_size;
  const int s = blockIdx.y / a.chunks, ci = blockIdx.y % a.chunks;
  const int c0 = blockIdx.x * 64;
  int c = c0 + mine;
  const bool live = c < a.inner;
  if (!live) c = a.inner - 1;
  const int q0 = a.q_start[s] + ci * L, len = min(L, a.q_len[s] - ci * L);
  if (len <= 0) return;
  for (int i = threadIdx.x; i < len * 64; i += 256) {
    const int tt = i >> 6, ch = min(c0 + (i & 63), a.inner - 1);
    const size_t t = size_t(q0 + tt);
    Ds[i] = softplus_of(a.dt[t * a.inner + ch]);
    Us[i] = ((const T*)a.u)[t * a.u_stride + a.u_off + ch];
    if (MODE == 2) Zs[i] = ((const T*)a.z)[t * a.z_stride + a.z_off + ch];
  }
  for (int i = threadIdx.x; i < len * 2 * NP; i += 256) {
    const int tt = i / (2 * NP), r = i % (2 * NP), which = r / NP, nn = r % NP;
    BCs[i] = nn < N ? to_float(((const T*)a.bc)[size_t(q0 + tt) * a.bc_stride + a.bc_off + which * N + nn]) : 0.f;
  }
  float* S = a.scratch + (size_t(blockIdx.y) * a.inner + c) * N;
  float st[KPT], ak[KPT];
#pragma unroll
  for (int k = 0; k < KPT; ++k) {
    const int n = ng * KPT + k;
    st[k] = (MODE == 2 && n < N) ? S[n] : 0.f;
    ak[k] = n < N ? a.a[size_t(c) * N + n] * 1.4426950408889634f : 0.f;      // in units of log 2: the decay is one exp2
  }
  const float skip = a.skip[c];
  __syncthreads();
  float steps = 0.f;
  if (MODE == 1) {
    for (int tt = 0; tt < len; ++tt) {
      const float d = Ds[tt * 64 + mine];
      const float du = d * to_float(Us[tt * 64 + mine]);
      steps += d;
      float b[KPT];
      lds_row<KPT>(BCs + tt * 2 * NP + ng * KPT, b);
#pragma unroll
      for (int k = 0; k < KPT; ++k) st[k] = fmaf(__builtin_amdgcn_exp2f(d * ak[k]), st[k], du * b[k]);
    }
  } else {
    // four tokens at a time: the four lanes of a channel exchange their shares so that lane ng ends with the whole sum
    // of token ng, and every lane finishes and stores one token's output
    for (int t0 = 0; t0 < len; t0 += 4) {
      float part[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tt = min(t0 + i, len - 1);
        const bool real = t0 + i < len;
        const float d = real ? Ds[tt * 64 + mine] : 0.f;      // a step size of 0: the state stays as it is
        const float du = d * to_float(Us[tt * 64 + mine]);
        float b[KPT], cv[KPT];
        lds_row<KPT>(BCs + tt * 2 * NP + ng * KPT, b);
        lds_row<KPT>(BCs + tt * 2 * NP + NP + ng * KPT, cv);
        float y = 0.f;
#pragma unroll
        for (int k = 0; k < KPT; ++k) {
          st[k] = fmaf(__builtin_amdgcn_exp2f(d * ak[k]), st[k], du * b[k]);
          y = fmaf(st[k], cv[k], y);
        }
        part[i] = y;
      }
      float two[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const float keep = (ng & 2) ? part[i + 2] : part[i], give = (ng & 2) ? part[i] : part[i + 2];
        two[i] = keep + __shfl_xor(give, 2, 64);
      }
      const float keep = (ng & 1) ? two[1] : two[0], give = (ng & 1) ? two[0] : two[1];
      const float y = keep + __shfl_xor(give, 1, 64);
      const int tt = t0 + ng;
      if (tt < len && live)
        ((T*)a.out)[size_t(q0 + tt) * a.inner + c] =
            from_float<T>(fmaf(skip, to_float(Us[tt * 64 + mine]), y) * silu_of(to_float(Zs[tt * 64 + mine])));
    }
  }
  if (MODE == 2 || !live) return;
#pragma unroll
  for (int k = 0; k < KPT; ++k) {
    const int n = ng * KPT + k;
    if (n < N) S[n] = st[k];
  }
  if (ng == 0) a.step_sums[size_t(blockIdx.y) * a.inner + c] = steps;
}

__global__ __launch_bounds__(256) void selective_carry_kernel(SelArgs a) {
  const int s = blockIdx.y;
  const size_t per_request = size_t(a.inner) * a.state_size;
  const size_t e = size_t(blockIdx.x) * 256 + threadIdx.x;
  if (e >= per_request) return;
  const int L = a.q_len[s];
  if (L <= 0) return;
  const int c = int(e / a.state_size), used = (L + a.chunk - 1) / a.chunk;
  const float rate = a.a[e];
  float* mine = a.state + size_t(a.state_slots[s]) * per_request + e;
  float S = *mine;
  for (int k = 0; k < used; ++k) {
    const size_t number = size_t(s) * a.chunks + k;
    float* at = a.scratch + number * per_request + e;
    const float added = *at;
    *at = S;
    S = fmaf(expf(rate * a.step_sums[number * a.inner + c]), S, added);
  }
  *mine = S;
}

// ------------------------------------------------------------------------------------------------ attention with mixed heads
struct CrossArgs {
  const void* qk;
  int nq, nkv, dim, width;
  const void* q_norm;
  const void* k_norm;
  float eps;
  const int32_t* positions;
  const double* freq;
  int rotary_dim;
  const int32_t* slot_mapping;
  void* q_out;
  void* k_pool;
  void* v_pool;
  int page_size;
};

// A block per (token, head of q or k): the head's norm, the turning of its first numbers in neighbouring pairs, and the
// copies that make every (query head, value head) pair a head of the attention kernels.
template <typename T, typename TW, bool F64>
__global__ __launch_bounds__(128) void qk_cross_prepare_kernel(CrossArgs a) {
  extern __shared__ float lds[];      // the head as it came [dim], normed [dim], 16 for the sum
  float* raw = lds;
  float* normed = lds + a.dim;
  float* scratch = normed + a.dim;
  const int t = blockIdx.x, hs = blockIdx.y;
  const bool is_q = hs < a.nq;
  const T* src = (const T*)a.qk + (size_t(t) * (a.nq + a.nkv) + hs) * a.dim;
  float ss = 0.f;
  for (int d = threadIdx.x; d < a.dim; d += 128) {
    const float v = to_float(src[d]);
    raw[d] = v;
    ss = fmaf(v, v, ss);
  }
  const float r = 1.0f / sqrtf(block_sum(ss, scratch) / float(a.dim) + a.eps);
  const TW* nw = (const TW*)(is_q ? a.q_norm : a.k_norm);
  for (int d = threadIdx.x; d < a.dim; d += 128) normed[d] = raw[d] * r * to_float(nw[d]);
  __syncthreads();
  const int pos = a.positions[t];
  const int group = a.nq / a.nkv, nkv2 = a.nkv * a.nkv;
  const int slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  for (int d = threadIdx.x; d < a.width; d += 128) {
    float o = 0.f;
    if (d < a.dim) {
      o = normed[d];
      if (d < a.rotary_dim) {
        float cs, sn;
        if (F64) {
          const double angle = double(pos) * a.freq[d >> 1];
          cs = float(cos(angle));
          sn = float(sin(angle));
        } else {
          sincosf(float(pos) * float(a.freq[d >> 1]), &sn, &cs);
        }
        const float other = normed[d ^ 1];
        o = (d & 1) ? fmaf(o, cs, other * sn) : fmaf(o, cs, -other * sn);
      }
    }
    if (is_q) {
      const int kv = hs / group, rr = hs % group;
      T* q_out = (T*)a.q_out + size_t(t) * a.nq * a.nkv * a.width;
      for (int c = 0; c < a.nkv; ++c) q_out[(size_t(kv * a.nkv + c) * group + rr) * a.width + d] = from_float<T>(o);
    } else if (slot >= 0) {
      const int kv = hs - a.nq, page = slot / a.page_size, off = slot % a.page_size;
      const T value = from_float<T>(d < a.dim ? raw[d] : 0.f);
      for (int c = 0; c < a.nkv; ++c) {
        ((T*)a.k_pool)[((size_t(page) * nkv2 + kv * a.nkv + c) * a.page_size + off) * a.width + d] = from_float<T>(o);
        ((T*)a.v_pool)[((size_t(page) * nkv2 + c * a.nkv + kv) * a.width + d) * a.page_size + off] = value;
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(128) void head_mix_kernel(const T* __restrict__ o, const float* __restrict__ talk, int nq, int nkv,
                                                       int dim, int width, T* __restrict__ out) {
  const int t = blockIdx.x, h = blockIdx.y, group = nq / nkv, mine = h / group;
  const T* row = o + size_t(t) * nq * nkv * width;
  for (int d = threadIdx.x; d < dim; d += 128) {
    float sum = 0.f;
    for (int g = 0; g < nq; ++g)
      sum = fmaf(talk[h * nq + g], to_float(row[(size_t((g / group) * nkv + mine) * group + g % group) * width + d]), sum);
    out[(size_t(t) * nq + h) * dim + d] = from_float<T>(sum);
  }
}

// The same for bfloat16 heads whose numbers come in whole eights at 16 bytes: a block a token, a thread eight neighbouring
// numbers of a head, sixteen bytes a load; the sum over the heads runs in the same order.
__global__ __launch_bounds__(256) void head_mix_eights_kernel(const bf16_t* __restrict__ o, const float* __restrict__ talk, int nq,
                                                              int nkv, int dim, int width, bf16_t* __restrict__ out) {
  const int t = blockIdx.x, group = nq / nkv, per = dim / 8;
  const bf16_t* row = o + size_t(t) * nq * nkv * width;
  for (int i = threadIdx.x; i < nq * per; i += 256) {
    const int h = i / per, d = 8 * (i % per), mine = h / group;
    float sum[8], v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) sum[j] = 0.f;
    for (int g = 0; g < nq; ++g) {
      unpack8(*reinterpret_cast<const uint4*>(row + (size_t((g / group) * nkv + mine) * group + g % group) * width + d), v);
      const float w = talk[h * nq + g];
#pragma unroll
      for (int j = 0; j < 8; ++j) sum[j] = fmaf(w, v[j], sum[j]);
    }
    uint4 packed;
    packed.x = uint32_t(f32_to_bf16_bits(sum[0])) | uint32_t(f32_to_bf16_bits(sum[1])) << 16;
    packed.y = uint32_t(f32_to_bf16_bits(sum[2])) | uint32_t(f32_to_bf16_bits(sum[3])) << 16;
    packed.z = uint32_t(f32_to_bf16_bits(sum[4])) | uint32_t(f32_to_bf16_bits(sum[5])) << 16;
    packed.w = uint32_t(f32_to_bf16_bits(sum[6])) | uint32_t(f32_to_bf16_bits(sum[7])) << 16;
    *reinterpret_cast<uint4*>(out + (size_t(t) * nq + h) * dim + d) = packed;
  }
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_short_conv(void* stream, int dtype, const void* x, long long x_stride, int x_off, int channels, int taps,
                             int w_dtype, const void* w, const void* bias, int act, int add_input, void* out,
                             long long out_stride, int out_off, const int32_t* q_start, const int32_t* q_len,
                             const int32_t* seq_of_token, const int32_t* state_slots, float* state, int T, int n_seqs,
                             int max_q_len) {
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_short_conv: unsupported dtype %d", dtype);
  SP_REQUIRE(w_dtype == dtype || w_dtype == kF32, "sp_short_conv: weights of dtype %d beside rows of dtype %d", w_dtype, dtype);
  SP_REQUIRE(channels > 0 && taps > 0 && taps <= 64 && T >= 0 && n_seqs >= 0, "sp_short_conv: bad sizes (%d channels, %d taps)", channels, taps);
  SP_REQUIRE(x_off >= 0 && out_off >= 0 && x_stride >= x_off + channels && out_stride >= out_off + channels,
             "sp_short_conv: %d channels do not fit the rows", channels);
  SP_REQUIRE(act == 0 || act == 1, "sp_short_conv: no activation %d (0 = none, 1 = SiLU)", act);
  SP_REQUIRE(x && w && out && x != out && q_start && q_len && seq_of_token && state_slots && (taps == 1 || state),
             "sp_short_conv: null or aliased operand");
  if (T == 0 || n_seqs == 0) return 0;
  const ConvArgs a = {x, x_stride, x_off, channels, taps, w, bias, act, add_input, out, out_stride, out_off,
                      q_start, q_len, seq_of_token, state_slots, state};
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(T, (channels + 255) / 256);
  if (max_q_len == 1 && taps > 1) {      // single tokens: one launch convolves and moves the state rows up
    if (dtype == kF32) short_conv_single_kernel<float, float><<<grid, 256, 0, s>>>(a);
    else if (w_dtype == kF32) short_conv_single_kernel<bf16_t, float><<<grid, 256, 0, s>>>(a);
    else short_conv_single_kernel<bf16_t, bf16_t><<<grid, 256, 0, s>>>(a);
    return check_launch("sp_short_conv (single tokens)");
  }
  const auto at16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool eights = dtype == kBF16 && w_dtype == kBF16 && T >= 64 && channels % 8 == 0 && x_off % 8 == 0 && out_off % 8 == 0 &&
                      x_stride % 8 == 0 && out_stride % 8 == 0 && at16(x) && at16(out) && at16(w) && at16(bias) && at16(state);
  if (eights) short_conv_eights_kernel<<<dim3(T, (channels / 8 + 255) / 256), 256, 0, s>>>(a);
  else if (dtype == kF32) short_conv_kernel<float, float><<<grid, 256, 0, s>>>(a);
  else if (w_dtype == kF32) short_conv_kernel<bf16_t, float><<<grid, 256, 0, s>>>(a);
  else short_conv_kernel<bf16_t, bf16_t><<<grid, 256, 0, s>>>(a);
  if (check_launch("sp_short_conv")) return 1;
  if (taps == 1) return 0;
  const dim3 grid2(n_seqs, (channels + 255) / 256);
  if (dtype == kF32) short_conv_state_kernel<float><<<grid2, 256, 0, s>>>(a);
  else short_conv_state_kernel<bf16_t><<<grid2, 256, 0, s>>>(a);
  return check_launch("sp_short_conv (state)");
}

extern "C" int sp_group_rmsnorm(void* stream, const float* x, int w_dtype, const void* w, float eps, int out_dtype, void* out,
                                int T, int parts, int size) {
  SP_REQUIRE(T >= 0 && parts > 0 && size > 0 && x && w && out, "sp_group_rmsnorm: bad arguments");
  SP_REQUIRE((w_dtype == kF32 || w_dtype == kBF16) && (out_dtype == kF32 || out_dtype == kBF16), "sp_group_rmsnorm: unsupported dtype");
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const unsigned rows = unsigned(T) * parts;
  if (w_dtype == kF32 && out_dtype == kF32) group_rmsnorm_kernel<float, float><<<rows, 256, 0, s>>>(x, (const float*)w, eps, (float*)out, parts, size);
  else if (w_dtype == kF32) group_rmsnorm_kernel<float, bf16_t><<<rows, 256, 0, s>>>(x, (const float*)w, eps, (bf16_t*)out, parts, size);
  else if (out_dtype == kF32) group_rmsnorm_kernel<bf16_t, float><<<rows, 256, 0, s>>>(x, (const bf16_t*)w, eps, (float*)out, parts, size);
  else group_rmsnorm_kernel<bf16_t, bf16_t><<<rows, 256, 0, s>>>(x, (const bf16_t*)w, eps, (bf16_t*)out, parts, size);
  return check_launch("sp_group_rmsnorm");
}

extern "C" int sp_activation(void* stream, int dtype, void* x, long long n, int kind) {
  SP_REQUIRE(kind == 0, "sp_activation: no activation %d (0 = the exact GELU)", kind);
  SP_REQUIRE((dtype == kF32 || dtype == kBF16) && n >= 0 && (x || n == 0), "sp_activation: bad arguments");
  if (n == 0) return 0;
  const unsigned blocks = unsigned(n / 256 + 1 < 65536 ? n / 256 + 1 : 65536);
  if (dtype == kF32) gelu_erf_kernel<float><<<blocks, 256, 0, (hipStream_t)stream>>>((float*)x, n);
  else gelu_erf_kernel<bf16_t><<<blocks, 256, 0, (hipStream_t)stream>>>((bf16_t*)x, n);
  return check_launch("sp_activation");
}

extern "C" int sp_scale_rows(void* stream, int dtype, const void* x, const float* weights, int top, void* out, int T, int H) {
  SP_REQUIRE((dtype == kF32 || dtype == kBF16) && T >= 0 && H > 0 && top > 0 && x && weights && out && x != out,
             "sp_scale_rows: bad arguments");
  if (T == 0) return 0;
  const dim3 grid(unsigned(T) * top, H > 2048 ? 4 : 1);
  if (dtype == kF32) scale_rows_kernel<float><<<grid, 256, 0, (hipStream_t)stream>>>((const float*)x, weights, top, (float*)out, H);
  else scale_rows_kernel<bf16_t><<<grid, 256, 0, (hipStream_t)stream>>>((const bf16_t*)x, weights, top, (bf16_t*)out, H);
  return check_launch("sp_scale_rows");
}

// A kernel that asks for more than the 64 KB of LDS it gets unasked is told so once.
template <auto Kernel>
static bool more_lds(size_t bytes) {
  static bool raised = false;      // one per kernel
  if (bytes <= 64 * 1024 || raised) return true;
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  if (e != hipSuccess) {
    set_error("scan: cannot raise the LDS limit: %s", hipGetErrorString(e));
    return false;
  }
  raised = true;
  return true;
}

// Portions of more than kScanLong tokens are walked in chunks of kScanChunk.
constexpr int kScanLong = 128;

extern "C" long long sp_ssd_scan_scratch_floats(int heads, int vdim, int state_size, int n_seqs, int max_q_len) {
  if (max_q_len <= kScanLong || n_seqs <= 0) return 0;
  const long long chunks = (max_q_len + kScanChunk - 1) / kScanChunk;
  if (n_seqs * chunks > 65535) return 0;      // more chunk numbers than a grid's second dimension counts
  return (long long)n_seqs * chunks * heads * ((long long)state_size * vdim + 1);
}

extern "C" long long sp_selective_scan_scratch_floats(int inner, int state_size, int n_seqs, int max_q_len) {
  if (max_q_len <= kScanLong || n_seqs <= 0) return 0;
  const long long chunks = (max_q_len + kScanChunk - 1) / kScanChunk;
  if (n_seqs * chunks > 65535) return 0;
  return (long long)n_seqs * chunks * inner * ((long long)state_size + 1);
}

extern "C" int sp_ssd_scan(void* stream, int dtype, const void* proj, long long proj_stride, int z_off, int dt_off,
                           const void* xbc, long long xbc_stride, int heads, int vdim, int state_size, int groups,
                           const float* dt_bias, const float* a_log, const float* skip, const int32_t* q_start,
                           const int32_t* q_len, const int32_t* state_slots, float* state, float* out, int T, int n_seqs,
                           int max_q_len, float* scratch) {
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_ssd_scan: unsupported dtype %d", dtype);
  SP_REQUIRE(heads > 0 && vdim > 0 && groups > 0 && heads % groups == 0 && state_size > 0 && state_size <= 256,
             "sp_ssd_scan: %d heads of %d in %d groups with a state of %d (up to 256)", heads, vdim, groups, state_size);
  const int inner = heads * vdim;
  SP_REQUIRE(z_off >= 0 && dt_off >= 0 && proj_stride >= z_off + inner && proj_stride >= dt_off + heads &&
                 xbc_stride >= inner + 2 * groups * state_size, "sp_ssd_scan: the columns do not fit the rows");
  SP_REQUIRE(proj && xbc && dt_bias && a_log && skip && q_start && q_len && state_slots && state && out && T >= 0 && n_seqs >= 0,
             "sp_ssd_scan: null operand");
  if (T == 0 || n_seqs == 0) return 0;
  SsdArgs a = {proj, proj_stride, z_off, dt_off, xbc, xbc_stride, heads, vdim, state_size, groups, dt_bias, a_log, skip,
               q_start, q_len, state_slots, state, out, 0, 1, nullptr, nullptr, 0};
  hipStream_t s = (hipStream_t)stream;
  // two neighbouring columns a lane where a head's values are an even number and rows start at eight bytes
  const bool pairs = vdim % 2 == 0 && (reinterpret_cast<uintptr_t>(state) & 7) == 0 && (!scratch || (reinterpret_cast<uintptr_t>(scratch) & 7) == 0);
  const int columns = pairs ? 64 : 32;
#define SP_SSD_MODE(KPT, MODE)                                                                    \
  do {                                                                                            \
    if (dtype == kF32 && pairs) ssd_scan_kernel<float, KPT, MODE, 2><<<grid, 256, 0, s>>>(a);     \
    else if (dtype == kF32) ssd_scan_kernel<float, KPT, MODE, 1><<<grid, 256, 0, s>>>(a);         \
    else if (pairs) ssd_scan_kernel<bf16_t, KPT, MODE, 2><<<grid, 256, 0, s>>>(a);                \
    else ssd_scan_kernel<bf16_t, KPT, MODE, 1><<<grid, 256, 0, s>>>(a);                           \
  } while (0)
#define SP_SSD(MODE)                                  \
  do {                                                \
    if (state_size <= 32) SP_SSD_MODE(4, MODE);       \
    else if (state_size <= 64) SP_SSD_MODE(8, MODE);  \
    else if (state_size <= 128) SP_SSD_MODE(16, MODE);\
    else SP_SSD_MODE(32, MODE);                       \
  } while (0)
  const long long need = sp_ssd_scan_scratch_floats(heads, vdim, state_size, n_seqs, max_q_len);
  if (need == 0 || !scratch) {
    const dim3 grid((inner + columns - 1) / columns, n_seqs);
    SP_SSD(0);
    return check_launch("sp_ssd_scan");
  }
  a.chunk = kScanChunk;
  a.chunks = (max_q_len + kScanChunk - 1) / kScanChunk;
  a.scratch = scratch;
  a.step_sums = scratch + size_t(n_seqs) * a.chunks * heads * state_size * vdim;
  const dim3 grid((inner + 31) / 32, n_seqs * a.chunks);
  // heads of whole 32s of values whose chunk fits 64 KB of LDS: the kernels that bring a chunk into LDS first
  const int kpt = state_size <= 32 ? 4 : state_size <= 64 ? 8 : state_size <= 128 ? 16 : 32;
  const size_t element = dtype == kF32 ? 4 : 2;
  // MODE 1 holds B alone and the block's columns of u; MODE 2 also C and z
  const size_t lds1 = size_t(kScanChunk) * ((2 + 8 * kpt) * sizeof(float) + 32 * element);
  const size_t lds2 = size_t(kScanChunk) * (2 * sizeof(float) + (16 * kpt + 64) * element);
  const bool staged = vdim % 32 == 0 && lds1 <= 96 * 1024 && lds2 <= 96 * 1024;
  a.by_column = staged;
#define SP_SSD_CHUNK_MODE(KPT, MODE)                                                                       \
  do {                                                                                                     \
    const size_t lds = MODE == 1 ? lds1 : lds2;                                                            \
    if (dtype == kF32) {                                                                                   \
      if (!more_lds<ssd_chunk_kernel<float, KPT, MODE>>(lds)) return 1;                                     \
      ssd_chunk_kernel<float, KPT, MODE><<<grid, 256, lds, s>>>(a);                                        \
    } else {                                                                                               \
      if (!more_lds<ssd_chunk_kernel<bf16_t, KPT, MODE>>(lds)) return 1;                                    \
      ssd_chunk_kernel<bf16_t, KPT, MODE><<<grid, 256, lds, s>>>(a);                                       \
    }                                                                                                      \
  } while (0)
#define SP_SSD_CHUNK(MODE)                          \
  do {                                              \
    if (kpt == 4) SP_SSD_CHUNK_MODE(4, MODE);       \
    else if (kpt == 8) SP_SSD_CHUNK_MODE(8, MODE);  \
    else if (kpt == 16) SP_SSD_CHUNK_MODE(16, MODE);\
    else SP_SSD_CHUNK_MODE(32, MODE);               \
  } while (0)
  const dim3 staged_grid = grid;
  if (staged) SP_SSD_CHUNK(1);
  else {
    const dim3 grid((inner + columns - 1) / columns, staged_grid.y);
    SP_SSD(1);
  }
  if (check_launch("sp_ssd_scan (chunks)")) return 1;
  ssd_carry_kernel<<<dim3((size_t(inner) * state_size + 255) / 256, n_seqs), 256, 0, s>>>(a);
  if (check_launch("sp_ssd_scan (carry)")) return 1;
  if (staged) SP_SSD_CHUNK(2);
  else {
    const dim3 grid((inner + columns - 1) / columns, staged_grid.y);
    SP_SSD(2);
  }
#undef SP_SSD_CHUNK
#undef SP_SSD_CHUNK_MODE
#undef SP_SSD
#undef SP_SSD_MODE
  return check_launch("sp_ssd_scan (outputs)");
}

extern "C" int sp_selective_scan(void* stream, int dtype, const void* u, long long u_stride, int u_off, const void* z,
                                 long long z_stride, int z_off, const float* dt, const void* bc, long long bc_stride, int bc_off,
                                 int inner, int state_size, const float* a, const float* skip, const int32_t* q_start,
                                 const int32_t* q_len, const int32_t* state_slots, float* state, void* out, int T, int n_seqs,
                                 int max_q_len, float* scratch) {
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_selective_scan: unsupported dtype %d", dtype);
  SP_REQUIRE(inner > 0 && state_size > 0 && state_size <= 256, "sp_selective_scan: %d channels with a state of %d (up to 256)",
             inner, state_size);
  SP_REQUIRE(u_off >= 0 && z_off >= 0 && bc_off >= 0 && u_stride >= u_off + inner && z_stride >= z_off + inner &&
                 bc_stride >= bc_off + 2 * state_size, "sp_selective_scan: the columns do not fit the rows");
  SP_REQUIRE(u && z && dt && bc && a && skip && q_start && q_len && state_slots && state && out && T >= 0 && n_seqs >= 0,
             "sp_selective_scan: null operand");
  if (T == 0 || n_seqs == 0) return 0;
  SelArgs args = {u, u_stride, u_off, z, z_stride, z_off, dt, bc, bc_stride, bc_off, inner, state_size, a, skip,
                  q_start, q_len, state_slots, state, out, 0, 1, nullptr, nullptr};
  hipStream_t s = (hipStream_t)stream;
#define SP_SEL_MODE(KPT, MODE)                                                             \
  do {                                                                                     \
    if (dtype == kF32) selective_scan_kernel<float, KPT, MODE><<<grid, 256, 0, s>>>(args); \
    else selective_scan_kernel<bf16_t, KPT, MODE><<<grid, 256, 0, s>>>(args);              \
  } while (0)
#define SP_SEL(MODE)                                   \
  do {                                                 \
    if (state_size <= 16) SP_SEL_MODE(4, MODE);        \
    else if (state_size <= 32) SP_SEL_MODE(8, MODE);   \
    else if (state_size <= 64) SP_SEL_MODE(16, MODE);  \
    else if (state_size <= 128) SP_SEL_MODE(32, MODE); \
    else SP_SEL_MODE(64, MODE);                        \
  } while (0)
  const long long need = sp_selective_scan_scratch_floats(inner, state_size, n_seqs, max_q_len);
  if (need == 0 || !scratch) {
    const dim3 grid((inner + 63) / 64, n_seqs);
    SP_SEL(0);
    return check_launch("sp_selective_scan");
  }
  args.chunk = kScanChunk;
  args.chunks = (max_q_len + kScanChunk - 1) / kScanChunk;
  args.scratch = scratch;
  args.step_sums = scratch + size_t(n_seqs) * args.chunks * inner * state_size;
  const dim3 grid((inner + 63) / 64, n_seqs * args.chunks);
  // where a chunk fits 64 KB of LDS: the kernels that bring it there first
  const int kpt = state_size <= 16 ? 4 : state_size <= 32 ? 8 : state_size <= 64 ? 16 : state_size <= 128 ? 32 : 64;
  const size_t lds = size_t(kScanChunk) * (64 + 8 * kpt) * sizeof(float) + 2 * size_t(kScanChunk) * 64 * (dtype == kF32 ? 4 : 2);
  const bool staged = lds <= 64 * 1024;
#define SP_SEL_CHUNK_MODE(KPT, MODE)                                                            \
  do {                                                                                          \
    if (dtype == kF32) selective_chunk_kernel<float, KPT, MODE><<<grid, 256, lds, s>>>(args);   \
    else selective_chunk_kernel<bf16_t, KPT, MODE><<<grid, 256, lds, s>>>(args);                \
  } while (0)
#define SP_SEL_CHUNK(MODE)                           \
  do {                                               \
    if (kpt == 4) SP_SEL_CHUNK_MODE(4, MODE);        \
    else if (kpt == 8) SP_SEL_CHUNK_MODE(8, MODE);   \
    else if (kpt == 16) SP_SEL_CHUNK_MODE(16, MODE); \
    else SP_SEL_CHUNK_MODE(32, MODE);                \
  } while (0)
  if (staged) SP_SEL_CHUNK(1);
  else SP_SEL(1);
  if (check_launch("sp_selective_scan (chunks)")) return 1;
  selective_carry_kernel<<<dim3((size_t(inner) * state_size + 255) / 256, n_seqs), 256, 0, s>>>(args);
  if (check_launch("sp_selective_scan (carry)")) return 1;
  if (staged) SP_SEL_CHUNK(2);
  else SP_SEL(2);
#undef SP_SEL_CHUNK
#undef SP_SEL_CHUNK_MODE
#undef SP_SEL
#undef SP_SEL_MODE
  return check_launch("sp_selective_scan (outputs)");
}

extern "C" int sp_qk_cross_prepare(void* stream, int dtype, const void* qk, int nq, int nkv, int dim, int width, int w_dtype,
                                   const void* q_norm, const void* k_norm, float eps, const int32_t* positions,
                                   const double* freq, int rotary_dim, const int32_t* slot_mapping, void* q_out, void* k_pool,
                                   void* v_pool, int page_size, int T) {
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_qk_cross_prepare: unsupported dtype %d", dtype);
  SP_REQUIRE(w_dtype == dtype || w_dtype == kF32, "sp_qk_cross_prepare: norm weights of dtype %d beside rows of dtype %d", w_dtype, dtype);
  SP_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0 && dim > 0 && width >= dim && dim <= 4096,
             "sp_qk_cross_prepare: %d heads over %d of %d numbers at width %d", nq, nkv, dim, width);
  SP_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= dim && (rotary_dim == 0 || freq),
             "sp_qk_cross_prepare: %d of %d numbers cannot turn in pairs", rotary_dim, dim);
  SP_REQUIRE(qk && q_norm && k_norm && positions && q_out && (!slot_mapping || (k_pool && v_pool && page_size > 0)) && T >= 0,
             "sp_qk_cross_prepare: null operand");
  if (T == 0) return 0;
  const CrossArgs a = {qk, nq, nkv, dim, width, q_norm, k_norm, eps, positions, freq, rotary_dim, slot_mapping, q_out,
                       k_pool, v_pool, page_size};
  const dim3 grid(T, nq + nkv);
  const size_t lds = sizeof(float) * (2 * size_t(dim) + 16);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == kF32) qk_cross_prepare_kernel<float, float, true><<<grid, 128, lds, s>>>(a);
  else if (w_dtype == kF32) qk_cross_prepare_kernel<bf16_t, float, false><<<grid, 128, lds, s>>>(a);
  else qk_cross_prepare_kernel<bf16_t, bf16_t, false><<<grid, 128, lds, s>>>(a);
  return check_launch("sp_qk_cross_prepare");
}

extern "C" int sp_head_mix(void* stream, int dtype, const void* o, const float* talk, int nq, int nkv, int dim, int width,
                           void* out, int T) {
  SP_REQUIRE((dtype == kF32 || dtype == kBF16) && nq > 0 && nkv > 0 && nq % nkv == 0 && dim > 0 && width >= dim && T >= 0 && o &&
                 talk && out && o != out, "sp_head_mix: bad arguments");
  if (T == 0) return 0;
  const dim3 grid(T, nq);
  if (dtype == kBF16 && dim % 8 == 0 && width % 8 == 0 && (reinterpret_cast<uintptr_t>(o) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    head_mix_eights_kernel<<<T, 256, 0, (hipStream_t)stream>>>((const bf16_t*)o, talk, nq, nkv, dim, width, (bf16_t*)out);
    return check_launch("sp_head_mix");
  }
  if (dtype == kF32) head_mix_kernel<float><<<grid, 128, 0, (hipStream_t)stream>>>((const float*)o, talk, nq, nkv, dim, width, (float*)out);
  else head_mix_kernel<bf16_t><<<grid, 128, 0, (hipStream_t)stream>>>((const bf16_t*)o, talk, nq, nkv, dim, width, (bf16_t*)out);
  return check_launch("sp_head_mix");
}

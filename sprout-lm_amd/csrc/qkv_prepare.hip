// Between the q/k/v projection and attention, for mixers whose keys and values differ in width or whose queries and
// keys are normed as whole rows: one kernel per step and layer that norms, turns, blends and writes the cache.
// All arithmetic is float32 (angles in float64 where the caller gives the table's float64 remainder); only loads and
// stores see the storage type.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

struct PrepareArgs {
  const void* proj;            // [T, stride]: q (nq * dim), k (nkv * dim), v (nkv * vdim) of a token, biases already added
  long long stride;
  int nq, nkv, dim, vdim, width;   // width: numbers a head takes in q_out and in the pools (>= dim, vdim; zeros behind)
  const void* q_norm;          // [nq * dim], [nkv * dim]: RMS norm over the whole q row and the whole k row (null: none)
  const void* k_norm;
  float eps;
  const int32_t* positions;
  const float* inv_freq;       // [rotary_dim / 2]; rotary_dim == 0: nothing turns
  const float* inv_freq_tail;  // the float64 table minus inv_freq (null: angles in float32)
  int rotary_dim;
  const void* blend;           // one number lambda: v <- (1 - lambda) v + lambda first (null: v as projected)
  void* first;                 // [T, nkv * vdim]: written with v where keep_first, read where blend is given
  int keep_first;
  const int32_t* slot_mapping; // null: nothing is cached
  void* k_pool;                // [pages][nkv][page_size][width]
  void* v_pool;                // [pages][nkv][width][page_size]
  int page_size;
  void* q_out;                 // [T, nq * width]
  float magnitude;             // on every cosine and sine (1: a plain rotation)
  int head_norm;               // every q and k head, after it has turned, is divided by its root mean square over dim (eps inside)
};

// Sum of the squares of n numbers over the whole block, as the scale of an RMS norm; every thread gets it.
template <typename T>
__device__ __forceinline__ float row_scale(const T* __restrict__ x, int n, float eps, float* scratch) {
  float sq = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) { const float v = to_float(x[i]); sq = fmaf(v, v, sq); }
  return 1.0f / sqrtf(block_sum(sq, scratch) / float(n) + eps);
}

// One head of one token (query heads, then key heads, then value heads), by `count` threads of which this is `lane`.
// `scratch` (16 floats): where `count` is the whole block, the head's sum of squares is taken over it; otherwise the
// head belongs to one wave.
template <typename T>
__device__ __forceinline__ void prepare_head(const PrepareArgs& a, int t, int head, float q_scale, float k_scale, int slot,
                                             int lane, int count, float* scratch, bool whole_block) {
  const T* row = (const T*)a.proj + size_t(t) * a.stride;
  const int nq = a.nq, nkv = a.nkv, D = a.dim, V = a.vdim, W = a.width;
  const int page = slot >= 0 ? slot / a.page_size : 0, off = slot >= 0 ? slot % a.page_size : 0;
  if (head >= nq + nkv) {
    // values: blended with the first flagged layer's, or kept for the later layers; written dimension-major
    const int g = head - nq - nkv;
    const T* vrow = row + size_t(nq + nkv) * D + size_t(g) * V;
    const float lam = a.blend ? to_float(*(const T*)a.blend) : 0.f;
    T* first = a.first ? (T*)a.first + size_t(t) * nkv * V + size_t(g) * V : nullptr;
    for (int d = lane; d < W; d += count) {
      float v = 0.f;
      if (d < V) {
        v = to_float(vrow[d]);
        if (a.blend) v = to_float(from_float<T>((1.0f - lam) * v + lam * to_float(first[d])));
        else if (a.keep_first) first[d] = from_float<T>(v);
      }
      if (slot >= 0) ((T*)a.v_pool)[((size_t(page) * nkv + g) * W + d) * a.page_size + off] = from_float<T>(v);
    }
    return;
  }
  const bool is_q = head < nq;
  if (!is_q && slot < 0) return;        // a key that nobody keeps
  const T* src = row + size_t(head) * D;                  // key heads follow the query heads in the row
  const T* nw = is_q ? (const T*)a.q_norm : (const T*)a.k_norm;
  if (nw) nw += size_t(is_q ? head : head - nq) * D;
  const float scale = is_q ? q_scale : k_scale;
  T* dst = is_q ? (T*)a.q_out + (size_t(t) * nq + head) * W
                : (T*)a.k_pool + ((size_t(page) * nkv + (head - nq)) * a.page_size + off) * W;
  const int half = a.rotary_dim / 2;
  auto normed = [&](int e) {
    float x = to_float(src[e]);
    if (nw) x = to_float(from_float<T>((x * scale) * to_float(nw[e])));   // the storage type's rounding, as a norm kernel would leave it
    return x;
  };
  // A turn by an angle times `magnitude` multiplies a pair's squares by magnitude^2, so the turned head's sum of squares
  // needs no sines: the turned numbers' squares times magnitude^2, the others' as they are.
  float unit = 1.f;
  if (a.head_norm) {
    float sq = 0.f;
    const float m2 = a.magnitude * a.magnitude;
    for (int d = lane; d < D; d += count) { const float x = normed(d); sq = fmaf(x * x, d < 2 * half ? m2 : 1.f, sq); }
    sq = whole_block ? block_sum(sq, scratch) : wave_sum(sq);
    unit = 1.0f / sqrtf(sq / float(D) + a.eps);
  }
  for (int d = lane; d < W; d += count) {
    if (d >= D) { dst[d] = from_float<T>(0.f); continue; }
    if (d >= 2 * half) { dst[d] = from_float<T>(normed(d) * unit); continue; }
    if (d >= half) continue;          // written by the owner of its pair
    float sn, cs;
    if (a.inv_freq_tail) {
      double sn64, cs64;
      sincos(double(a.positions[t]) * (double(a.inv_freq[d]) + double(a.inv_freq_tail[d])), &sn64, &cs64);
      sn = float(sn64 * double(a.magnitude));
      cs = float(cs64 * double(a.magnitude));
    } else {
      sincosf(float(a.positions[t]) * a.inv_freq[d], &sn, &cs);
      sn *= a.magnitude;
      cs *= a.magnitude;
    }
    const float x = normed(d), y = normed(d + half);
    dst[d] = from_float<T>((x * cs - y * sn) * unit);
    dst[d + half] = from_float<T>((y * cs + x * sn) * unit);
  }
}

// The same four numbers at a time (8-byte loads and stores), for bfloat16 rows whose sizes are all in fours.
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                     __uint_as_float(v.y & 0xffff0000u));
}
__device__ __forceinline__ uint2 pack4(float4 v) {
  return make_uint2(uint32_t(f32_to_bf16_bits(v.x)) | (uint32_t(f32_to_bf16_bits(v.y)) << 16),
                    uint32_t(f32_to_bf16_bits(v.z)) | (uint32_t(f32_to_bf16_bits(v.w)) << 16));
}
__device__ __forceinline__ float4 round4(float4 v) {
  const uint2 p = pack4(v);
  return make_float4(__uint_as_float(p.x << 16), __uint_as_float(p.x & 0xffff0000u), __uint_as_float(p.y << 16),
                     __uint_as_float(p.y & 0xffff0000u));
}
__device__ __forceinline__ void prepare_head_fours(const PrepareArgs& a, int t, int head, float q_scale, float k_scale, int slot,
                                                   int lane, int count) {
  const bf16_t* row = (const bf16_t*)a.proj + size_t(t) * a.stride;
  const int nq = a.nq, nkv = a.nkv, D = a.dim, V = a.vdim, W = a.width;
  const int page = slot >= 0 ? slot / a.page_size : 0, off = slot >= 0 ? slot % a.page_size : 0;
  if (head >= nq + nkv) {
    const int g = head - nq - nkv;
    const bf16_t* vrow = row + size_t(nq + nkv) * D + size_t(g) * V;
    const float lam = a.blend ? to_float(*(const bf16_t*)a.blend) : 0.f;
    bf16_t* first = a.first ? (bf16_t*)a.first + size_t(t) * nkv * V + size_t(g) * V : nullptr;
    for (int d = 4 * lane; d < W; d += 4 * count) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (d < V) {
        v = load4(vrow + d);
        if (a.blend) {
          const float4 f = load4(first + d);
          v = make_float4((1.0f - lam) * v.x + lam * f.x, (1.0f - lam) * v.y + lam * f.y, (1.0f - lam) * v.z + lam * f.z,
                          (1.0f - lam) * v.w + lam * f.w);
        } else if (a.keep_first) {
          *reinterpret_cast<uint2*>(first + d) = pack4(v);
        }
      }
      if (slot >= 0) {
        const uint2 p = pack4(v);
        bf16_t* dst = (bf16_t*)a.v_pool + ((size_t(page) * nkv + g) * W + d) * a.page_size + off;
        dst[0] = bf16_t{uint16_t(p.x & 0xffffu)};
        dst[a.page_size] = bf16_t{uint16_t(p.x >> 16)};
        dst[2 * size_t(a.page_size)] = bf16_t{uint16_t(p.y & 0xffffu)};
        dst[3 * size_t(a.page_size)] = bf16_t{uint16_t(p.y >> 16)};
      }
    }
    return;
  }
  const bool is_q = head < nq;
  if (!is_q && slot < 0) return;
  const bf16_t* src = row + size_t(head) * D;
  const bf16_t* nw = is_q ? (const bf16_t*)a.q_norm : (const bf16_t*)a.k_norm;
  if (nw) nw += size_t(is_q ? head : head - nq) * D;
  const float scale = is_q ? q_scale : k_scale;
  bf16_t* dst = is_q ? (bf16_t*)a.q_out + (size_t(t) * nq + head) * W
                     : (bf16_t*)a.k_pool + ((size_t(page) * nkv + (head - nq)) * a.page_size + off) * W;
  const int half = a.rotary_dim / 2;
  auto normed = [&](int e) {
    float4 x = load4(src + e);
    if (nw) {
      const float4 w = load4(nw + e);
      x = round4(make_float4((x.x * scale) * w.x, (x.y * scale) * w.y, (x.z * scale) * w.z, (x.w * scale) * w.w));
    }
    return x;
  };
  for (int d = 4 * lane; d < W; d += 4 * count) {
    if (d >= D) { *reinterpret_cast<uint2*>(dst + d) = make_uint2(0u, 0u); continue; }
    if (d >= 2 * half) { *reinterpret_cast<uint2*>(dst + d) = pack4(normed(d)); continue; }
    if (d >= half) continue;
    const float pos = float(a.positions[t]);
    float sn[4], cs[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) sincosf(pos * a.inv_freq[d + j], &sn[j], &cs[j]);
    const float4 x = normed(d), y = normed(d + half);
    *reinterpret_cast<uint2*>(dst + d) = pack4(make_float4(x.x * cs[0] - y.x * sn[0], x.y * cs[1] - y.y * sn[1],
                                                           x.z * cs[2] - y.z * sn[2], x.w * cs[3] - y.w * sn[3]));
    *reinterpret_cast<uint2*>(dst + d + half) = pack4(make_float4(y.x * cs[0] + x.x * sn[0], y.y * cs[1] + x.y * sn[1],
                                                                  y.z * cs[2] + x.z * sn[2], y.w * cs[3] + x.w * sn[3]));
  }
}

// PER_HEAD: one block per (token, head), for the few tokens of a decode step: the work still spreads over the chip and
// every block waits for memory once; a block of a normed head sums the squares of its whole row by itself (a few
// kilobytes that the other heads' blocks read at the same time).  Otherwise one block a token: the row's two sums
// are taken once, and the block's waves take the heads in turn.
__device__ __forceinline__ float row_scale_fours(const bf16_t* __restrict__ x, int n, float eps, float* scratch) {
  float sq = 0.f;
  for (int i = 4 * threadIdx.x; i < n; i += 4 * blockDim.x) {
    const float4 v = load4(x + i);
    sq = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, sq))));
  }
  return 1.0f / sqrtf(block_sum(sq, scratch) / float(n) + eps);
}

// FOURS (bfloat16 only): every size is in fours and every row starts at a multiple of 8 bytes.
template <typename T, bool PER_HEAD, bool FOURS>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(PrepareArgs a) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = (const T*)a.proj + size_t(t) * a.stride;
  const int slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  const int heads = a.nq + 2 * a.nkv;
  if (PER_HEAD) {
    const int head = blockIdx.y;
    float scale = 1.f;
    if (a.q_norm && head < a.nq + a.nkv && (head < a.nq || slot >= 0)) {
      const T* whole = head < a.nq ? row : row + size_t(a.nq) * a.dim;
      const int n = (head < a.nq ? a.nq : a.nkv) * a.dim;
      if constexpr (FOURS) scale = row_scale_fours(whole, n, a.eps, scratch);
      else scale = row_scale(whole, n, a.eps, scratch);
    }
    if constexpr (FOURS) prepare_head_fours(a, t, head, scale, scale, slot, threadIdx.x, blockDim.x);
    else prepare_head<T>(a, t, head, scale, scale, slot, threadIdx.x, blockDim.x, scratch, true);
    return;
  }
  float q_scale = 1.f, k_scale = 1.f;
  if (a.q_norm) {
    if constexpr (FOURS) {
      q_scale = row_scale_fours(row, a.nq * a.dim, a.eps, scratch);
      k_scale = row_scale_fours(row + size_t(a.nq) * a.dim, a.nkv * a.dim, a.eps, scratch);
    } else {
      q_scale = row_scale(row, a.nq * a.dim, a.eps, scratch);
      k_scale = row_scale(row + size_t(a.nq) * a.dim, a.nkv * a.dim, a.eps, scratch);
    }
  }
  const int wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  for (int head = wave; head < heads; head += waves) {
    if constexpr (FOURS) prepare_head_fours(a, t, head, q_scale, k_scale, slot, threadIdx.x & 63, 64);
    else prepare_head<T>(a, t, head, q_scale, k_scale, slot, threadIdx.x & 63, 64, scratch, false);
  }
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_qkv_prepare(void* stream, int dtype, const void* proj, long long stride, int nq, int nkv, int dim, int vdim,
                              int width, const void* q_norm, const void* k_norm, float eps, const int32_t* positions,
                              const float* inv_freq, const float* inv_freq_tail, int rotary_dim, const void* blend,
                              void* first, int keep_first, const int32_t* slot_mapping, void* k_pool, void* v_pool,
                              int page_size, int num_pages, void* q_out, int T, float magnitude, int head_norm) {
  SP_REQUIRE(T >= 0 && nq > 0 && nkv > 0 && dim > 0 && vdim > 0 && width >= dim && width >= vdim,
             "sp_qkv_prepare: bad sizes nq=%d nkv=%d dim=%d vdim=%d width=%d", nq, nkv, dim, vdim, width);
  SP_REQUIRE(stride >= (long long)(nq + nkv) * dim + (long long)nkv * vdim, "sp_qkv_prepare: a row of %lld numbers does not hold q, k and v", stride);
  SP_REQUIRE(proj && q_out, "sp_qkv_prepare: null operand");
  SP_REQUIRE((q_norm == nullptr) == (k_norm == nullptr), "sp_qkv_prepare: queries and keys are normed together or not at all");
  SP_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= dim, "sp_qkv_prepare: %d numbers cannot turn in a head of %d", rotary_dim, dim);
  SP_REQUIRE(rotary_dim == 0 || (positions && inv_freq), "sp_qkv_prepare: a rotation needs positions and frequencies");
  SP_REQUIRE(!(blend || keep_first) || first, "sp_qkv_prepare: blending values needs the buffer of the first layer's");
  SP_REQUIRE(!slot_mapping || (k_pool && v_pool && page_size > 0 && num_pages > 0), "sp_qkv_prepare: bad cache geometry");
  if (T == 0) return 0;
  PrepareArgs a = {proj, stride, nq, nkv, dim, vdim, width, q_norm, k_norm, eps, positions, inv_freq, inv_freq_tail, rotary_dim,
                   blend, first, keep_first, slot_mapping, k_pool, v_pool, page_size, q_out, magnitude, head_norm};
  hipStream_t s = (hipStream_t)stream;
  SP_REQUIRE(nq + 2 * nkv <= 65535, "sp_qkv_prepare: %d heads are more than a launch's second dimension holds", nq + 2 * nkv);
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_qkv_prepare: unsupported dtype %d", dtype);
  auto eight = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7) == 0; };
  const bool fours = dtype == kBF16 && !inv_freq_tail && !head_norm && magnitude == 1.0f && dim % 4 == 0 && vdim % 4 == 0 && width % 4 == 0 && rotary_dim % 8 == 0 &&
                     stride % 4 == 0 && eight(proj) && eight(q_out) && eight(q_norm) && eight(k_norm) && eight(first) &&
                     eight(k_pool);
  if (T * (nq + 2 * nkv) <= 2048) {      // few tokens: a block per head
    const dim3 grid(T, nq + 2 * nkv);
    const int threads = width <= 64 ? 64 : 128;
    if (dtype == kF32) qkv_prepare_kernel<float, true, false><<<grid, threads, 0, s>>>(a);
    else if (fours) qkv_prepare_kernel<bf16_t, true, true><<<grid, 64, 0, s>>>(a);
    else qkv_prepare_kernel<bf16_t, true, false><<<grid, threads, 0, s>>>(a);
  } else {
    if (dtype == kF32) qkv_prepare_kernel<float, false, false><<<T, 256, 0, s>>>(a);
    else if (fours) qkv_prepare_kernel<bf16_t, false, true><<<T, 256, 0, s>>>(a);
    else qkv_prepare_kernel<bf16_t, false, false><<<T, 256, 0, s>>>(a);
  }
  return check_launch("sp_qkv_prepare");
}

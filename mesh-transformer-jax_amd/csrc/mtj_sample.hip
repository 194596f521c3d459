// Samplers: greedy argmax, and nucleus (top-k / top-p) filtering with an inverse-CDF draw.
#include <cstring>
#include "mtj_common.h"
#include <rocprim/device/device_segmented_radix_sort.hpp>

namespace {

constexpr int SNT = 1024;  // threads per row

// x_next[b, :] = W[token, :] + bias, by the whole workgroup (token is uniform)
__device__ __forceinline__ void embed_next(const mtj_next_embed& ne, int b, int V, int token) {
  if (!ne.w) return;
  const bool hit = (uint32_t)token < (uint32_t)V;
  float* xo = ne.x_next + (int64_t)b * ne.d;
  for (int64_t c = threadIdx.x; c < ne.d; c += blockDim.x) {
    float w = 0.f;
    if (hit) w = ne.dtype == MTJ_F32 ? reinterpret_cast<const float*>(ne.w)[(int64_t)token * ne.d + c]
                                     : elem<bf16_t>::load(reinterpret_cast<const bf16_t*>(ne.w) + (int64_t)token * ne.d + c);
    xo[c] = w + ne.bias[c];
  }
}

// ---------------------------------------------------------------- greedy
__global__ __launch_bounds__(SNT) void greedy_kernel(const float* __restrict__ logits, int V, int32_t* __restrict__ tok,
                                                     int32_t* __restrict__ out_tokens, int64_t ld_tokens,
                                                     int32_t* __restrict__ pos, const int32_t* __restrict__ pos_start,
                                                     const mtj_next_embed ne) {
  __shared__ float sv[SNT / 64];
  __shared__ int si[SNT / 64];
  __shared__ int chosen;
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* row = logits + (int64_t)b * V;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  const int V4 = ((reinterpret_cast<uintptr_t>(row) & 15u) == 0) ? (V & ~3) : 0;   // float4 body when aligned
  for (int i = tid * 4; i < V4; i += SNT * 4) {
    const floatx4 v = *reinterpret_cast<const floatx4*>(row + i);
    if (v.x > best) { best = v.x; bi = i; }          // indices grow, so '>' keeps the lowest id of a tie
    if (v.y > best) { best = v.y; bi = i + 1; }
    if (v.z > best) { best = v.z; bi = i + 2; }
    if (v.w > best) { best = v.w; bi = i + 3; }
  }
  for (int i = V4 + tid; i < V; i += SNT) {
    const float v = row[i];
    if (v > best || (v == best && i < bi)) { best = v; bi = i; }
  }
  if (bi == 0x7fffffff && tid < V) bi = tid;  // rows of NaN / -inf still yield a valid id
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o);
    const int oi = __shfl_xor(bi, o);
    if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
  }
  if (lane == 0) { sv[wave] = best; si[wave] = bi; }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < SNT / 64; ++w)
      if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
    if (bi >= V) bi = 0;
    tok[b] = bi;
    if (out_tokens) out_tokens[(int64_t)b * ld_tokens + (pos[b] - pos_start[b])] = bi;
    pos[b] += 1;
    chosen = bi;
  }
  __syncthreads();
  embed_next(ne, b, V, chosen);
}

// ---------------------------------------------------------------- nucleus
// Sort key: monotone image of the float in the high 32 bits, token id below it.  Sorting these
// descending gives descending logits with the HIGHER id first among equal logits, which is the order
// jnp.argsort(logits)[:, ::-1] produces (sampling.py:12).  All keys are distinct.
__device__ __forceinline__ uint64_t sort_key(float f, uint32_t id) {
  f += 0.0f;  // -0.0 -> +0.0: they compare equal in a sort
  uint32_t u = __float_as_uint(f);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return ((uint64_t)u << 16) | id;
}
__device__ __forceinline__ float key_value(uint64_t k) {
  uint32_t u = (uint32_t)(k >> 16);
  u = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
  return __uint_as_float(u);
}

__global__ void make_keys_kernel(const float* __restrict__ logits, int64_t total, int V, uint64_t* __restrict__ keys) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) keys[i] = sort_key(logits[i], (uint32_t)(i % V));
}

__global__ void offsets_kernel(uint32_t* off, int B, int V) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i <= B) off[i] = (uint32_t)i * (uint32_t)V;
}

// f - a*b with the product rounded to float32 first (no fused multiply-add): logits -= 1e10 * mask is
// two array operations in the reference (sampling.py:24-26)
__device__ __forceinline__ float sub_product(float f, float a, float b) {
#pragma clang fp contract(off)
  const float p = a * b;
  return f - p;
}

// block-wide helpers (double)
__device__ double block_sum(double v, double* sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  __syncthreads();
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  double t = 0.0;
  for (int w = 0; w < SNT / 64; ++w) t += sh[w];
  return t;
}
__device__ double block_max(double v, double* sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmax(v, __shfl_xor(v, o));
  __syncthreads();
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  double t = sh[0];
  for (int w = 1; w < SNT / 64; ++w) t = fmax(t, sh[w]);
  return t;
}
// exclusive prefix over per-thread totals, in thread order
__device__ double block_exclusive(double v, double* sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  double inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const double t = __shfl_up(inc, o);
    if (lane >= o) inc += t;
  }
  __syncthreads();
  if (lane == 63) sh[wave] = inc;
  __syncthreads();
  double base = 0.0;
  for (int w = 0; w < wave; ++w) base += sh[w];
  return base + inc - v;
}

// One workgroup per row, each thread owns a contiguous run of the sorted order.
__global__ __launch_bounds__(SNT) void nucleus_kernel(const float* __restrict__ logits, const uint64_t* __restrict__ sorted,
                                                      int V, const double* __restrict__ top_p,
                                                      const double* __restrict__ temp, const int32_t* __restrict__ top_k,
                                                      const double* __restrict__ uniforms, int64_t ld_u,
                                                      int32_t* __restrict__ tok, int32_t* __restrict__ out_tokens,
                                                      int64_t ld_tokens, int32_t* __restrict__ pos,
                                                      const int32_t* __restrict__ pos_start,
                                                      uint8_t* __restrict__ keep_mask, float* __restrict__ filtered,
                                                      float* __restrict__ fsorted, const mtj_next_embed ne) {
  __shared__ double sh[SNT / 64];
  __shared__ int sh_i[SNT / 64];
  __shared__ int chosen;
  const int b = blockIdx.x, tid = threadIdx.x;
  const uint64_t* srt = sorted + (int64_t)b * V;
  float* fs = fsorted + (int64_t)b * V;           // filtered logits in sorted order
  const int per = (V + SNT - 1) / SNT;
  const int j0 = tid * per, j1 = (j0 + per < V) ? j0 + per : V;
  const int step = pos[b] - pos_start[b];
  const double tp = top_p[b], tmp = temp[b], u = uniforms[(int64_t)b * ld_u + step];
  const int kk = top_k ? top_k[b] : 0x7fffffff;

  // ---- softmax of the sorted logits (max is element 0) and its running sum
  const double l0 = (double)key_value(srt[0]);
  double loc = 0.0;
  for (int j = j0; j < j1; ++j) loc += exp((double)key_value(srt[j]) - l0);
  const double Z = block_sum(loc, sh);
  double run = block_exclusive(loc / Z, sh);      // mass strictly before j0
  // ---- filter: remove rank j when the mass of ranks [0, j-1] already exceeds top_p (sampling.py:28-30)
  double tmax = -INFINITY;
  for (int j = j0; j < j1; ++j) {
    const uint64_t key = srt[j];
    const uint32_t id = (uint32_t)(key & 0xffffu);
    const float l = logits[(int64_t)b * V + id];   // the original bits (keeps -0.0)
    const bool rm = (j > 0) && (run > tp);
    run += exp((double)key_value(key) - l0) / Z;
    float f = l;
    if (j >= kk) f = sub_product(f, 1e10f, (float)id);   // top-k quirk: subtracts 1e10 * token id
    f = f - (rm ? 1e10f : 0.0f);
    fs[j] = f;
    if (filtered) filtered[(int64_t)b * V + id] = f;
    if (keep_mask) keep_mask[(int64_t)b * V + id] = (f == l) ? 1 : 0;
    tmax = fmax(tmax, (double)f / tmp);
  }
  tmax = block_max(tmax, sh);
  // ---- inverse-CDF draw over exp(filtered / temp - max) in sorted order
  double wloc = 0.0;
  for (int j = j0; j < j1; ++j) wloc += exp((double)fs[j] / tmp - tmax);
  const double total = block_sum(wloc, sh);
  double cum = block_exclusive(wloc, sh);
  const double target = u * total;
  int first = 0x7fffffff, lastpos = -1;
  for (int j = j0; j < j1; ++j) {
    const double w = exp((double)fs[j] / tmp - tmax);
    cum += w;
    if (w > 0.0) lastpos = j;
    if (cum > target && first == 0x7fffffff) first = j;
  }
  // min over first, max over lastpos
  const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    first = min(first, __shfl_xor(first, o));
    lastpos = max(lastpos, __shfl_xor(lastpos, o));
  }
  __syncthreads();
  if (lane == 0) { sh_i[wave] = first; sh[wave] = (double)lastpos; }
  __syncthreads();
  if (tid == 0) {
    int f = 0x7fffffff, lp = -1;
    for (int w = 0; w < SNT / 64; ++w) { f = min(f, sh_i[w]); lp = max(lp, (int)sh[w]); }
    int j = (f != 0x7fffffff) ? f : (lp >= 0 ? lp : 0);
    const int id = (int)(srt[j] & 0xffffu);
    tok[b] = id;
    if (out_tokens) out_tokens[(int64_t)b * ld_tokens + step] = id;
    pos[b] += 1;
    chosen = id;
  }
  __syncthreads();
  embed_next(ne, b, V, chosen);
}

struct sample_layout {
  size_t keys_in, keys_out, fsorted, offsets, sort_temp, total;
};
size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// rocPRIM's scratch need for B segments of V 64-bit keys; fixed upper bound so that the size query does
// not need a device: the segmented sort asks for a partition scratch of a few words per segment.
sample_layout layout(int64_t B, int64_t V) {
  sample_layout L;
  size_t o = 0;
  L.keys_in = o;  o += align256((size_t)B * V * 8);
  L.keys_out = o; o += align256((size_t)B * V * 8);
  L.fsorted = o;  o += align256((size_t)B * V * 4);
  L.offsets = o;  o += align256((size_t)(B + 1) * 4);
  L.sort_temp = o; o += align256((size_t)B * V * 8 + (size_t)B * 64 + (1 << 16));
  L.total = o;
  return L;
}

}  // namespace

static int check_next(const mtj_next_embed* next, mtj_next_embed* ne, const char* who) {
  *ne = mtj_next_embed{nullptr, nullptr, nullptr, 0, 0};
  if (!next || !next->w) return MTJ_OK;
  MTJ_REQUIRE(next->bias && next->x_next && next->d > 0 && (next->dtype == MTJ_F32 || next->dtype == MTJ_BF16), MTJ_EINVAL,
              "%s: incomplete next-step embedding", who);
  *ne = *next;
  return MTJ_OK;
}

extern "C" int mtj_sample_greedy(const float* logits, int64_t B, int64_t V, int32_t* tok, int32_t* out_tokens,
                                 int64_t ld_tokens, int32_t* pos, const int32_t* pos_start, const mtj_next_embed* next,
                                 void* stream) {
  MTJ_REQUIRE(logits && tok && pos && pos_start, MTJ_EINVAL, "mtj_sample_greedy: null pointer");
  MTJ_REQUIRE(B > 0 && V > 0 && V < (1ll << 31), MTJ_EINVAL, "mtj_sample_greedy: bad shape");
  mtj_next_embed ne;
  if (int rc = check_next(next, &ne, "mtj_sample_greedy")) return rc;
  greedy_kernel<<<(unsigned)B, SNT, 0, (hipStream_t)stream>>>(logits, (int)V, tok, out_tokens, ld_tokens, pos, pos_start, ne);
  return mtj_check_launch("mtj_sample_greedy");
}

extern "C" int64_t mtj_sample_work_bytes(int64_t B, int64_t V) { return (int64_t)layout(B, V).total; }

extern "C" int mtj_sample_nucleus(const float* logits, int64_t B, int64_t V, const double* top_p, const double* temp,
                                  const int32_t* top_k, const double* uniforms, int64_t ld_u, int32_t* tok,
                                  int32_t* out_tokens, int64_t ld_tokens, int32_t* pos, const int32_t* pos_start,
                                  uint8_t* keep_mask, float* filtered, void* work, const mtj_next_embed* next,
                                  void* stream) {
  MTJ_REQUIRE(logits && top_p && temp && uniforms && tok && pos && pos_start && work, MTJ_EINVAL,
              "mtj_sample_nucleus: null pointer");
  MTJ_REQUIRE(B > 0 && V > 0 && V <= 65536 && B * V < (1ll << 31), MTJ_EINVAL,
              "mtj_sample_nucleus: V=%lld must be <= 65536 (token id shares the sort key)", (long long)V);
  MTJ_REQUIRE((reinterpret_cast<uintptr_t>(work) & 255u) == 0, MTJ_EALIGN, "mtj_sample_nucleus: work must be 256-byte aligned");
  mtj_next_embed ne;
  if (int rc = check_next(next, &ne, "mtj_sample_nucleus")) return rc;
  hipStream_t s = (hipStream_t)stream;
  const sample_layout L = layout(B, V);
  unsigned char* w = reinterpret_cast<unsigned char*>(work);
  uint64_t* kin = reinterpret_cast<uint64_t*>(w + L.keys_in);
  uint64_t* kout = reinterpret_cast<uint64_t*>(w + L.keys_out);
  float* fsorted = reinterpret_cast<float*>(w + L.fsorted);
  uint32_t* off = reinterpret_cast<uint32_t*>(w + L.offsets);
  const int64_t total = B * V;
  make_keys_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(logits, total, (int)V, kin);
  offsets_kernel<<<(unsigned)((B + 1 + 255) / 256), 256, 0, s>>>(off, (int)B, (int)V);
  size_t need = 0;
  hipError_t e = rocprim::segmented_radix_sort_keys_desc(nullptr, need, kin, kout, (unsigned)total, (unsigned)B, off,
                                                         off + 1, 0, 48, s, false);
  if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "mtj_sample_nucleus: sort size query: %s", hipGetErrorString(e));
  const size_t have = L.total - L.sort_temp;
  MTJ_REQUIRE(need <= have, MTJ_ELIMIT, "mtj_sample_nucleus: sort scratch %zu > reserved %zu", need, have);
  e = rocprim::segmented_radix_sort_keys_desc(w + L.sort_temp, need, kin, kout, (unsigned)total, (unsigned)B, off,
                                              off + 1, 0, 48, s, false);
  if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "mtj_sample_nucleus: sort: %s", hipGetErrorString(e));
  nucleus_kernel<<<(unsigned)B, SNT, 0, s>>>(logits, kout, (int)V, top_p, temp, top_k, uniforms, ld_u, tok, out_tokens,
                                             ld_tokens, pos, pos_start, keep_mask, filtered, fsorted, ne);
  return mtj_check_launch("mtj_sample_nucleus");
}

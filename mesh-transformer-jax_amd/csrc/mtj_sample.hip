// Samplers: greedy argmax, and nucleus (top-k / top-p) filtering with an inverse-CDF draw.
#include <cstring>
#include "mtj_common.h"
#include <rocprim/device/device_merge_sort.hpp>

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

// All rows are sorted by one device-wide sort (a sort per row would leave most of the chip idle): bits 48..62
// carry B-1-row, so that descending order keeps row 0 first and row b occupies [b*V, (b+1)*V) of the output.
__global__ void make_keys_kernel(const float* __restrict__ logits, int64_t total, int V, int B, uint64_t* __restrict__ keys) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) {
    const int64_t row = i / V;
    keys[i] = ((uint64_t)(B - 1 - row) << 48) | sort_key(logits[i], (uint32_t)(i - row * V));
  }
}

struct key_desc {
  __device__ __forceinline__ bool operator()(const uint64_t& a, const uint64_t& b) const { return a > b; }
};

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

// wave-wide inclusive prefix sum (double), lanes in order
__device__ __forceinline__ double wave_inclusive(double v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const double t = __shfl_up(v, o);
    if (lane >= o) v += t;
  }
  return v;
}

// One workgroup of 16 wavefronts per row.  Wavefront w owns ranks [w*NT*64, (w+1)*NT*64) of the sorted order in
// NT tiles of 64 consecutive ranks (lane = rank inside the tile: coalesced reads); the sorted values and ids
// stay in registers for all three sweeps, and running sums are carried tile to tile inside the wavefront.
template <int NT_MAX>        // tiles per wavefront: V <= 16 * 64 * NT_MAX
__global__ __launch_bounds__(SNT) void nucleus_kernel(const float* __restrict__ logits, const uint64_t* __restrict__ sorted,
                                                      int V, const double* __restrict__ top_p,
                                                      const double* __restrict__ temp, const int32_t* __restrict__ top_k,
                                                      const double* __restrict__ uniforms, int64_t ld_u,
                                                      int32_t* __restrict__ tok, int32_t* __restrict__ out_tokens,
                                                      int64_t ld_tokens, int32_t* __restrict__ pos,
                                                      const int32_t* __restrict__ pos_start,
                                                      uint8_t* __restrict__ keep_mask, float* __restrict__ filtered,
                                                      const mtj_next_embed ne) {
  __shared__ double sh[SNT / 64];
  __shared__ int sh_i[SNT / 64];
  __shared__ int chosen;
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint64_t* srt = sorted + (int64_t)b * V;
  const int nt = (V + SNT - 1) / SNT;             // tiles per wavefront (uniform), <= NT_MAX
  const int jw = wave * nt * 64 + lane;           // my rank in tile 0
  const int step = pos[b] - pos_start[b];
  const double tp = top_p[b], tmp = temp[b], u = uniforms[(int64_t)b * ld_u + step];
  const int kk = top_k ? top_k[b] : 0x7fffffff;

  float val[NT_MAX];                              // sorted logits of my ranks (-inf beyond V)
  uint32_t idp[NT_MAX / 2];                       // their token ids, two per register
#pragma unroll
  for (int t = 0; t < NT_MAX; ++t) {
    val[t] = -INFINITY;
    if ((t & 1) == 0) idp[t / 2] = 0;
    if (t < nt) {
      const int j = jw + t * 64;
      if (j < V) {
        const uint64_t key = srt[j];
        val[t] = key_value(key);
        idp[t / 2] |= (uint32_t)(key & 0xffffu) << (16 * (t & 1));
      }
    }
  }
  auto id_of = [&](int t) { return (idp[t / 2] >> (16 * (t & 1))) & 0xffffu; };

  // ---- softmax of the sorted logits (the maximum is rank 0)
  const double l0 = (double)key_value(srt[0]);
  double loc = 0.0;
#pragma unroll
  for (int t = 0; t < NT_MAX; ++t)
    if (t < nt) loc += (jw + t * 64 < V) ? exp((double)val[t] - l0) : 0.0;
  const double Z = block_sum(loc, sh);            // leaves the per-wavefront sums in sh
  double base = 0.0;                              // mass of the ranks before my wavefront's
  for (int w = 0; w < wave; ++w) base += sh[w] / Z;
  __syncthreads();

  // ---- filter: remove rank j when the mass of ranks [0, j-1] already exceeds top_p (sampling.py:28-30)
  uint64_t removed = 0;                           // bit t: my rank of tile t is outside the nucleus
  double tmax = -INFINITY;
  auto filtered_of = [&](int t, uint32_t id, float l) {
    float f = l;
    if (jw + t * 64 >= kk) f = sub_product(f, 1e10f, (float)id);   // top-k quirk: subtracts 1e10 * token id
    return f - (((removed >> t) & 1) ? 1e10f : 0.0f);
  };
#pragma unroll
  for (int t = 0; t < NT_MAX; ++t) {
    if (t < nt) {
      const int j = jw + t * 64;
      const bool live = j < V;
      if (base > tp) {
        // the mass before this tile already exceeds top_p (base is the same in every lane, and it only grows):
        // every rank of the tile is outside the nucleus, no exponential needed
        if (live && j > 0) removed |= 1ull << t;
      } else {
        const double e = live ? exp((double)val[t] - l0) / Z : 0.0;
        const double incl = wave_inclusive(e);
        const double before = base + (incl - e);
        if (live && j > 0 && before > tp) removed |= 1ull << t;
        base += __shfl(incl, 63);
      }
      if (live) {
        const uint32_t id = id_of(t);
        // the sort key folds -0.0 into +0.0: fetch the original bits for a zero
        const float l = (val[t] == 0.0f) ? logits[(int64_t)b * V + id] : val[t];
        const float f = filtered_of(t, id, l);
        if (filtered) filtered[(int64_t)b * V + id] = f;
        if (keep_mask) keep_mask[(int64_t)b * V + id] = (f == l) ? 1 : 0;
        tmax = fmax(tmax, (double)f / tmp);
      }
    }
  }
  tmax = block_max(tmax, sh);
  // ---- inverse-CDF draw over exp(filtered / temp - max) in sorted order
  // exp(x) is exactly 0 in float64 below -745.14: what the filter pushed down by 1e10 (almost every rank of a peaked
  // distribution) needs no exponential
  auto weight = [&](int t) {
    const double x = (double)filtered_of(t, id_of(t), val[t]) / tmp - tmax;
    return x < -746.0 ? 0.0 : exp(x);
  };
  double wloc = 0.0;
#pragma unroll
  for (int t = 0; t < NT_MAX; ++t)
    if (t < nt && jw + t * 64 < V) wloc += weight(t);
  const double total = block_sum(wloc, sh);
  double cum = 0.0;
  for (int w = 0; w < wave; ++w) cum += sh[w];
  const double target = u * total;
  int first = 0x7fffffff, lastpos = -1;
#pragma unroll
  for (int t = 0; t < NT_MAX; ++t) {
    if (t < nt) {
      const int j = jw + t * 64;
      const double w = (j < V) ? weight(t) : 0.0;
      const double incl = wave_inclusive(w);
      if (w > 0.0) lastpos = j;
      if (cum + incl > target && j < V && first == 0x7fffffff) first = j;
      cum += __shfl(incl, 63);
    }
  }
  // min over first, max over lastpos
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
  size_t keys_in, keys_out, sort_temp, total;
};
size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// rocPRIM's merge sort needs one more buffer of keys plus a few words per block; a fixed upper bound, so that
// the size query does not need a device.
sample_layout layout(int64_t B, int64_t V) {
  sample_layout L;
  size_t o = 0;
  L.keys_in = o;  o += align256((size_t)B * V * 8);
  L.keys_out = o; o += align256((size_t)B * V * 8);
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
  MTJ_REQUIRE(B > 0 && B <= 32768 && V > 0 && V <= 65536 && B * V < (1ll << 31), MTJ_EINVAL,
              "mtj_sample_nucleus: V=%lld must be <= 65536 (token id shares the sort key)", (long long)V);
  MTJ_REQUIRE((reinterpret_cast<uintptr_t>(work) & 255u) == 0, MTJ_EALIGN, "mtj_sample_nucleus: work must be 256-byte aligned");
  mtj_next_embed ne;
  if (int rc = check_next(next, &ne, "mtj_sample_nucleus")) return rc;
  hipStream_t s = (hipStream_t)stream;
  const sample_layout L = layout(B, V);
  unsigned char* w = reinterpret_cast<unsigned char*>(work);
  uint64_t* kin = reinterpret_cast<uint64_t*>(w + L.keys_in);
  uint64_t* kout = reinterpret_cast<uint64_t*>(w + L.keys_out);
  const int64_t total = B * V;
  make_keys_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(logits, total, (int)V, (int)B, kin);
  size_t need = 0;
  hipError_t e = rocprim::merge_sort(nullptr, need, kin, kout, (size_t)total, key_desc(), s, false);
  if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "mtj_sample_nucleus: sort size query: %s", hipGetErrorString(e));
  const size_t have = L.total - L.sort_temp;
  MTJ_REQUIRE(need <= have, MTJ_ELIMIT, "mtj_sample_nucleus: sort scratch %zu > reserved %zu", need, have);
  e = rocprim::merge_sort(w + L.sort_temp, need, kin, kout, (size_t)total, key_desc(), s, false);
  if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "mtj_sample_nucleus: sort: %s", hipGetErrorString(e));
  if (V <= SNT * 50)      // GPT-J's 50400-entry vocabulary: everything stays in registers
    nucleus_kernel<50><<<(unsigned)B, SNT, 0, s>>>(logits, kout, (int)V, top_p, temp, top_k, uniforms, ld_u, tok, out_tokens,
                                                   ld_tokens, pos, pos_start, keep_mask, filtered, ne);
  else
    nucleus_kernel<64><<<(unsigned)B, SNT, 0, s>>>(logits, kout, (int)V, top_p, temp, top_k, uniforms, ld_u, tok, out_tokens,
                                                   ld_tokens, pos, pos_start, keep_mask, filtered, ne);
  return mtj_check_launch("mtj_sample_nucleus");
}

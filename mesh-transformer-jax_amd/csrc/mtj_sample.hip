// Samplers: greedy argmax, and nucleus (top-k / top-p) filtering with an inverse-CDF draw.
#include <cstring>
#include "mtj_common.h"

namespace {

constexpr int SNT = 1024;  // threads per row

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

// f - a*b with the product rounded to float32 first (no fused multiply-add): logits -= 1e10 * mask is
// two array operations in the reference (sampling.py:24-26)
__device__ __forceinline__ float sub_product(float f, float a, float b) {
#pragma clang fp contract(off)
  const float p = a * b;
  return f - p;
}

// The sampler never sorts a row.  Both of its questions - where does the running softmax mass first exceed top_p,
// and which token does u * total land on - ask for the first rank of the descending order at which a running
// sum of non-negative weights exceeds a threshold, and so does top_k with unit weights.  Each is answered by
// selection: a histogram of the weights over 4096 buckets that respect the order, a scan for the bucket where the
// running sum crosses, and then the exact key among the few tokens of that bucket.
// Weights are accumulated as integers (the float64 weight, at most 1, times 2^62, in 96 bits): integer sums do not
// depend on the order of the atomic adds, so a row gives the same token on every run, and the sum of a bucket is
// exactly the sum of its members, so the crossing found in the histogram is always found again inside the bucket.
// A weight below 2^-62 counts as 0; a sum over 65536 tokens is therefore within 2^-46 of the float64 one, the same
// order as the rounding of a sequential float64 sum.
namespace sel {
constexpr int NB = 4096;         // buckets per pass
constexpr int LIST_CAP = 1024;   // keys of the crossing bucket kept in LDS
constexpr double Q_ZERO = -43.0; // exp(t) * 2^62 < 1 below this

struct acc {                     // 96-bit unsigned
  uint64_t lo;
  uint32_t hi;
};
__device__ __forceinline__ acc add(acc a, acc b) {
  acc r;
  r.lo = a.lo + b.lo;
  r.hi = a.hi + b.hi + (r.lo < a.lo ? 1u : 0u);
  return r;
}
__device__ __forceinline__ bool gt(acc a, acc b) { return a.hi != b.hi ? a.hi > b.hi : a.lo > b.lo; }
__device__ __forceinline__ double to_double(acc a) { return (double)a.hi * 0x1p64 + (double)a.lo; }
__device__ __forceinline__ acc from_double(double d) {   // 0 <= d < 2^96
  acc r;
  r.hi = (uint32_t)(d * 0x1p-64);
  r.lo = (uint64_t)(d - (double)r.hi * 0x1p64);
  return r;
}
// Copies the compiler knows nothing about: what one pass derives from a logit (its key, its bucket, whether its
// token exists) is computed again in the next pass instead of being kept - fifty of each per thread would not fit
// the register file.
__device__ __forceinline__ float opaque(float x) {
  asm volatile("" : "+v"(x));
  return x;
}
__device__ __forceinline__ int opaque(int x) {
  asm volatile("" : "+v"(x));
  return x;
}
// A constant the compiler has to keep in scalar registers (it would otherwise copy it into vector registers
// in front of every multiply-add that uses it).
__device__ __forceinline__ double scalar_const(double c) {
  asm volatile("" : "+s"(c));
  return c;
}
// floor(exp(t) * 2^62) for -43 <= t <= 0, as the integer weight of a token: t = k ln 2 + r with |r| <= ln 2 / 2, the
// Taylor polynomial of degree 13 for exp(r) (truncation error (ln 2 / 2)^14 / 14! = 4e-18), scaled by 2^(k + 62).
struct exp_q {
  double log2e, ln2_hi, ln2_lo, c[12];
  __device__ __forceinline__ exp_q() {
    log2e = scalar_const(0x1.71547652b82fep+0);
    ln2_hi = scalar_const(-0x1.62e42fefa39efp-1);
    ln2_lo = scalar_const(-0x1.abc9e3b39803fp-56);
    double f = 1.0;
    for (int i = 0; i < 12; ++i) {            // c[i] = 1 / (i + 2)!
      f *= (double)(i + 2);
      c[i] = scalar_const(1.0 / f);
    }
  }
  __device__ __forceinline__ uint64_t operator()(double t) const {
    const double kd = __builtin_rint(t * log2e);
    double r = __builtin_fma(kd, ln2_hi, t);
    r = __builtin_fma(kd, ln2_lo, r);
    double p = c[11];
#pragma unroll
    for (int i = 10; i >= 0; --i) p = __builtin_fma(r, p, c[i]);
    p = __builtin_fma(r, p, 1.0);
    p = __builtin_fma(r, p, 1.0);
    return (uint64_t)__builtin_ldexp(p, (int)kd + 62);
  }
};

struct smem {
  uint64_t ha[NB];               // per bucket: sum of the weights' bits 32 and up ...
  uint64_t hb[NB];               // ... and of their low 32 bits (neither can overflow: no carry to pass on)
  uint64_t list[LIST_CAP];
  uint64_t wave_lo[SNT / 64];
  uint32_t wave_hi[SNT / 64];
  float fsh[SNT / 64];
  uint64_t above_lo;
  uint64_t key;
  uint32_t above_hi;
  int digit;
  int n_list;
  int hit;
};

// Bucket of pass 0: the distance below the row maximum in units of 1/scale, descending bucket = descending value.
// Any weakly monotone function of the value would do; scale spreads the part of the row that can carry weight
// over all buckets (the high bits of the float would put half of a row in two or three).
__device__ __forceinline__ int coarse(float l, float l0, float scale) {
  const int c = (int)fminf((l0 - l) * scale, (float)(NB - 1));   // NaN -> NB-1
  return NB - 1 - max(c, 0);
}
__device__ __forceinline__ float coarse_scale(float range) { return (float)(NB - 1) / range; }

template <bool COUNT>
__device__ __forceinline__ void hist_add(smem& S, int b, uint64_t q) {
  if (!COUNT) atomicAdd(reinterpret_cast<unsigned long long*>(&S.ha[b]), (unsigned long long)(q >> 32));
  atomicAdd(reinterpret_cast<unsigned long long*>(&S.hb[b]), (unsigned long long)(q & 0xffffffffull));
}
__device__ __forceinline__ acc bucket(const smem& S, int b) {
  const uint64_t a = S.ha[b], c = S.hb[b];
  acc r;
  r.lo = (a << 32) + c;
  r.hi = (uint32_t)(a >> 32) + (r.lo < c ? 1u : 0u);
  return r;
}

struct scan_t {
  acc s[4];      // running sums over this thread's four buckets, in descending bucket order
  acc before;    // sum of the buckets ahead of them
  acc grand;     // sum of all buckets
};
// thread t owns buckets NB-1-4t .. NB-4-4t
__device__ __forceinline__ scan_t scan_hist(smem& S) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  scan_t r;
  acc run{0, 0};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    run = add(run, bucket(S, NB - 1 - (4 * tid + j)));
    r.s[j] = run;
  }
  acc inc = run;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    acc t;
    t.lo = __shfl_up((unsigned long long)inc.lo, o);
    t.hi = __shfl_up(inc.hi, o);
    if (lane >= o) inc = add(inc, t);
  }
  acc ex;
  ex.lo = __shfl_up((unsigned long long)inc.lo, 1);
  ex.hi = __shfl_up(inc.hi, 1);
  if (lane == 0) ex = acc{0, 0};
  if (lane == 63) { S.wave_lo[wave] = inc.lo; S.wave_hi[wave] = inc.hi; }
  __syncthreads();
  acc base{0, 0}, grand{0, 0};
  for (int w = 0; w < SNT / 64; ++w) {
    const acc t{S.wave_lo[w], S.wave_hi[w]};
    if (w < wave) base = add(base, t);
    grand = add(grand, t);
  }
  r.before = add(base, ex);
  r.grand = grand;
  return r;
}
// The bucket in which `above` + running sum first exceeds T, if any: returns its index (-1: none) and moves `above`
// to the sum ahead of it.  All threads return the same answer.
__device__ __forceinline__ int pick(smem& S, const scan_t& sc, acc& above, acc T) {
  const int tid = threadIdx.x;
  const acc base = add(above, sc.before);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const acc excl = j ? add(base, sc.s[j - 1]) : base;
    const acc incl = add(base, sc.s[j]);
    if (!gt(excl, T) && gt(incl, T)) {
      S.digit = NB - 1 - (4 * tid + j);
      S.above_lo = excl.lo;
      S.above_hi = excl.hi;
    }
  }
  __syncthreads();
  const int d = S.digit;
  if (d >= 0) above = acc{S.above_lo, S.above_hi};
  __syncthreads();
  return d;
}
__device__ __forceinline__ void clear_hist(smem& S) {
  for (int i = threadIdx.x; i < NB; i += SNT) { S.ha[i] = 0; S.hb[i] = 0; }
  if (threadIdx.x == 0) { S.digit = -1; S.hit = 0; }
}
__device__ __forceinline__ uint64_t readlane_u64(uint64_t v, int j) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, j);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), j);
  return ((uint64_t)hi << 32) | lo;
}

// First key of the descending order at which the running sum of wq(l, id, key) exceeds thr(total) (a double in the
// same 2^-62 units; negative: the first key with a weight; NaN or no crossing: returns false).  l0 is the row
// maximum, scale the bucket width of pass 0.  COUNT: the weights are 0 or 1.
template <int NT_MAX, bool COUNT, class WQ, class THR>
__device__ __forceinline__ bool select(smem& S, const float (&l)[NT_MAX], int V, float l0, float scale, WQ wq, THR thr,
                                       uint64_t& key_out) {
  const int tid = threadIdx.x;
  // ---- pass 0: every token of the row into its bucket
  clear_hist(S);
  if (tid == 0) S.n_list = 0;
  __syncthreads();
#pragma unroll
  for (int n = 0; n < NT_MAX; ++n) {
    const int id = opaque(tid) + n * SNT;
    if (id < V) {
      const float x = opaque(l[n]);
      const uint64_t q = wq(x, (uint32_t)id, sort_key(x, (uint32_t)id));
      if (q) hist_add<COUNT>(S, coarse(x, l0, scale), q);
    }
    __builtin_amdgcn_sched_barrier(0);   // one token at a time: fifty exponentials in flight would spill
  }
  __syncthreads();
  scan_t sc = scan_hist(S);
  const double td = thr(to_double(sc.grand));
  if (!(td < 0x1p95)) return false;               // NaN or beyond any sum (every thread has the same td)
  const acc T = td > 0.0 ? from_double(td) : acc{0, 0};
  acc above{0, 0};
  const int g = pick(S, sc, above, T);
  if (g < 0) return false;
  // ---- the keys of that bucket go to LDS if they fit
#pragma unroll
  for (int n = 0; n < NT_MAX; ++n) {
    const int id = opaque(tid) + n * SNT;
    const float x = opaque(l[n]);
    if (id < V && coarse(x, l0, scale) == g) {
      const int at = atomicAdd(&S.n_list, 1);
      if (at < LIST_CAP) S.list[at] = sort_key(x, (uint32_t)id);
    }
  }
  __syncthreads();
  const int n_list = __builtin_amdgcn_readfirstlane(S.n_list);
  if (n_list <= 64) {
    // ---- one wavefront, one key per lane: the sum ahead of a key is the sum over the keys above it
    if (tid < 64) {
      uint64_t key = 0, q = 0;
      if (tid < n_list) {
        key = S.list[tid];
        q = wq(key_value(key), (uint32_t)(key & 0xffffu), key);
      }
      acc ahead = above;
      for (int j = 0; j < n_list; ++j) {
        const uint64_t kj = readlane_u64(key, j), qj = readlane_u64(q, j);
        const acc t = add(ahead, acc{qj, 0});
        if (kj > key) ahead = t;
      }
      if (tid < n_list && !gt(ahead, T) && gt(add(ahead, acc{q, 0}), T)) { S.key = key; S.hit = 1; }
    }
    __syncthreads();
    if (!S.hit) return false;                     // cannot happen: the sums are exact
    key_out = S.key;
    __syncthreads();
    return true;
  }
  // ---- a crowded bucket (many equal or nearly equal logits): four 12-bit digits of the key inside it
  uint64_t prefix = 0;
  for (int d = 1; d <= 4; ++d) {
    const int shift = 48 - 12 * d;
    clear_hist(S);
    __syncthreads();
    if (n_list <= LIST_CAP) {
      for (int i = tid; i < n_list; i += SNT) {
        const uint64_t key = S.list[i];
        if ((key >> (shift + 12)) == prefix) {
          const uint64_t q = wq(key_value(key), (uint32_t)(key & 0xffffu), key);
          if (q) hist_add<COUNT>(S, (int)((key >> shift) & (NB - 1)), q);
        }
      }
    } else {
#pragma unroll
      for (int n = 0; n < NT_MAX; ++n) {
        const int id = opaque(tid) + n * SNT;
        const float x = opaque(l[n]);
        if (id < V && coarse(x, l0, scale) == g) {
          const uint64_t key = sort_key(x, (uint32_t)id);
          if ((key >> (shift + 12)) == prefix) {
            const uint64_t q = wq(x, (uint32_t)id, key);
            if (q) hist_add<COUNT>(S, (int)((key >> shift) & (NB - 1)), q);
          }
        }
      }
    }
    __syncthreads();
    sc = scan_hist(S);
    const int dg = pick(S, sc, above, T);
    if (dg < 0) return false;                     // cannot happen: the sums are exact
    prefix = (prefix << 12) | (uint64_t)dg;
  }
  key_out = prefix;
  return true;
}

__device__ __forceinline__ float block_max_f(smem& S, float v) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  __syncthreads();
  if (lane == 0) S.fsh[wave] = v;
  __syncthreads();
  float t = S.fsh[0];
  for (int w = 1; w < SNT / 64; ++w) t = fmaxf(t, S.fsh[w]);
  return t;
}
__device__ __forceinline__ double block_max_d(smem& S, double v) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  double* sh = reinterpret_cast<double*>(S.wave_lo);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmax(v, __shfl_xor(v, o));
  __syncthreads();
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  double t = sh[0];
  for (int w = 1; w < SNT / 64; ++w) t = fmax(t, sh[w]);
  return t;
}
// minimum (want_max = false) or maximum of a 64-bit key over the workgroup
__device__ __forceinline__ uint64_t block_ext_u64(smem& S, uint64_t v, bool want_max) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint64_t t = __shfl_xor((unsigned long long)v, o);
    v = want_max ? (t > v ? t : v) : (t < v ? t : v);
  }
  __syncthreads();
  if (lane == 0) S.wave_lo[wave] = v;
  __syncthreads();
  uint64_t r = S.wave_lo[0];
  for (int w = 1; w < SNT / 64; ++w) r = want_max ? (S.wave_lo[w] > r ? S.wave_lo[w] : r) : (S.wave_lo[w] < r ? S.wave_lo[w] : r);
  return r;
}
}  // namespace sel

constexpr size_t SEL_LDS_BYTES = sizeof(sel::smem);

// One workgroup of 1024 threads per row; thread t keeps tokens t, t + 1024, ... in registers for every pass.
template <int NT_MAX>        // tokens per thread: V <= 1024 * NT_MAX
__global__ __launch_bounds__(SNT) void nucleus_kernel(const float* __restrict__ logits, int V,
                                                      const double* __restrict__ top_p, const double* __restrict__ temp,
                                                      const int32_t* __restrict__ top_k,
                                                      const double* __restrict__ uniforms, int64_t ld_u,
                                                      int32_t* __restrict__ tok, int32_t* __restrict__ out_tokens,
                                                      int64_t ld_tokens, int32_t* __restrict__ pos,
                                                      const int32_t* __restrict__ pos_start,
                                                      uint8_t* __restrict__ keep_mask, float* __restrict__ filtered,
                                                      const mtj_next_embed ne) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  sel::smem& S = *reinterpret_cast<sel::smem*>(smem_raw);
  const int b = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + (int64_t)b * V;
  const int step = pos[b] - pos_start[b];
  const double tp = top_p[b], tmp = temp[b], u = uniforms[(int64_t)b * ld_u + step];
  const int kk = top_k ? top_k[b] : 0x7fffffff;

  float l[NT_MAX];
#pragma unroll
  for (int n = 0; n < NT_MAX; ++n) l[n] = row[min(tid + n * SNT, V - 1)];     // all loads in flight together
  float lmax = -INFINITY, lmin = INFINITY;
#pragma unroll
  for (int n = 0; n < NT_MAX; ++n) {
    const bool live = tid + n * SNT < V;
    lmin = fminf(lmin, live ? l[n] : INFINITY);
    l[n] = live ? l[n] : -INFINITY;
    lmax = fmaxf(lmax, l[n]);
  }
  const float l0 = sel::block_max_f(S, lmax);
  const float spread = l0 + sel::block_max_f(S, -lmin);      // row maximum - row minimum
  const double l0d = (double)l0;
  const sel::exp_q expq;

  // ---- top_p: rank j > 0 leaves the nucleus when the softmax mass of ranks [0, j-1] exceeds top_p (sampling.py:28-30),
  // that is, every key below the one at which the running mass first exceeds it
  uint64_t key_p = 0, key_k = 0;
  const bool cut_p = sel::select<NT_MAX, false>(
      S, l, V, l0, sel::coarse_scale(fminf(spread, 43.0f)),
      [&](float x, uint32_t, uint64_t) {
        const double t = (double)x - l0d;
        return t < sel::Q_ZERO ? (uint64_t)0 : expq(t);
      },
      [&](double total) { return tp * total; }, key_p);
  // ---- top_k: ranks >= top_k, every key below the one of rank top_k - 1
  bool cut_k = false;
  if (kk >= 1 && kk < V)
    cut_k = sel::select<NT_MAX, true>(
        S, l, V, l0, sel::coarse_scale(fminf(spread, 1e4f)), [](float, uint32_t, uint64_t) { return (uint64_t)1; },
        [&](double) { return (double)(kk - 1); }, key_k);
  auto filtered_of = [&](float x, uint32_t id, uint64_t key) {
    float f = x;
    if (kk < 1 || (cut_k && key < key_k)) f = sub_product(f, 1e10f, (float)id);   // top-k quirk: subtracts 1e10 * token id
    return f - ((cut_p && key < key_p) ? 1e10f : 0.0f);
  };

  // ---- the filter's output, when asked for
  if (filtered || keep_mask) {
#pragma unroll
    for (int n = 0; n < NT_MAX; ++n) {
      const int id = sel::opaque(tid) + n * SNT;
      if (id < V) {
        const float x = sel::opaque(l[n]);
        const float f = filtered_of(x, (uint32_t)id, sort_key(x, (uint32_t)id));
        if (filtered) filtered[(int64_t)b * V + id] = f;
        if (keep_mask) keep_mask[(int64_t)b * V + id] = (f == x) ? 1 : 0;
      }
    }
  }
  // ---- the largest filtered / temp
  double tmax;
  if (tmp > 0.0 && kk >= 1) {
    // the filter only lowers a logit and leaves rank 0 alone, and x -> x / temp is monotone
    tmax = l0d / tmp;
  } else {                    // top_k < 1 penalises every rank, temp <= 0 or NaN turns the order around: token by token
    double m = -INFINITY;
#pragma unroll
    for (int n = 0; n < NT_MAX; ++n) {
      const int id = sel::opaque(tid) + n * SNT;
      const float x = sel::opaque(l[n]);
      if (id < V) m = fmax(m, (double)filtered_of(x, (uint32_t)id, sort_key(x, (uint32_t)id)) / tmp);
    }
    tmax = sel::block_max_d(S, m);
  }

  // ---- inverse-CDF draw over exp(filtered / temp - max) in descending order of the raw logits
  // In the usual case a token the filter touched has no weight at all (its filtered / temp is 1e10 / temp lower,
  // far below the 2^-62 that still counts) and needs no arithmetic; token 0 is exempt from the top-k penalty, which
  // multiplies by the token id.
  const bool plain = tmp > 0.0 && tmp <= 1e6 && kk >= 1 && fabsf(l0) <= 1e6f;
  uint64_t key_t = 0;
  const bool hit = sel::select<NT_MAX, false>(
      S, l, V, l0, sel::coarse_scale(fminf(spread, tmp > 0.0 ? (float)fmin(43.0 * fmax(tmp, 1.0), 1e30) : 1e30f)),
      [&](float x, uint32_t id, uint64_t key) {
        double t;
        if (plain) {
          if ((cut_p && key < key_p) || (cut_k && key < key_k && id != 0)) return (uint64_t)0;
          t = (double)x / tmp - tmax;
        } else {
          t = (double)filtered_of(x, id, key) / tmp - tmax;
        }
        return (t < sel::Q_ZERO || !(t <= 0.0)) ? (uint64_t)0 : expq(t);
      },
      [&](double total) { return u * total; }, key_t);
  if (!hit) {
    // u * total is not exceeded: the last rank with a weight (exp(x) is exactly 0 in float64 below -745.14), else rank 0
    uint64_t lowest = ~0ull, top = 0;
#pragma unroll
    for (int n = 0; n < NT_MAX; ++n) {
      const int id = sel::opaque(tid) + n * SNT;
      if (id < V) {
        const float x = sel::opaque(l[n]);
        const uint64_t key = sort_key(x, (uint32_t)id);
        top = key > top ? key : top;
        const double t = (double)filtered_of(x, (uint32_t)id, key) / tmp - tmax;
        if (t >= -746.0 && exp(t) > 0.0) lowest = key < lowest ? key : lowest;
      }
    }
    lowest = sel::block_ext_u64(S, lowest, false);
    top = sel::block_ext_u64(S, top, true);
    key_t = lowest != ~0ull ? lowest : top;
  }
  const int id = (int)(key_t & 0xffffu);
  if (tid == 0) {
    tok[b] = id;
    if (out_tokens) out_tokens[(int64_t)b * ld_tokens + step] = id;
    pos[b] += 1;
  }
  embed_next(ne, b, V, id);
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

// The selection kernel keeps everything in registers and LDS; the work buffer of the ABI is not used by it.
extern "C" int64_t mtj_sample_work_bytes(int64_t B, int64_t V) {
  (void)B; (void)V;
  return 256;
}

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
  static mtj_device_once once50, once64;
  if (int rc = mtj_allow_lds(once50, "mtj_sample_nucleus", &nucleus_kernel<50>, SEL_LDS_BYTES)) return rc;
  if (int rc = mtj_allow_lds(once64, "mtj_sample_nucleus", &nucleus_kernel<64>, SEL_LDS_BYTES)) return rc;
  if (V <= SNT * 50)      // GPT-J's 50400-entry vocabulary
    nucleus_kernel<50><<<(unsigned)B, SNT, SEL_LDS_BYTES, s>>>(logits, (int)V, top_p, temp, top_k, uniforms, ld_u, tok, out_tokens,
                                                   ld_tokens, pos, pos_start, keep_mask, filtered, ne);
  else
    nucleus_kernel<64><<<(unsigned)B, SNT, SEL_LDS_BYTES, s>>>(logits, (int)V, top_p, temp, top_k, uniforms, ld_u, tok, out_tokens,
                                                   ld_tokens, pos, pos_start, keep_mask, filtered, ne);
  return mtj_check_launch("mtj_sample_nucleus");
}

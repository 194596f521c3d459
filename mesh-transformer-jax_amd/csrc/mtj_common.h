// Shared host/device helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <atomic>
#include <mutex>
#include "mtj_abi.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16_t;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uint32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t uint32x2 __attribute__((ext_vector_type(2)));

#define MTJ_WAVE 64

// ---------------------------------------------------------------- error plumbing (host)
int mtj_fail(int code, const char* fmt, ...);
int mtj_check_launch(const char* what);

#define MTJ_REQUIRE(cond, code, ...) \
  do {                               \
    if (!(cond)) return mtj_fail(code, __VA_ARGS__); \
  } while (0)

static inline bool mtj_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Set-up that has to run once per device and process (kernel attributes, symbol addresses): f(device) runs under a
// lock the first time the calling thread's current device reaches this point; later calls cost one hipGetDevice
// and one atomic load.  Thread-safe; a failed f is retried by the next call.
constexpr int MTJ_MAX_DEVICES = 64;
struct mtj_device_once {
  std::atomic<uint64_t> done{0};
  std::mutex mu;
};
template <class F>
static inline int mtj_once_per_device(mtj_device_once& o, const char* who, F&& f) {
  int dev = 0;
  const hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  if (dev < 0 || dev >= MTJ_MAX_DEVICES) return mtj_fail(MTJ_ELIMIT, "%s: device index %d is beyond %d", who, dev, MTJ_MAX_DEVICES);
  const uint64_t bit = 1ull << dev;
  if (o.done.load(std::memory_order_acquire) & bit) return MTJ_OK;
  std::lock_guard<std::mutex> guard(o.mu);
  if (o.done.load(std::memory_order_relaxed) & bit) return MTJ_OK;
  const int rc = f(dev);
  if (rc == MTJ_OK) o.done.fetch_or(bit, std::memory_order_release);
  return rc;
}

// Raises the dynamic-LDS limit of `kernel` once per device.
template <class K>
static inline int mtj_allow_lds(mtj_device_once& o, const char* who, K kernel, size_t bytes) {
  return mtj_once_per_device(o, who, [&](int) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "%s: hipFuncSetAttribute: %s", who, hipGetErrorString(e));
    return (int)MTJ_OK;
  });
}

// ---------------------------------------------------------------- device helpers
// bf16 <-> f32.  Rounding to bf16 is round-to-nearest-even (what jnp.astype(bfloat16) does).
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t hi16) { return __uint_as_float(hi16 << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }
// gfx950 converts in hardware (v_cvt_pk_bf16_f32, round to nearest even)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  const __bf16 b = (__bf16)f;
  return (uint32_t)__builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const bf16x2 r = __builtin_convertvector(f32x2{lo, hi}, bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}

// float32 -> float16, round to nearest even, saturating at the largest finite value instead of overflowing to inf
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  const f16_t h = (f16_t)__builtin_amdgcn_fmed3f(f, -65504.f, 65504.f);
  return (uint32_t)__builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  const f16x2 r = {(f16_t)__builtin_amdgcn_fmed3f(lo, -65504.f, 65504.f), (f16_t)__builtin_amdgcn_fmed3f(hi, -65504.f, 65504.f)};
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ float f16_lo(uint32_t packed) { return (float)__builtin_bit_cast(f16x2, packed).x; }
__device__ __forceinline__ float f16_hi(uint32_t packed) { return (float)__builtin_bit_cast(f16x2, packed).y; }
// two floats -> one 32-bit word of two 16-bit elements of run-time type dtype (MTJ_BF16 or MTJ_F16)
__device__ __forceinline__ uint32_t pack_16x2(float lo, float hi, int dtype) {
  return dtype == MTJ_F16 ? pack_f16x2(lo, hi) : pack_bf16x2(lo, hi);
}
// the same with the type known at compile time
template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float lo, float hi) { return pack_bf16x2(lo, hi); }
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float lo, float hi) { return pack_f16x2(lo, hi); }
template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t w);
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t w);
template <> __device__ __forceinline__ float unpack_lo<bf16_t>(uint32_t w) { return bf16_lo(w); }
template <> __device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t w) { return bf16_hi(w); }
template <> __device__ __forceinline__ float unpack_lo<f16_t>(uint32_t w) { return f16_lo(w); }
template <> __device__ __forceinline__ float unpack_hi<f16_t>(uint32_t w) { return f16_hi(w); }

static inline int mtj_elem_size(int dtype) { return dtype == MTJ_F32 ? 4 : 2; }
static inline bool mtj_is_dtype(int dtype) { return dtype == MTJ_F32 || dtype == MTJ_BF16 || dtype == MTJ_F16; }

template <typename T> struct elem;
template <> struct elem<float> {
  static constexpr int dtype = MTJ_F32;
  __device__ static __forceinline__ float load(const float* p) { return *p; }
  __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct elem<bf16_t> {
  static constexpr int dtype = MTJ_BF16;
  __device__ static __forceinline__ float load(const bf16_t* p) {
    return bf16_bits_to_f32(*reinterpret_cast<const uint16_t*>(p));
  }
  __device__ static __forceinline__ void store(bf16_t* p, float v) {
    *reinterpret_cast<uint16_t*>(p) = (uint16_t)f32_to_bf16_bits(v);
  }
};

template <> struct elem<f16_t> {
  static constexpr int dtype = MTJ_F16;
  __device__ static __forceinline__ float load(const f16_t* p) { return (float)*p; }
  __device__ static __forceinline__ void store(f16_t* p, float v) {
    *reinterpret_cast<uint16_t*>(p) = (uint16_t)f32_to_f16_bits(v);
  }
};

// store a float into a buffer whose element type is only known at run time
__device__ __forceinline__ void store_as(void* base, int64_t idx, float v, int dtype) {
  if (dtype == MTJ_F32) reinterpret_cast<float*>(base)[idx] = v;
  else if (dtype == MTJ_F16) reinterpret_cast<uint16_t*>(base)[idx] = (uint16_t)f32_to_f16_bits(v);
  else reinterpret_cast<uint16_t*>(base)[idx] = (uint16_t)f32_to_bf16_bits(v);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

// ---------------------------------------------------------------- cached K/V rows
template <typename T> struct kvrow;   // one 16-byte piece of a cached row -> EPC floats
template <> struct kvrow<float> {
  static constexpr int EPC = 4;
  __device__ static __forceinline__ void get(const uint32x4& w, float* f) {
    f[0] = __uint_as_float(w.x); f[1] = __uint_as_float(w.y); f[2] = __uint_as_float(w.z); f[3] = __uint_as_float(w.w);
  }
};
template <> struct kvrow<bf16_t> {
  static constexpr int EPC = 8;
  __device__ static __forceinline__ void get(const uint32x4& w, float* f) {
    f[0] = bf16_lo(w.x); f[1] = bf16_hi(w.x); f[2] = bf16_lo(w.y); f[3] = bf16_hi(w.y);
    f[4] = bf16_lo(w.z); f[5] = bf16_hi(w.z); f[6] = bf16_lo(w.w); f[7] = bf16_hi(w.w);
  }
};
template <> struct kvrow<f16_t> {
  static constexpr int EPC = 8;
  __device__ static __forceinline__ void get(const uint32x4& w, float* f) {
    f[0] = f16_lo(w.x); f[1] = f16_hi(w.x); f[2] = f16_lo(w.y); f[3] = f16_hi(w.y);
    f[4] = f16_lo(w.z); f[5] = f16_hi(w.z); f[6] = f16_lo(w.w); f[7] = f16_hi(w.w);
  }
};

// ---------------------------------------------------------------- merge of one-token attention partials
// Partials of one (sequence, head): wb[s * stride] = {max, sum, -, -, V[dh]} for key range s < S <= 8.
// Returns elements e .. e+3 of sum_s exp(max_s - max) V_s / sum_s exp(max_s - max) sum_s.  The ranges are taken four at
// a time with a running maximum (four vectors and eight statistics in registers at once: the callers have their
// weight tiles in registers too); inside a batch every load is issued before the first is used.  Ranges beyond S
// read range S-1 again with weight 0.
constexpr int MTJ_DEC_MAXS = 8;
constexpr int MTJ_DEC_PAD = 4;
__device__ __forceinline__ floatx4 mtj_merge_partials(const float* __restrict__ wb, int S, int stride, int e) {
  float mm = -INFINITY, lt = 0.f;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < S; s0 += 4) {
    float m[4], l[4];
    floatx4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float* p = wb + (int64_t)(s0 + i < S ? s0 + i : S - 1) * stride;
      m[i] = p[0];
      l[i] = p[1];
      v[i] = *reinterpret_cast<const floatx4*>(p + MTJ_DEC_PAD + e);
    }
    float mb = mm;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (s0 + i >= S) m[i] = -INFINITY;
      mb = fmaxf(mb, m[i]);
    }
    if (mb == -INFINITY) continue;                                      // only empty ranges so far
    const float r = (mm == -INFINITY) ? 0.f : __expf(mm - mb);
    lt *= r;
    acc *= r;
    mm = mb;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float f = (m[i] == -INFINITY) ? 0.f : __expf(m[i] - mm);    // an empty range has max -inf
      lt = fmaf(f, l[i], lt);
      acc += f * v[i];
    }
  }
  const float inv = lt > 0.f ? 1.0f / lt : 0.f;
  return acc * inv;
}

// Exchange between the two 32-lane halves of a wavefront without going through LDS: after the swap `a` holds the
// lower half's values in both halves and `b` the upper half's, so op(a, b) is the reduction over lanes l and l ^ 32.
__device__ __forceinline__ void swap_halves(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float max_halves(float x) {
  float a = x, b = x;
  swap_halves(a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float sum_halves(float x) {
  float a = x, b = x;
  swap_halves(a, b);
  return a + b;
}

// destination of a global -> LDS load (buffer_load ... lds)
typedef __attribute__((address_space(3))) void* lds_ptr;

// s_waitcnt immediates that constrain one counter only (gfx9 encoding: vmcnt [3:0] and [15:14], expcnt [6:4],
// lgkmcnt [11:8])
constexpr int wait_vmcnt(int n) { return (n & 0xf) | (((n >> 4) & 3) << 14) | (0x7 << 4) | (0xf << 8); }
constexpr int wait_lgkmcnt(int n) { return 0xf | (3 << 14) | (0x7 << 4) | ((n & 0xf) << 8); }

// jax.nn.gelu(approximate=True): 0.5 x (1 + tanh(u)), u = sqrt(2/pi) (x + 0.044715 x^3).
// 0.5 (1 + tanh(u)) = 1 / (1 + exp(-2u)) = 1 / (1 + 2^(x (k1 + k2 x^2))) with k1 = -2 log2(e) sqrt(2/pi) and
// k2 = 0.044715 k1: three multiplications, one fma, one addition, v_exp_f32 and v_rcp_f32 (about 1 ulp each).  The
// plain spelling x / (1 + expf(-2u)) compiles to a correctly rounded division of about twenty instructions, which made
// the fc_in columns of the prefill epilogue twice as expensive.  For very negative x the power overflows to +inf and the
// result is -0; for large x it underflows to 0 and the result is x.
__device__ __forceinline__ float gelu_tanh(float x) {
  const float k1 = -2.3022082f;        // -2 * 1.4426950408889634 * 0.7978845608028654
  const float k2 = -0.10294324f;       // k1 * 0.044715
  const float p = fmaf(x * x, k2, k1);
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * p));
}

// ---------------------------------------------------------------- fused input-projection epilogue
// One output element (row m, column n) of q|v|k|fc_in, in two halves so that a bandwidth-bound caller can
// issue the loads (position, sin/cos, bias) long before the accumulator is ready: inproj_prepare does every
// global read, inproj_finish only arithmetic and stores.  `own` is the accumulator of column n, `partner`
// that of column n ^ 1 of the same row (the interleaved rotation of layers.py:137-148:
// out[2i] = x[2i] cos - x[2i+1] sin, out[2i+1] = x[2i+1] cos + x[2i] sin).
struct inproj_pre {
  int kind;        // 0 q, 1 v, 2 k, 3 fc_in, -1 nothing to store (padding row)
  float sn, cs;    // rotation of this element (cs = 1, sn = 0 outside the rotary dims); kind 3: cs is the fc_in bias
  int64_t idx;     // destination element in q / k_cache / v_cache / act
  int pos_t;       // kind 1 with a transposed copy wanted: the position, i.e. the column of v_t; else -1
};                 // (kept small: these registers stay live across the whole weight stream of a GEMV)

__device__ __forceinline__ inproj_pre inproj_prepare(const mtj_inproj& ip, const float* __restrict__ b1, int64_t m,
                                                     int64_t n) {
  inproj_pre p;
  p.sn = 0.f; p.cs = 1.f; p.idx = 0; p.pos_t = -1;
  const int d = ip.n_heads * ip.d_head;
  const int b = (int)(m / ip.Tp), t = (int)(m - (int64_t)b * ip.Tp);
  if (n >= 3 * (int64_t)d) {  // fc_in -> gelu
    const int64_t c = n - 3 * (int64_t)d;
    p.kind = 3;
    p.cs = b1[c];
    p.idx = m * ip.ld_act + d + c;
    return p;
  }
  const int pos = ip.pos0[b] + t;
  if (pos < 0) { p.kind = -1; return p; }  // left padding: nothing reaches the cache
  const int seg = (int)(n / d);            // 0 q, 1 v, 2 k
  const int c = (int)(n - (int64_t)seg * d);
  const int h = c / ip.d_head, e = c - h * ip.d_head;
  p.kind = seg;
  if (seg != 1 && e < ip.rotary_dims) {
    const int pp = pos < ip.max_pos ? pos : ip.max_pos - 1;
    const float sn = ip.sin_tab[(int64_t)pp * (ip.rotary_dims / 2) + (e >> 1)];
    p.cs = ip.cos_tab[(int64_t)pp * (ip.rotary_dims / 2) + (e >> 1)];
    p.sn = (e & 1) ? sn : -sn;
  }
  if (seg == 0) {
    p.idx = (((int64_t)b * ip.n_heads + h) * ip.Tp + t) * ip.d_head + e;
  } else {
    const int slot = pos % ip.Tcap;
    p.idx = (((int64_t)b * ip.n_heads + h) * ip.Tcap + slot) * ip.d_head + e;
    if (seg == 1 && ip.v_t && pos < ip.ldvt) p.pos_t = pos;   // transposed copy, indexed by position like the cache
  }
  return p;
}

// The same two halves for row 0 of a one-token call (Tp == 1: sequence 0, token 0, no transposed copy of V), as the
// matrix-vector kernels need them: 32-bit arithmetic, a single division, four registers.  Same values; the
// destination index must fit 31 bits (n_heads * Tcap * d_head and ld_act below 2^31, which the callers check).
struct inproj_tok {
  int kind;        // as inproj_pre
  float sn, cs;
  int idx;
};

__device__ __forceinline__ inproj_tok inproj_prepare_token(const mtj_inproj& ip, const float* __restrict__ b1, int n) {
  inproj_tok p;
  p.sn = 0.f; p.cs = 1.f; p.idx = 0;
  const int d = ip.n_heads * ip.d_head;
  if (n >= 3 * d) {  // fc_in -> gelu
    const int c = n - 3 * d;
    p.kind = 3;
    p.cs = b1[c];
    p.idx = d + c;
    return p;
  }
  const int pos = ip.pos0[0];
  if (pos < 0) { p.kind = -1; return p; }
  const int seg = (n >= d ? 1 : 0) + (n >= 2 * d ? 1 : 0);   // 0 q, 1 v, 2 k
  const int c = n - seg * d;
  const int h = (int)((unsigned)c / (unsigned)ip.d_head), e = c - h * ip.d_head;
  p.kind = seg;
  if (seg != 1 && e < ip.rotary_dims) {
    const int pp = pos < ip.max_pos ? pos : ip.max_pos - 1;
    const float sn = ip.sin_tab[(int64_t)pp * (ip.rotary_dims / 2) + (e >> 1)];
    p.cs = ip.cos_tab[(int64_t)pp * (ip.rotary_dims / 2) + (e >> 1)];
    p.sn = (e & 1) ? sn : -sn;
  }
  if (seg == 0) p.idx = c;
  else p.idx = (h * ip.Tcap + (int)((unsigned)pos % (unsigned)ip.Tcap)) * ip.d_head + e;
  return p;
}

__device__ __forceinline__ void inproj_finish_token(const mtj_inproj& ip, const inproj_tok& p, float own, float partner) {
  if (p.kind < 0) return;
  if (p.kind == 3) {
    store_as(ip.act, p.idx, gelu_tanh(own + p.cs), ip.act_dtype);
    return;
  }
  const float val = own * p.cs + partner * p.sn;
  if (p.kind == 0) store_as(ip.q, p.idx, val, ip.q_dtype);
  else store_as(p.kind == 1 ? ip.v_cache : ip.k_cache, p.idx, val, ip.kv_dtype);
}

__device__ __forceinline__ void inproj_finish(const mtj_inproj& ip, const inproj_pre& p, float own, float partner) {
  const int kv_dtype = ip.kv_dtype;
  if (p.kind < 0) return;
  if (p.kind == 3) {
    store_as(ip.act, p.idx, gelu_tanh(own + p.cs), ip.act_dtype);
    return;
  }
  const float val = own * p.cs + partner * p.sn;
  if (p.kind == 0) {
    store_as(ip.q, p.idx, val, ip.q_dtype);
  } else {
    store_as(p.kind == 1 ? ip.v_cache : ip.k_cache, p.idx, val, kv_dtype);
    if (p.pos_t >= 0) {   // idx = ((b*H + h)*Tcap + slot)*dh + e  ->  v_t[((b*H + h)*dh + e)*ldvt + pos]
      const int64_t bh = p.idx / ((int64_t)ip.Tcap * ip.d_head), e = p.idx % ip.d_head;
      store_as(ip.v_t, (bh * ip.d_head + e) * ip.ldvt + p.pos_t, val, kv_dtype);
    }
  }
}

__device__ __forceinline__ void inproj_store(const mtj_inproj& ip, const float* __restrict__ b1, int64_t m, int64_t n,
                                             float own, float partner) {
  inproj_finish(ip, inproj_prepare(ip, b1, m, n), own, partner);
}

// x_next[b, :] = W[token, :] + bias by the whole workgroup (token is uniform): the embedding of the token a sampler
// just chose (EmbeddingShard, layers.py:187-202), which is the input of the next decode step
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

// One whole batch-1 decode step (all layers + logits) as ONE persistent launch: a workgroup per CU, phases
// separated by grid barriers.  Separate launches per GEMV / attention cost ~4.6 us each in ramp, drain and launch
// gap (114 per step); here the first weight tile of the next matrix is requested before a barrier is entered, so
// the memory pipeline keeps streaming while workgroups wait and while the small activation vectors are staged.
//
// Coherence on a multi-die GPU without device-scope fences (which write back a whole L2): everything one phase
// hands to the next (x, q, act, the new K/V row, attention partials) is written and read with agent-scope relaxed
// atomic stores / loads, which bypass the non-coherent L2s; weights and the old K/V rows are ordinary loads.
// Barriers are monotonically counted agent-scope atomics (one counter per group of workgroups, one global),
// zeroed by the caller before the launch; every spin is bounded and a time-out makes all workgroups leave.
#include "mtj_common.h"

namespace {

constexpr int ST_NT = 1024;     // threads per workgroup
constexpr int ST_U = 8;         // 16-byte weight loads in flight per lane
constexpr int ST_CHUNK = 64;    // keys per attention range

__device__ __forceinline__ float ldc(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void stc(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

template <typename T> struct wchunk;
template <> struct wchunk<bf16_t> {
  static constexpr int EPC = 8;
  __device__ static __forceinline__ void fma(const uint32x4& w, const float* __restrict__ xs, float& acc) {
    const floatx4 x0 = *reinterpret_cast<const floatx4*>(xs);
    const floatx4 x1 = *reinterpret_cast<const floatx4*>(xs + 4);
    acc = fmaf(bf16_lo(w.x), x0.x, acc); acc = fmaf(bf16_hi(w.x), x0.y, acc);
    acc = fmaf(bf16_lo(w.y), x0.z, acc); acc = fmaf(bf16_hi(w.y), x0.w, acc);
    acc = fmaf(bf16_lo(w.z), x1.x, acc); acc = fmaf(bf16_hi(w.z), x1.y, acc);
    acc = fmaf(bf16_lo(w.w), x1.z, acc); acc = fmaf(bf16_hi(w.w), x1.w, acc);
  }
  __device__ static __forceinline__ float round(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }
};
template <> struct wchunk<float> {
  static constexpr int EPC = 4;
  __device__ static __forceinline__ void fma(const uint32x4& w, const float* __restrict__ xs, float& acc) {
    const floatx4 x0 = *reinterpret_cast<const floatx4*>(xs);
    acc = fmaf(__uint_as_float(w.x), x0.x, acc); acc = fmaf(__uint_as_float(w.y), x0.y, acc);
    acc = fmaf(__uint_as_float(w.z), x0.z, acc); acc = fmaf(__uint_as_float(w.w), x0.w, acc);
  }
  __device__ static __forceinline__ float round(float v) { return v; }
};

struct step_args {
  mtj_step s;
  float *q, *act, *kv_new, *partials;
  unsigned* sync;               // [0..7]*16: group counters, [8*16]: global counter, [9*16]: failure flag
  int S;                        // attention ranges = ceil(Tcap / 64)
};

// ---- grid barrier number `epoch` (1, 2, ...).  false: timed out (or somebody else did) - leave the kernel.
// `prefetch` requests the first weight tile of the next phase.  It runs after this workgroup's coherent stores have
// completed (the release fence waits for every outstanding memory operation, so a request made earlier would delay
// the arrival) and, for the wavefront that spins, after the spin (loads return in order: its polls would queue
// behind the tile).
template <class F>
__device__ __forceinline__ bool grid_barrier(unsigned* sync, unsigned epoch, F&& prefetch) {
  __shared__ int ok;
  const int wave = threadIdx.x >> 6;
  // every coherent store of this wavefront has been acknowledged by memory before the workgroup arrives (a
  // workgroup-scope fence does not wait for global stores: within a CU they are ordered by the shared L1)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (wave != 0) prefetch();
  if (threadIdx.x == 0) {
    const unsigned nwg = gridDim.x, ngroups = nwg < 8 ? nwg : 8;
    const unsigned g = blockIdx.x % ngroups;
    const unsigned members = nwg / ngroups + (g < nwg % ngroups ? 1u : 0u);
    unsigned* global = sync + 8 * 16;
    unsigned* fail = sync + 9 * 16;
    const unsigned old = __hip_atomic_fetch_add(sync + g * 16, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old + 1 == epoch * members) __hip_atomic_fetch_add(global, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    int good = 0;
    for (int spin = 0; spin < (1 << 22); ++spin) {
      if (__hip_atomic_load(global, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= epoch * ngroups) { good = 1; break; }
      if ((spin & 1023) == 1023 && __hip_atomic_load(fail, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
    }
    if (!good) __hip_atomic_store(fail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ok = good;
  }
  if (wave == 0) prefetch();
  __syncthreads();
  return ok != 0;
}

// ---- rows of a matrix-vector product owned by this wavefront, and its first weight tile
struct row_range { int64_t row0; int nrows; };
__device__ __forceinline__ row_range my_rows(int64_t N, int upw) {
  const int wave = threadIdx.x >> 6, nwaves = ST_NT >> 6;
  const int64_t units = N / upw;
  const int64_t gw = (int64_t)blockIdx.x * nwaves + wave, nw = (int64_t)gridDim.x * nwaves;
  row_range r;
  r.row0 = (units * gw / nw) * upw;
  r.nrows = (int)((units * (gw + 1) / nw) * upw - r.row0);
  return r;
}
template <typename T, bool FULL>
__device__ __forceinline__ void first_tile(const T* W, int K, const row_range& rr, uint32x4 (&w)[ST_U]) {
  constexpr int EPC = wchunk<T>::EPC;
  const int lane = threadIdx.x & 63;
  // unconditional loads (chunks beyond K and wavefronts without rows re-read valid memory): a conditionally
  // defined tile would have to be kept alive, merged and spilled across every phase of the kernel
  const T* rowp = W + (rr.nrows > 0 ? rr.row0 : 0) * K;
#pragma unroll
  for (int u = 0; u < ST_U; ++u) {
    const int k = (u * 64 + lane) * EPC;
    w[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(rowp + (FULL || k < K ? k : 0)));
  }
}
// streams the rows; lane r ends up with the sum of row rr.row0 + r
template <typename T, bool FULL>
__device__ __forceinline__ float stream_rows(const T* W, int K, const row_range& rr, uint32x4 (&w)[ST_U], const float* xs) {
  constexpr int EPC = wchunk<T>::EPC, STEP = 64 * EPC;
  const int lane = threadIdx.x & 63;
  const int tpr = (K + STEP * ST_U - 1) / (STEP * ST_U);
  float mine = 0.f;
  for (int r = 0; r < rr.nrows; ++r) {
    const T* rowp = W + (rr.row0 + r) * K;
    float acc = 0.f;
    for (int kt = 0; kt < tpr; ++kt) {
      if (r | kt) {
#pragma unroll
        for (int u = 0; u < ST_U; ++u) {
          const int k = (kt * ST_U + u) * STEP + lane * EPC;
          w[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(rowp + (FULL || k < K ? k : 0)));
        }
      }
#pragma unroll
      for (int u = 0; u < ST_U; ++u) {
        const int k = (kt * ST_U + u) * STEP + lane * EPC;
        if (FULL || k < K) wchunk<T>::fma(w[u], xs + k, acc);
      }
    }
    const float sum = wave_sum(acc);
    if (lane == r) mine = sum;
  }
  return mine;
}

// x (coherent) -> LayerNorm -> xs in LDS (layers.py:17-36)
__device__ __forceinline__ void stage_layernorm(const float* x, const float* scale, const float* offset, int K, float* xs,
                                                float (*red)[16]) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = ST_NT >> 6;
  float s = 0.f;
#pragma unroll 4
  for (int k = tid; k < K; k += ST_NT) {
    const float v = ldc(x + k);
    xs[k] = v;
    s += v;
  }
  s = wave_sum(s);
  if (lane == 0) red[0][wave] = s;
  __syncthreads();
  float tot = 0.f;
  for (int i = 0; i < nwaves; ++i) tot += red[0][i];
  const float mean = tot / (float)K;
  float qq = 0.f;
  for (int k = tid; k < K; k += ST_NT) {
    const float t = xs[k] - mean;
    qq += t * t;
  }
  qq = wave_sum(qq);
  if (lane == 0) red[1][wave] = qq;
  __syncthreads();
  float var = 0.f;
  for (int i = 0; i < nwaves; ++i) var += red[1][i];
  const float inv = rsqrtf(var / (float)K + 1e-5f);
  for (int k = tid; k < K; k += ST_NT) xs[k] = (scale[k] * inv) * (xs[k] - mean) + offset[k];
  __syncthreads();
}

// FULL: every row length is a whole number of wavefront tiles (ST_U x 64 lanes x 16 bytes), so no load is clamped
template <typename T, int DH, bool FULL>
__global__ __launch_bounds__(ST_NT) void decode_step_kernel(const step_args a) {
  extern __shared__ __align__(16) float smem[];
  __shared__ float red[2][16];
  __shared__ float wgt[ST_CHUNK + 1];
  const mtj_step& s = a.s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int d = s.d_model, F = 4 * s.d_model, H = s.n_heads, r = s.rotary_dims, Tcap = s.Tcap;
  const int pos = s.pos[0];
  const int slot_new = pos % Tcap;
  const int nvalid = (pos + 1 < Tcap) ? pos + 1 : Tcap;
  const int ns = (nvalid + ST_CHUNK - 1) / ST_CHUNK;
  const int pp = pos < s.max_pos ? pos : s.max_pos - 1;
  unsigned epoch = 0;
  float* xs = smem;

  const row_range rin = my_rows(3 * (int64_t)d + F, 2), rout = my_rows(d, 1), rlog = my_rows(s.n_vocab, 1);
  uint32x4 w[ST_U];
  first_tile<T, FULL>(reinterpret_cast<const T*>(s.layers[0].w_in), d, rin, w);

#pragma unroll 1
  for (int l = 0; l < s.n_layers; ++l) {
    const mtj_step_layer L = s.layers[l];
    // ================= phase A: LayerNorm + q|v|k|fc_in rows, RoPE, K/V append, bias + GELU
    {
      // epilogue operands of "my" row first (lane j finishes row rin.row0 + j): nothing may wait behind the stream
      const int64_t n = rin.row0 + lane;
      const bool mine_ok = lane < rin.nrows;
      const int seg = n >= 3 * (int64_t)d ? 3 : (int)(n / d);         // 0 q, 1 v, 2 k, 3 fc_in
      const int c = (int)(n - (int64_t)(seg < 3 ? seg : 3) * d);
      const int e = c % DH;
      float sn = 0.f, cs = 1.f, bias = 0.f;
      if (mine_ok) {
        if (seg == 3) bias = L.b1[c];
        else if (seg != 1 && e < r) {
          const float t = s.sin_tab[(int64_t)pp * (r / 2) + (e >> 1)];
          cs = s.cos_tab[(int64_t)pp * (r / 2) + (e >> 1)];
          sn = (e & 1) ? t : -t;
        }
      }
      stage_layernorm(s.x, L.ln_scale, L.ln_offset, d, xs, red);
      const float own = stream_rows<T, FULL>(reinterpret_cast<const T*>(L.w_in), d, rin, w, xs);
      const float partner = __shfl_xor(own, 1);
      if (mine_ok) {
        if (seg == 3) {
          stc(a.act + d + c, gelu_tanh(own + bias));
        } else {
          const float val = own * cs + partner * sn;
          if (seg == 0) {
            stc(a.q + c, val);
          } else {
            const float rv = wchunk<T>::round(val);
            T* cache = reinterpret_cast<T*>(seg == 1 ? L.v_cache : L.k_cache);
            elem<T>::store(cache + ((int64_t)(c / DH) * Tcap + slot_new) * DH + e, val);   // for the steps to come
            stc(a.kv_new + (seg == 1 ? d : 0) + c, rv);                                     // for this step
          }
        }
      }
    }
    if (!grid_barrier(a.sync, ++epoch, [] {})) return;

    // ================= phase B: attention partials over the cached rows (the new row is added in phase C)
    {
      constexpr int EPC = wchunk<T>::EPC, LPK = DH / EPC, KPL = 64 / LPK, NI = ST_CHUNK / (4 * KPL);
      float* sc = smem;                                   // [4][64]
      float* part = smem + 4 * ST_CHUNK;                  // [4][4][DH]
      const int grp = wave >> 2, gw = wave & 3;           // 4 groups of 4 wavefronts, one (head, range) each
      const int sub = lane / LPK, el = (lane % LPK) * EPC;
      const int total = H * ns, stride = gridDim.x * 4;
      const int iters = (total + stride - 1) / stride;
#pragma unroll 1
      for (int it = 0; it < iters; ++it) {
        const int vb = it * stride + blockIdx.x * 4 + grp;
        const bool active = vb < total;
        const int h = active ? vb / ns : 0, sp = active ? vb % ns : 0;
        const int k0 = sp * ST_CHUNK;
        const int nk = !active ? 0 : ((k0 + ST_CHUNK < nvalid) ? ST_CHUNK : nvalid - k0);
        // K rows first, V rows after the scores: half the registers of having both in flight.  Loads are
        // unconditional (rows beyond the range re-read its first row) so that no register is conditionally defined.
        uint32x4 kr[NI];
        const T* kbase = reinterpret_cast<const T*>(L.k_cache) + ((int64_t)h * Tcap + k0) * DH + el;
        const T* vbase = reinterpret_cast<const T*>(L.v_cache) + ((int64_t)h * Tcap + k0) * DH + el;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int kk = (i * 4 + gw) * KPL + sub;
          kr[i] = *reinterpret_cast<const uint32x4*>(kbase + (int64_t)(kk < nk ? kk : 0) * DH);
        }
        float qv[EPC];
#pragma unroll
        for (int j = 0; j < EPC; ++j) qv[j] = ldc(a.q + h * DH + el + j);
        const float scale = rsqrtf((float)DH);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int kk = (i * 4 + gw) * KPL + sub;
          float dd;
          const uint32x4 ww = kr[i];
          if (sizeof(T) == 2) {
            dd = bf16_lo(ww.x) * qv[0] + bf16_hi(ww.x) * qv[1 % EPC] + bf16_lo(ww.y) * qv[2 % EPC] + bf16_hi(ww.y) * qv[3 % EPC] +
                 bf16_lo(ww.z) * qv[4 % EPC] + bf16_hi(ww.z) * qv[5 % EPC] + bf16_lo(ww.w) * qv[6 % EPC] + bf16_hi(ww.w) * qv[7 % EPC];
          } else {
            dd = __uint_as_float(ww.x) * qv[0] + __uint_as_float(ww.y) * qv[1] + __uint_as_float(ww.z) * qv[2] +
                 __uint_as_float(ww.w) * qv[3];
          }
#pragma unroll
          for (int o = LPK / 2; o > 0; o >>= 1) dd += __shfl_xor(dd, o);
          // the slot of the new token holds a row that may not have reached this CU yet: it is left out here
          if (kk < nk && (lane % LPK) == 0) sc[grp * ST_CHUNK + kk] = (k0 + kk == slot_new) ? -INFINITY : dd * scale;
        }
        uint32x4 vr[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int kk = (i * 4 + gw) * KPL + sub;
          vr[i] = *reinterpret_cast<const uint32x4*>(vbase + (int64_t)(kk < nk ? kk : 0) * DH);
        }
        __syncthreads();
        const float sv = (lane < nk) ? sc[grp * ST_CHUNK + lane] : -INFINITY;
        const float m = wave_max(sv);
        const float pv = (lane < nk && m != -INFINITY) ? expf(sv - m) : 0.f;
        const float lsum = wave_sum(pv);
        float acc[EPC];
#pragma unroll
        for (int j = 0; j < EPC; ++j) acc[j] = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int kk = (i * 4 + gw) * KPL + sub;
          const float pk = __shfl(pv, kk);              // by every lane: a lane switched off cannot be read from
          const float p = (kk < nk) ? pk : 0.f;         // p == 0 for the slot left out (its V row is never multiplied)
          const uint32x4 ww = vr[i];
          if (p != 0.f) {
            if (sizeof(T) == 2) {
              acc[0] += p * bf16_lo(ww.x); acc[1 % EPC] += p * bf16_hi(ww.x);
              acc[2 % EPC] += p * bf16_lo(ww.y); acc[3 % EPC] += p * bf16_hi(ww.y);
              acc[4 % EPC] += p * bf16_lo(ww.z); acc[5 % EPC] += p * bf16_hi(ww.z);
              acc[6 % EPC] += p * bf16_lo(ww.w); acc[7 % EPC] += p * bf16_hi(ww.w);
            } else {
              acc[0] += p * __uint_as_float(ww.x); acc[1] += p * __uint_as_float(ww.y);
              acc[2] += p * __uint_as_float(ww.z); acc[3] += p * __uint_as_float(ww.w);
            }
          }
        }
#pragma unroll
        for (int j = 0; j < EPC; ++j)
#pragma unroll
          for (int o = 32; o >= LPK; o >>= 1) acc[j] += __shfl_xor(acc[j], o);
        if (lane < LPK)
#pragma unroll
          for (int j = 0; j < EPC; ++j) part[(grp * 4 + gw) * DH + el + j] = acc[j];
        __syncthreads();
        if (active) {
          float* wout = a.partials + ((int64_t)h * a.S + sp) * (DH + 2);
          const int t4 = tid & 255;
#pragma unroll 1
          for (int e2 = t4; e2 < DH; e2 += 256) {
            const float* pg = part + grp * 4 * DH + e2;
            stc(wout + 2 + e2, (pg[0] + pg[DH]) + (pg[2 * DH] + pg[3 * DH]));
          }
          if (t4 == 0) { stc(wout, m); stc(wout + 1, lsum); }
        }
        __syncthreads();
      }
    }
    if (!grid_barrier(a.sync, ++epoch, [] {})) return;

    // ================= phase C: merge the partials of a head with the new token's own key / value
#pragma unroll 1
    for (int h = blockIdx.x; h < H; h += gridDim.x) {
      float* prod = smem;                                  // [DH] products q * k_new
#pragma unroll 1
      for (int e2 = tid; e2 < DH; e2 += ST_NT) prod[e2] = ldc(a.q + h * DH + e2) * ldc(a.kv_new + h * DH + e2);
      __syncthreads();
      if (wave == 0) {
        float dn = 0.f;
#pragma unroll 1
        for (int e2 = lane; e2 < DH; e2 += 64) dn += prod[e2];
        const float m_new = wave_sum(dn) * rsqrtf((float)DH);
        const float* wb = a.partials + (int64_t)h * a.S * (DH + 2);
        const float ms = (lane < ns) ? ldc(wb + (int64_t)lane * (DH + 2)) : -INFINITY;
        const float ls = (lane < ns) ? ldc(wb + (int64_t)lane * (DH + 2) + 1) : 0.f;
        const float mm = fmaxf(wave_max(ms), m_new);
        const float f = (lane < ns && ms != -INFINITY) ? expf(ms - mm) : 0.f;
        const float fn = expf(m_new - mm);
        const float lt = wave_sum(f * ls) + fn;
        wgt[lane] = f / lt;
        if (lane == 0) wgt[ST_CHUNK] = fn / lt;
      }
      __syncthreads();
#pragma unroll 1
      for (int e2 = tid; e2 < DH; e2 += ST_NT) {
        const float* wb = a.partials + (int64_t)h * a.S * (DH + 2) + 2 + e2;
        float acc0 = wgt[ST_CHUNK] * ldc(a.kv_new + d + h * DH + e2);
#pragma unroll 2
        for (int s2 = 0; s2 < ns; ++s2) {
          const float ws = wgt[s2];
          if (ws != 0.f) acc0 += ws * ldc(wb + (int64_t)s2 * (DH + 2));
        }
        stc(a.act + h * DH + e2, acc0);
      }
      __syncthreads();
    }
    // the weight request keeps the memory pipeline busy while the workgroups wait and the activations are staged
    if (!grid_barrier(a.sync, ++epoch, [&] { first_tile<T, FULL>(reinterpret_cast<const T*>(L.w_out), d + F, rout, w); })) return;

    // ================= phase D: out | fc_out rows + bias + residual
    {
      const int64_t n = rout.row0 + lane;
      const bool mine_ok = lane < rout.nrows;
      float add = 0.f;
      if (mine_ok) add = L.b2[n] + ldc(s.x + n);          // phase A of this layer is long done with x
      const int K = d + F;
#pragma unroll 4
      for (int k = tid; k < K; k += ST_NT) xs[k] = ldc(a.act + k);
      __syncthreads();
      const float own = stream_rows<T, FULL>(reinterpret_cast<const T*>(L.w_out), K, rout, w, xs);
      if (mine_ok) stc(s.x + n, own + add);
    }
    const bool last = l + 1 == s.n_layers;
    const T* wnext = reinterpret_cast<const T*>(last ? s.w_p : s.layers[last ? l : l + 1].w_in);
    if (!grid_barrier(a.sync, ++epoch, [&] { first_tile<T, FULL>(wnext, d, last ? rlog : rin, w); })) return;
  }
  // ================= final LayerNorm + logits (ProjectionShard, layers.py:561-567)
  {
    const int64_t n = rlog.row0 + lane;
    const bool mine_ok = lane < rlog.nrows;
    const float bias = mine_ok ? s.b_p[n] : 0.f;
    stage_layernorm(s.x, s.pln_scale, s.pln_offset, d, xs, red);
    const float own = stream_rows<T, FULL>(reinterpret_cast<const T*>(s.w_p), d, rlog, w, xs);
    if (mine_ok) s.logits[n] = own + bias;
  }
}

struct step_layout { size_t sync, q, act, kv_new, partials, total; };
step_layout layout(int64_t d, int64_t H, int64_t dh, int64_t Tcap) {
  step_layout L;
  const int64_t S = (Tcap + ST_CHUNK - 1) / ST_CHUNK;
  size_t o = 0;
  auto take = [&](size_t bytes) { const size_t at = o; o += (bytes + 255) & ~(size_t)255; return at; };
  L.sync = take(1024);
  L.q = take((size_t)d * 4);
  L.act = take((size_t)5 * d * 4);
  L.kv_new = take((size_t)2 * d * 4);
  L.partials = take((size_t)H * S * (dh + 2) * 4);
  L.total = o;
  return L;
}

}  // namespace

extern "C" int64_t mtj_decode_step_work_bytes(int64_t d_model, int64_t n_heads, int64_t d_head, int64_t Tcap) {
  if (d_model <= 0 || n_heads <= 0 || d_head <= 0 || Tcap <= 0) return 0;
  return (int64_t)layout(d_model, n_heads, d_head, Tcap).total;
}

extern "C" int mtj_decode_step(const mtj_step* st, void* work, void* stream) {
  MTJ_REQUIRE(st && work, MTJ_EINVAL, "mtj_decode_step: null pointer");
  const mtj_step& s = *st;
  MTJ_REQUIRE(s.layers && s.pos && s.sin_tab && s.cos_tab && s.x && s.pln_scale && s.pln_offset && s.w_p && s.b_p && s.logits,
              MTJ_EINVAL, "mtj_decode_step: null pointer in the description");
  MTJ_REQUIRE(s.dtype == MTJ_F32 || s.dtype == MTJ_BF16, MTJ_EDTYPE, "mtj_decode_step: dtype %d", s.dtype);
  MTJ_REQUIRE(s.n_layers > 0 && s.d_model > 0 && s.n_heads > 0 && s.n_heads <= 64 && s.d_model == s.n_heads * s.d_head &&
                  (s.d_head == 64 || s.d_head == 256) && s.rotary_dims % 2 == 0 && s.rotary_dims <= s.d_head &&
                  s.Tcap > 0 && s.Tcap <= 64 * ST_CHUNK && s.n_vocab > 0 && s.max_pos > 0 && s.d_model % 8 == 0,
              MTJ_EINVAL, "mtj_decode_step: unsupported geometry (d_head 64 or 256, at most 64 heads and 4096 window slots)");
  MTJ_REQUIRE((reinterpret_cast<uintptr_t>(work) & 255u) == 0, MTJ_EALIGN, "mtj_decode_step: work must be 256-byte aligned");
  // the staged activations (5 * d_model floats); the attention phase reuses it for 4 x 64 scores + 16 x d_head partials
  size_t lds = (size_t)5 * s.d_model * sizeof(float);
  if (lds < (4 * ST_CHUNK + 16 * 256) * sizeof(float)) lds = (4 * ST_CHUNK + 16 * 256) * sizeof(float);
  MTJ_REQUIRE(lds <= 140 * 1024, MTJ_ELIMIT,
              "mtj_decode_step: d_model %d does not fit the staging area", s.d_model);
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess || cus <= 0) return mtj_fail(MTJ_EHIP, "mtj_decode_step: cannot query the device: %s", hipGetErrorString(e));
  // every workgroup must be resident at once (they wait for each other): one per CU
  const int grid = cus;
  // a lane finishes one row of its wavefront's share: at most 64 rows per wavefront
  const int64_t nwaves = (int64_t)grid * (ST_NT / 64);
  MTJ_REQUIRE((5 * (int64_t)s.d_model + s.d_model * 2) / nwaves + 2 <= 64 && s.n_vocab / nwaves + 1 <= 64, MTJ_ELIMIT,
              "mtj_decode_step: %d compute units are too few for d_model %d / n_vocab %d", cus, s.d_model, s.n_vocab);
  const step_layout L = layout(s.d_model, s.n_heads, s.d_head, s.Tcap);
  unsigned char* wb = reinterpret_cast<unsigned char*>(work);
  step_args a;
  a.s = s;
  a.sync = reinterpret_cast<unsigned*>(wb + L.sync);
  a.q = reinterpret_cast<float*>(wb + L.q);
  a.act = reinterpret_cast<float*>(wb + L.act);
  a.kv_new = reinterpret_cast<float*>(wb + L.kv_new);
  a.partials = reinterpret_cast<float*>(wb + L.partials);
  a.S = (s.Tcap + ST_CHUNK - 1) / ST_CHUNK;
  hipStream_t hs = (hipStream_t)stream;
#define MTJ_STEP(T, DH, FULL)                                                                                            \
  do {                                                                                                                   \
    static bool attr_set = false;                                                                                        \
    if (!attr_set) {                                                                                                     \
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(&decode_step_kernel<T, DH, FULL>),                           \
                              hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);                                   \
      if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "mtj_decode_step: hipFuncSetAttribute: %s", hipGetErrorString(e));  \
      attr_set = true;                                                                                                   \
    }                                                                                                                    \
    decode_step_kernel<T, DH, FULL><<<grid, ST_NT, lds, hs>>>(a);                                                        \
  } while (0)
  const int tile = ST_U * 64 * 16 / (s.dtype == MTJ_BF16 ? 2 : 4);      // elements of a row per wavefront tile
  const bool full = s.d_model % tile == 0;                              // then 5 * d_model is a whole number too
  if (s.dtype == MTJ_BF16) {
    if (s.d_head == 256) { if (full) MTJ_STEP(bf16_t, 256, true); else MTJ_STEP(bf16_t, 256, false); }
    else { if (full) MTJ_STEP(bf16_t, 64, true); else MTJ_STEP(bf16_t, 64, false); }
  } else {
    if (s.d_head == 256) { if (full) MTJ_STEP(float, 256, true); else MTJ_STEP(float, 256, false); }
    else { if (full) MTJ_STEP(float, 64, true); else MTJ_STEP(float, 64, false); }
  }
#undef MTJ_STEP
  return mtj_check_launch("mtj_decode_step");
}

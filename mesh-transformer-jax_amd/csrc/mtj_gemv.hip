// Batch-1 decode GEMV: y = f(x) @ W^T, W row-major [N, K] (float32 or bf16), float32 activations and
// accumulation.  HBM-bound: every weight byte is read exactly once, as 16-byte loads that a wavefront
// issues over 1 KiB of one row; x (optionally LayerNorm'd on the fly) lives in LDS.
#include "mtj_common.h"

namespace {

template <typename T> struct chunk;  // one 16-byte load of weights -> EPC floats
template <> struct chunk<bf16_t> {
  static constexpr int EPC = 8;
  __device__ static __forceinline__ void fma(const uint32x4& w, const float* __restrict__ xs, float& acc) {
    const floatx4 x0 = *reinterpret_cast<const floatx4*>(xs);
    const floatx4 x1 = *reinterpret_cast<const floatx4*>(xs + 4);
    acc = fmaf(bf16_lo(w.x), x0.x, acc);
    acc = fmaf(bf16_hi(w.x), x0.y, acc);
    acc = fmaf(bf16_lo(w.y), x0.z, acc);
    acc = fmaf(bf16_hi(w.y), x0.w, acc);
    acc = fmaf(bf16_lo(w.z), x1.x, acc);
    acc = fmaf(bf16_hi(w.z), x1.y, acc);
    acc = fmaf(bf16_lo(w.w), x1.z, acc);
    acc = fmaf(bf16_hi(w.w), x1.w, acc);
  }
};
template <> struct chunk<f16_t> {
  static constexpr int EPC = 8;
  __device__ static __forceinline__ void fma(const uint32x4& w, const float* __restrict__ xs, float& acc) {
    const floatx4 x0 = *reinterpret_cast<const floatx4*>(xs);
    const floatx4 x1 = *reinterpret_cast<const floatx4*>(xs + 4);
    acc = fmaf(f16_lo(w.x), x0.x, acc);
    acc = fmaf(f16_hi(w.x), x0.y, acc);
    acc = fmaf(f16_lo(w.y), x0.z, acc);
    acc = fmaf(f16_hi(w.y), x0.w, acc);
    acc = fmaf(f16_lo(w.z), x1.x, acc);
    acc = fmaf(f16_hi(w.z), x1.y, acc);
    acc = fmaf(f16_lo(w.w), x1.z, acc);
    acc = fmaf(f16_hi(w.w), x1.w, acc);
  }
};
template <> struct chunk<float> {
  static constexpr int EPC = 4;
  __device__ static __forceinline__ void fma(const uint32x4& w, const float* __restrict__ xs, float& acc) {
    const floatx4 x0 = *reinterpret_cast<const floatx4*>(xs);
    acc = fmaf(__uint_as_float(w.x), x0.x, acc);
    acc = fmaf(__uint_as_float(w.y), x0.y, acc);
    acc = fmaf(__uint_as_float(w.z), x0.z, acc);
    acc = fmaf(__uint_as_float(w.w), x0.w, acc);
  }
};

struct gemv_args {
  const float* x;
  const float* ln_scale;
  const float* ln_offset;
  const void* W;
  const float* bias;
  int64_t N, K;
  int epi;
  void* out;
  int out_dtype;
  mtj_inproj ip;
  mtj_attn_merge am;      // partials == NULL: x is read as it is
  int upb, upb_rem;       // units per workgroup: the first upb_rem workgroups take upb + 1 (set by launch())
  // ARGMAX only: the greedy sampler behind a STORE of one row of logits
  unsigned long long* am_work;   // [0] best (value image, ~index) so far, [16] arrivals; both 0 between launches
  int32_t* tok;
  int32_t* out_tokens;        // row 0 of the token buffer (one sequence)
  int32_t* pos;
  const int32_t* pos_start;
  mtj_next_embed ne;
};

// Stages the input vector of a matrix-vector kernel into LDS: LayerNorm on the fly (two passes, as the reference
// computes jnp.var), or the attention partials merged into the leading H * dh entries (MERGE), or a plain copy.
// xv holds this thread's four values when fast_x (K == 4 * blockDim.x, requested by the caller before anything else).
// Ends with a workgroup barrier.
template <bool MERGE>
__device__ __forceinline__ void stage_x(const gemv_args& a, float* __restrict__ xs, float (&red)[2][16], const floatx4& xv,
                                        bool fast_x) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const int K = (int)a.K;
  const bool ln = a.ln_scale != nullptr;
  if (ln) {
    float s = 0.f;
    if (fast_x) {
      s = (xv.x + xv.y) + (xv.z + xv.w);
    } else {
      for (int k = tid; k < K; k += blockDim.x) {
        const float v = a.x[k];
        xs[k] = v;
        s += v;
      }
    }
    s = wave_sum(s);
    if (lane == 0) red[0][wave] = s;
    __syncthreads();
    float tot = 0.f;
    for (int i = 0; i < nwaves; ++i) tot += red[0][i];
    const float mean = tot / (float)K;
    float q = 0.f;
    if (fast_x) {
      const floatx4 t = xv - mean;
      q = (t.x * t.x + t.y * t.y) + (t.z * t.z + t.w * t.w);
    } else {
      for (int k = tid; k < K; k += blockDim.x) {
        const float t = xs[k] - mean;
        q += t * t;
      }
    }
    q = wave_sum(q);
    if (lane == 0) red[1][wave] = q;
    __syncthreads();
    float var = 0.f;
    for (int i = 0; i < nwaves; ++i) var += red[1][i];
    const float inv = rsqrtf(var / (float)K + 1e-5f);
    if (fast_x) {
      const floatx4 sc = *reinterpret_cast<const floatx4*>(a.ln_scale + 4 * tid);
      const floatx4 of = *reinterpret_cast<const floatx4*>(a.ln_offset + 4 * tid);
      *reinterpret_cast<floatx4*>(xs + 4 * tid) = (sc * inv) * (xv - mean) + of;
    } else {
      for (int k = tid; k < K; k += blockDim.x)
        xs[k] = (a.ln_scale[k] * inv) * (xs[k] - mean) + a.ln_offset[k];
    }
  } else {
    // the leading H * dh inputs may come from the per-range partials of the one-token attention
    const int dm = MERGE ? a.am.n_heads * a.am.d_head : 0;
    if (MERGE)
    for (int k = tid * 4; k < dm; k += blockDim.x * 4) {
      const int h = k / a.am.d_head, e = k - h * a.am.d_head;
      *reinterpret_cast<floatx4*>(xs + k) =
          mtj_merge_partials(a.am.partials + (int64_t)h * a.am.splits * (a.am.d_head + MTJ_DEC_PAD), a.am.splits,
                             a.am.d_head + MTJ_DEC_PAD, e);
    }
    for (int k = dm + tid * 4; k < K; k += blockDim.x * 4)
      *reinterpret_cast<floatx4*>(xs + k) = *reinterpret_cast<const floatx4*>(a.x + k);
  }
  __syncthreads();

}

// One workgroup of 16 wavefronts per CU, all resident at once (a second round of workgroups would pay the
// prologue and the drain of the memory pipeline twice).  The rows (row pairs for the fused input projection,
// whose rotary epilogue needs both halves of a pair) are dealt out in equal contiguous ranges over all
// wavefronts of the grid.  Nothing on the streaming path depends on a second global load: x is requested
// first, then the first U KiB of weights (so the LayerNorm prologue overlaps the first HBM round trip), and
// every epilogue operand (position, sin/cos, biases, the residual) is fetched up front by the lane that
// will finish that row - under load a dependent load costs tens of microseconds.
//
// FULL: K is a whole number of wavefront tiles (U x 64 lanes x 16 bytes).  The rows of a wavefront are then one
// contiguous run of whole tiles, which is streamed with two tiles in flight - the next one is requested before the
// current one is consumed, so a wavefront never has an empty memory queue - and no load is conditional.  (Dealing
// the rows out round-robin instead, so that the chip reads one contiguous window at a time, streams ~5 % faster in
// a plain read but not here: 43.5 us against 40.2 for the 235 MB launch with every lane's epilogue scattered, 40.9
// against 39.4 with the row sums routed through LDS so that one thread finishes a row and adjacent threads adjacent
// rows; cutting the rows into 1 KiB pieces so that consecutive wavefronts read consecutive KiB takes 49.7 us.)
// MERGE: the leading inputs are merged from one-token attention partials (a.am) instead of being read from x.
// ARGMAX (with a STORE epilogue): the launch also is the greedy sampler of the row it writes.  Every workgroup folds
// the best of its rows into one 64-bit word with an atomic maximum - the monotone image of the float above the
// complement of the index, so that the largest value wins and among equal values the lowest index - and then counts
// its arrival; the workgroup whose arrival completes the count reads the word, which by then holds every
// workgroup's contribution, and does what the sampler does (token, position, embedding of the token for the next
// step), and puts both words back to 0.  Nobody waits for anybody: the order in which workgroups run does not matter.
template <typename T, int U, bool FULL, bool MERGE, bool ARGMAX = false>
__global__ __launch_bounds__(1024) void gemv_kernel(const gemv_args a) {
  extern __shared__ __align__(16) float xs[];
  __shared__ float red[2][16];
  constexpr int EPC = chunk<T>::EPC;
  constexpr int STEP = 64 * EPC;  // elements one wavefront covers per load
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = (int)a.K;
  const T* __restrict__ W = reinterpret_cast<const T*>(a.W);

  const bool pairs = a.epi == MTJ_EPI_INPROJ;
  const int upw = pairs ? 2 : 1;
  // The units of a workgroup (an equal contiguous share of all, cut on the host: no division stands between the
  // start of a wavefront and its first request) go to its sixteen wavefronts in contiguous runs, the odd ones to the
  // FIRST wavefronts: under a saturated memory system the wavefronts of a SIMD are served oldest first and the
  // youngest finish last, so they should be the ones with less to do.
  const int bx = blockIdx.x;
  const int ub0 = bx * a.upb + (bx < a.upb_rem ? bx : a.upb_rem);
  const int cnt = a.upb + (bx < a.upb_rem ? 1 : 0), per = cnt >> 4, rem = cnt & 15;
  const int64_t row0 = (int64_t)(ub0 + wave * per + (wave < rem ? wave : rem)) * upw;
  const int nrows = (per + (wave < rem ? 1 : 0)) * upw;       // <= 64 (the host sizes the grid for that)

  // ---- x first (4 values per thread while K <= 4096; the general loop below covers the rest) ...
  const bool ln = a.ln_scale != nullptr;
  floatx4 xv = {0.f, 0.f, 0.f, 0.f};
  const bool fast_x = ln && K == 4 * (int)blockDim.x;
  if (fast_x) xv = *reinterpret_cast<const floatx4*>(a.x + 4 * tid);
  // ---- ... then the first tile of weights: everything else a wavefront has to work out happens while it is on
  // its way.  (One tile: the CU's memory pipeline takes about 100 KB of requests; the youngest wavefronts already
  // wait 3 us to place theirs, and the LayerNorm's barriers wait for them.  With two tiles per wavefront requested
  // up front they wait 6 us and the launch takes 43 us instead of 39.)
  const int tpr = (K + STEP * U - 1) / (STEP * U);          // tiles per row
  uint32x4 w[U], w2[U];
  __builtin_amdgcn_sched_barrier(0);
  if (FULL) {
    const T* rowp = W + (nrows > 0 ? row0 : 0) * a.K;      // a wavefront without rows reads (and drops) row 0
#pragma unroll
    for (int u = 0; u < U; ++u) w[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(rowp + u * STEP + lane * EPC));
  } else if (nrows > 0) {
    const T* rowp = W + row0 * a.K;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = u * STEP + lane * EPC;
      if (k < K) w[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(rowp + k));
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // ---- ... then the epilogue operands of "my" row (lane j finishes row row0 + j)
  inproj_tok pre;
  pre.kind = -1;
  float pre_add = 0.f;
  if (lane < nrows) {
    const int64_t n = row0 + lane;
    if (pairs) pre = inproj_prepare_token(a.ip, a.bias, (int)n);
    else {
      pre_add = a.bias ? a.bias[n] : 0.f;
      if (a.epi == MTJ_EPI_RESID) pre_add += reinterpret_cast<const float*>(a.out)[n];
    }
  }

  stage_x<MERGE>(a, xs, red, xv, fast_x);

  // ---- stream my rows; lane r keeps the sum of row r
  float mine = 0.f;
  if (FULL) {
    constexpr int TILE = STEP * U;
    const T* base = W + row0 * a.K + lane * EPC;            // tile g of this wavefront starts at base + g * TILE
    const int ntiles = nrows * tpr;
    float acc = 0.f;
    int kt = 0, r = 0;
    auto consume = [&](const uint32x4 (&t)[U]) {
      const float* xk = xs + kt * TILE + lane * EPC;
#pragma unroll
      for (int u = 0; u < U; ++u) chunk<T>::fma(t[u], xk + u * STEP, acc);
      if (++kt == tpr) {                                    // the row is complete
        const float sum = wave_sum(acc);
        if (lane == r) mine = sum;
        acc = 0.f; kt = 0; ++r;
      }
    };
    auto request = [&](uint32x4 (&t)[U], int g) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        t[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(base + (int64_t)g * TILE + u * STEP));
    };
    // steady state without a conditional load: the wait before a tile is consumed then counts only the loads
    // issued before it, and leaves the younger tile in flight
    int g = 0;
    for (; g + 2 < ntiles; g += 2) {
      request(w2, g + 1);
      consume(w);
      request(w, g + 2);
      consume(w2);
    }
    if (g + 1 < ntiles) {
      request(w2, g + 1);
      consume(w);
      consume(w2);
    } else if (g < ntiles) {
      consume(w);
    }
  } else
  for (int r = 0; r < nrows; ++r) {
    const T* rowp = W + (row0 + r) * a.K;
    float acc = 0.f;
    for (int kt = 0; kt < tpr; ++kt) {
      if (r | kt) {   // tile (0, 0) is already in registers
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int k = (kt * U + u) * STEP + lane * EPC;
          if (k < K) w[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(rowp + k));
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k = (kt * U + u) * STEP + lane * EPC;
        if (k < K) chunk<T>::fma(w[u], xs + k, acc);
      }
    }
    const float sum = wave_sum(acc);
    if (lane == r) mine = sum;
  }

  // ---- epilogue: every lane finishes its own row
  if (pairs) {
    const float partner = __shfl_xor(mine, 1);
    if (lane < nrows) inproj_finish_token(a.ip, pre, mine, partner);
  } else if (lane < nrows) {
    const int64_t n = row0 + lane;
    if (a.epi == MTJ_EPI_STORE) store_as(a.out, n, mine + pre_add, a.out_dtype);
    else reinterpret_cast<float*>(a.out)[n] = mine + pre_add;
  }
  if constexpr (ARGMAX) {
    __shared__ unsigned long long best_of_wave[16];
    __shared__ int chosen;                                   // the token, in the workgroup that arrives last; else -1
    unsigned long long best = 0;
    if (lane < nrows) {
      const float v = (mine + pre_add) + 0.0f;               // -0.0 -> +0.0: equal to it in a comparison
      uint32_t u = __float_as_uint(v);
      u = (v != v) ? 0u : ((u & 0x80000000u) ? ~u : (u | 0x80000000u));   // a NaN never wins
      best = ((unsigned long long)u << 32) | (uint32_t)~(uint32_t)(row0 + lane);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const unsigned long long t = __shfl_xor(best, o);
      best = t > best ? t : best;
    }
    if (lane == 0) best_of_wave[wave] = best;
    if (tid == 0) chosen = -1;
    __syncthreads();
    if (tid == 0) {
#pragma unroll
      for (int w = 1; w < 16; ++w) best = best_of_wave[w] > best ? best_of_wave[w] : best;
      unsigned long long seen =
          __hip_atomic_fetch_max(a.am_work, best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      asm volatile("" : "+v"(seen) : : "memory");            // the maximum is in place before the arrival is counted
      const unsigned long long before =
          __hip_atomic_fetch_add(a.am_work + 16, 1ull + (seen & 0ull), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (before == (unsigned long long)gridDim.x - 1) {
        const unsigned long long all = __hip_atomic_load(a.am_work, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(a.am_work, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(a.am_work + 16, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int t = (int)(uint32_t)~(uint32_t)all;
        if (t < 0 || t >= (int)a.N) t = 0;
        a.tok[0] = t;
        if (a.out_tokens) a.out_tokens[a.pos[0] - a.pos_start[0]] = t;
        a.pos[0] += 1;
        chosen = t;
      }
    }
    __syncthreads();
    if (chosen >= 0) embed_next(a.ne, 0, (int)a.N, chosen);
  }
}

template <typename T, int U, bool FULL, bool MERGE, bool ARGMAX = false>
int launch(const gemv_args& a, hipStream_t s) {
  const size_t lds = (size_t)a.K * sizeof(float);
  const int64_t units = a.epi == MTJ_EPI_INPROJ ? a.N / 2 : a.N;
  int64_t grid = 256;                                       // one workgroup per CU
  if (grid > (units + 15) / 16) grid = (units + 15) / 16;   // at least one unit per wavefront
  if (grid < 1) grid = 1;
  const int64_t upw = a.epi == MTJ_EPI_INPROJ ? 2 : 1;
  while ((units + grid * 16 - 1) / (grid * 16) * upw > 62) grid *= 2;   // a lane per row: <= 64 rows per wavefront
  static mtj_device_once once;
  if (int rc = mtj_allow_lds(once, "mtj_gemv", &gemv_kernel<T, U, FULL, MERGE, ARGMAX>, 160 * 1024 - 512)) return rc;
  gemv_args b = a;
  b.upb = (int)(units / grid);
  b.upb_rem = (int)(units % grid);
  gemv_kernel<T, U, FULL, MERGE, ARGMAX><<<(unsigned)grid, 1024, lds, s>>>(b);
  return mtj_check_launch("mtj_gemv");
}

// ------------------------------------------------------------------------------------------------
// Out projection of a decode layer with the one-token attention inside it:  x += [attention | gelu] @ W_out^T + b.
//
// The attention output is only the first H*dh of the K inputs, so the kernel streams the other columns of its rows
// first and needs the attention result only for the last tile(s) of every row.  The attention itself is spread over
// the first H*S workgroups - workgroup b reduces key range b % S of head b / S to a partial (max, sum, weighted V), as
// attn_decode_kernel does - right after the first weight tiles have been requested, so its loads travel with the weight
// stream.  The partials go to memory with agent-scope stores, every workgroup then bumps an arrival counter, and just
// before the attention columns are due (some 20 us later at the 6B shape) a workgroup waits until all arrivals of
// this launch are in, merges the S partials of every head into its copy of the input vector and finishes its rows.
// One launch instead of attention launch + merge.  Measured at the 6B shape, 650 keys (33.3 us against 30.6 + 6.5):
// the workgroups with a key range run ~3.5 us behind the others from the start (their K/V rows compete with the 32 MB
// of first weight tiles that the whole grid requests at once, whichever is asked for first) and their arrival
// costs another ~5 us (agent-scope stores are acknowledged by memory, not by the L2), both hidden behind the ~17 us
// of the first pass; exposed are the merge (two batches of four partials, ~2.8 us) and the pipeline drain.
//
// The wait needs every workgroup of the grid to be resident at once: the host launches at most one workgroup per
// CU.  The wait is bounded by real time (5 ms); if it ever gave up, word 2 of the counter block is set, the result is
// unusable, and every later launch skips its wait until the caller has cleared that word.
// Counter block: work[0] 64-bit arrival counter (never reset: a launch's target is the next multiple of the grid
// size above the value its own arrival returned; the caller zeroes `work` once), then the partials, one per
// (head, range), each in its own 128-byte lines so that no line is shared between writers of different L2s.
constexpr int OA_NI = 4;              // K (and V) loads per lane and attention step: 128 keys of d_head 256 per workgroup
constexpr int OA_HEAD = 32;           // floats in front of the partials (counter block)
constexpr uint64_t OA_WAIT_TICKS = 500000;   // longest wait for the partials: 5 ms of the 100 MHz real-time counter

struct outatt_args {
  gemv_args g;                         // x (entries [0, H*dh) unused), W, bias, N, K, out (residual, in place)
  const float* q;                      // [H, dh]
  const void* kc;
  const void* vc;
  const int32_t* pos;
  int H, Tcap, S;
  float* work;
};

__device__ __forceinline__ int oa_pstride(int dh) { return (dh + MTJ_DEC_PAD + 31) / 32 * 32; }

// mtj_merge_partials for partials that other workgroups of the SAME launch have written: every load carries sc1, the
// cache policy of an agent-scope atomic load, so it is served from the level all XCDs share and never from a line this
// XCD's L2 (or this CU's vector cache) may still hold from an earlier launch - the partials live at the same addresses in
// every launch.  rs covers the partials (everything behind the counter block), hoff is the byte offset of the head's
// first partial in it.  Same arithmetic, same order as mtj_merge_partials.
constexpr int OA_SC1 = 16;            // cache-policy operand of a buffer load: bit 4 = sc1
__device__ __forceinline__ floatx4 oa_merge_coherent(__amdgpu_buffer_rsrc_t rs, int hoff, int S, int stride, int e) {
  float mm = -INFINITY, lt = 0.f;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < S; s0 += 4) {
    float m[4], l[4];
    floatx4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int off = hoff + (s0 + i < S ? s0 + i : S - 1) * stride * 4;
      const uint32x2 st = __builtin_bit_cast(uint32x2, __builtin_amdgcn_raw_buffer_load_b64(rs, off, 0, OA_SC1));
      m[i] = __uint_as_float(st.x);
      l[i] = __uint_as_float(st.y);
      v[i] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rs, off + (MTJ_DEC_PAD + e) * 4, 0, OA_SC1));
    }
    float mb = mm;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (s0 + i >= S) m[i] = -INFINITY;
      mb = fmaxf(mb, m[i]);
    }
    if (mb == -INFINITY) continue;
    const float r = (mm == -INFINITY) ? 0.f : __expf(mm - mb);
    lt *= r;
    acc *= r;
    mm = mb;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float f = (m[i] == -INFINITY) ? 0.f : __expf(m[i] - mm);
      lt = fmaf(f, l[i], lt);
      acc += f * v[i];
    }
  }
  const float inv = lt > 0.f ? 1.0f / lt : 0.f;
  return acc * inv;
}

template <typename T, typename TKV, int DH>
__global__ __launch_bounds__(1024) void gemv_outatt_kernel(const outatt_args oa) {
  const gemv_args& a = oa.g;
  extern __shared__ __align__(16) float xs[];                 // K floats
  __shared__ float part[16][DH];
  __shared__ float stat[16][2];
  constexpr int EPC = chunk<T>::EPC;
  constexpr int STEP = 64 * EPC;
  constexpr int U = 8;
  constexpr int TILE = STEP * U;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = (int)a.K;
  const T* __restrict__ W = reinterpret_cast<const T*>(a.W);
  const int dm = oa.H * DH;                                    // inputs that come from the attention
  const int ta = dm / TILE, tpr = K / TILE;                    // tiles of a row: [0, ta) attention, [ta, tpr) the rest
  const int nwg = gridDim.x;

  // rows of this wavefront: as in gemv_kernel
  const int bx = blockIdx.x;
  const int ub0 = bx * a.upb + (bx < a.upb_rem ? bx : a.upb_rem);
  const int cnt = a.upb + (bx < a.upb_rem ? 1 : 0), per = cnt >> 4, rem = cnt & 15;
  const int64_t row0 = ub0 + wave * per + (wave < rem ? wave : rem);
  const int nrows = per + (wave < rem ? 1 : 0);

  const int p = oa.pos[0];
  float pre_add = 0.f;
  if (lane < nrows) {
    const int64_t n = row0 + lane;
    pre_add = (a.bias ? a.bias[n] : 0.f) + reinterpret_cast<const float*>(a.out)[n];
  }
  // tile number i of the first pass is tile ta + i % (tpr - ta) of row i / (tpr - ta); of the second pass tile i % ta of
  // row i / ta.  A wavefront without rows reads (and drops) row 0.
  const T* base = W + (nrows > 0 ? row0 : 0) * a.K + lane * EPC;
  const int n1 = nrows * (tpr - ta), n2 = nrows * ta;
  auto request = [&](uint32x4 (&t)[U], int i, int t0, int tn) {
    const int r = i / tn, tt = t0 + i - r * tn;
    const T* src = base + (int64_t)r * K + tt * TILE;
#pragma unroll
    for (int u = 0; u < U; ++u) t[u] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(src + u * STEP));
  };
  uint32x4 w[U], w2[U];

  // ---- attention: requests
  constexpr int KEPC = kvrow<TKV>::EPC;
  constexpr int LPK = DH / KEPC, KPL = 64 / LPK, NI = OA_NI;
  constexpr int ASTEP = 16 * NI * KPL;                         // keys per workgroup step
  const int S = oa.S;
  const bool has_att = (int)blockIdx.x < oa.H * S;
  const int h = blockIdx.x / S, split = blockIdx.x - h * S;
  const int nvalid = (p + 1 < oa.Tcap) ? p + 1 : oa.Tcap;
  const int kper = (nvalid + S - 1) / S;
  const int k0 = split * kper;
  const int nk = !has_att ? 0 : (k0 + kper <= nvalid) ? kper : nvalid - k0;
  const int sub = lane / LPK, el = (lane % LPK) * KEPC;
  const TKV* kbase = reinterpret_cast<const TKV*>(oa.kc) + ((int64_t)h * oa.Tcap + k0) * DH + el;
  const TKV* vbase = reinterpret_cast<const TKV*>(oa.vc) + ((int64_t)h * oa.Tcap + k0) * DH + el;
  uint32x4 kr[NI], vr[NI];
  auto att_request = [&](int kb) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      int kk = kb + (i * 16 + wave) * KPL + sub;
      kk = kk < nk ? kk : nk - 1;
      // streaming loads, like the weights: nothing of the window is read twice in a step
      kr[i] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(kbase + (int64_t)kk * DH));
      vr[i] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(vbase + (int64_t)kk * DH));
    }
  };
  // a workgroup with a key range asks for its K/V rows first, so that they do not queue behind 8 KiB of weights
  // per wavefront (loads return in the order they were issued)
  float qv[KEPC];
  if (nk > 0) {
    att_request(0);
#pragma unroll
    for (int j = 0; j < KEPC; ++j) qv[j] = oa.q[h * DH + el + j];
  }
  __builtin_amdgcn_sched_barrier(0);
  request(w, 0, ta, tpr - ta);                                 // n1 >= 1 whenever nrows >= 1; harmless otherwise
  __builtin_amdgcn_sched_barrier(0);

  // ---- stage the inputs that do not come from the attention
  for (int k = dm + tid * 4; k < K; k += 4096)
    *reinterpret_cast<floatx4*>(xs + k) = *reinterpret_cast<const floatx4*>(a.x + k);

  // ---- attention: reduce my key range
  float m_run = -INFINITY, l_run = 0.f;
  float acc_a[KEPC];
#pragma unroll
  for (int j = 0; j < KEPC; ++j) acc_a[j] = 0.f;
  if (nk > 0) {
    const float scale = rsqrtf((float)DH);
    for (int kb = 0; kb < nk; kb += ASTEP) {
      float sc[NI];
      float mt = -INFINITY;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        float kf[KEPC];
        kvrow<TKV>::get(kr[i], kf);
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < KEPC; ++j) d = fmaf(kf[j], qv[j], d);
#pragma unroll
        for (int o = LPK / 2; o > 0; o >>= 1) d += __shfl_xor(d, o);
        const int kk = kb + (i * 16 + wave) * KPL + sub;
        sc[i] = kk < nk ? d * scale : -INFINITY;
        mt = fmaxf(mt, sc[i]);
      }
#pragma unroll
      for (int o = 32; o >= LPK; o >>= 1) mt = fmaxf(mt, __shfl_xor(mt, o));
      const float m_new = fmaxf(m_run, mt);
      float pr[NI];
      if (m_new != -INFINITY) {                               // else this wavefront has had no key yet
        const float alpha = __expf(m_run - m_new);
        l_run *= alpha;
#pragma unroll
        for (int j = 0; j < KEPC; ++j) acc_a[j] *= alpha;
        m_run = m_new;
      }
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        pr[i] = (m_new != -INFINITY) ? __expf(sc[i] - m_new) : 0.f;
        l_run += pr[i];
        float vf[KEPC];
        kvrow<TKV>::get(vr[i], vf);
#pragma unroll
        for (int j = 0; j < KEPC; ++j) acc_a[j] = fmaf(pr[i], vf[j], acc_a[j]);
      }
      if (kb + ASTEP < nk) att_request(kb + ASTEP);
    }
  }
  if (has_att) {
    // key subgroups of a wavefront, then the sixteen wavefronts
#pragma unroll
    for (int o = 32; o >= LPK; o >>= 1) {
      l_run += __shfl_xor(l_run, o);
#pragma unroll
      for (int j = 0; j < KEPC; ++j) acc_a[j] += __shfl_xor(acc_a[j], o);
    }
    if (lane < LPK) {
#pragma unroll
      for (int j = 0; j < KEPC; ++j) part[wave][el + j] = acc_a[j];
    }
    if (lane == 0) { stat[wave][0] = m_run; stat[wave][1] = l_run; }
  }
  __syncthreads();                                            // x in LDS; attention pieces in LDS
  if (has_att) {
    float mm = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) mm = fmaxf(mm, stat[i][0]);
    float* wout = oa.work + OA_HEAD + (int64_t)blockIdx.x * oa_pstride(DH);
    for (int e = tid; e < DH + 2; e += 1024) {
      float v = 0.f;
      if (e < DH) {
#pragma unroll
        for (int i = 0; i < 16; ++i) v += (stat[i][0] == -INFINITY ? 0.f : __expf(stat[i][0] - mm)) * part[i][e];
      } else if (e == DH) {
        v = mm;
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) v += (stat[i][0] == -INFINITY ? 0.f : __expf(stat[i][0] - mm)) * stat[i][1];
      }
      const int at = e < DH ? MTJ_DEC_PAD + e : e - DH;        // {max, sum, -, -, V[DH]}
      __hip_atomic_store(wout + at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  // Every store of this workgroup has reached the coherence point before its arrival is counted.  The second weight
  // tile is requested first: memory operations complete in order, so waiting until only its 8 loads are outstanding
  // waits for the stores without waiting for the tile.
  __builtin_amdgcn_sched_barrier(0);
  if (n1 > 1) {
    request(w2, 1, ta, tpr - ta);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0f78);                        // vmcnt(8), expcnt and lgkmcnt unconstrained
  } else {
    __builtin_amdgcn_s_waitcnt(0x0f70);                        // vmcnt(0)
  }
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();
  // the value the counter had is not needed before the wait: nothing stalls on the atomic's return here
  unsigned long long arrived_at = 0;
  if (tid == 0)
    arrived_at = __hip_atomic_fetch_add(reinterpret_cast<unsigned long long*>(oa.work), 1ull, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);

  // ---- first pass: the columns that do not depend on the attention
  float mine = 0.f, acc = 0.f;
  int ct = ta, cr = 0;                                         // consumer cursor: tile, row
  auto consume = [&](const uint32x4 (&t)[U], int t_end, bool add) {
    const float* xk = xs + ct * TILE + lane * EPC;
#pragma unroll
    for (int u = 0; u < U; ++u) chunk<T>::fma(t[u], xk + u * STEP, acc);
    if (++ct == t_end) {
      const float sum = wave_sum(acc);
      if (lane == cr) mine = add ? mine + sum : sum;
      acc = 0.f; ++cr;
      ct = add ? 0 : ta;
    }
  };
  {
    int g = 0;
    for (; g + 3 < n1; g += 2) {                               // tiles g and g+1 are in w and w2
      consume(w, tpr, false);
      request(w, g + 2, ta, tpr - ta);
      consume(w2, tpr, false);
      request(w2, g + 3, ta, tpr - ta);
    }
    if (g + 2 < n1) {                                          // three left
      consume(w, tpr, false);
      request(w, g + 2, ta, tpr - ta);
      consume(w2, tpr, false);
      consume(w, tpr, false);
    } else if (g + 1 < n1) {
      consume(w, tpr, false);
      consume(w2, tpr, false);
    } else if (g < n1) {
      consume(w, tpr, false);
    }
  }
  // ---- second pass: the attention columns.  Their first tile is requested before the wait.
  if (n2 > 0) request(w, 0, 0, ta);
  if (tid == 0) {
    // Bounded by real time (the 100 MHz counter): a launch whose workgroups are not all resident - CUs masked off, or
    // held by another stream for longer than this - ends after OA_WAIT_TICKS, flagged (word 2 of the counter block),
    // instead of hanging.  Once the flag is up no launch waits any more, so a queue of launches drains at once instead
    // of timing out one by one; the results are void until the caller has cleared the flag.
    const unsigned long long* cnt = reinterpret_cast<const unsigned long long*>(oa.work);
    unsigned* flag = reinterpret_cast<unsigned*>(oa.work) + 2;
    const unsigned long long target = (arrived_at / (unsigned)nwg + 1) * (unsigned)nwg;
    const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
    while (__hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      __builtin_amdgcn_s_sleep(8);
      if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) break;
      if (__builtin_amdgcn_s_memrealtime() - t0 > OA_WAIT_TICKS) {   // some workgroup never arrived: give up, flag it
        __hip_atomic_store(flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
  }
  __syncthreads();
  {
    // The partials were written by other workgroups of this launch with agent-scope stores that had completed
    // (s_waitcnt) before their writers' arrivals were counted, and the count was seen complete before this point, so
    // they are at the level the XCDs share; the loads carry sc1 so that they are served from there.
    const int ps = oa_pstride(DH);
    const __amdgpu_buffer_rsrc_t prs =
        __builtin_amdgcn_make_buffer_rsrc(oa.work + OA_HEAD, 0, oa.H * S * ps * 4, 0x00020000);
    for (int k = tid * 4; k < dm; k += 4096) {
      const int hh = k / DH, e = k - hh * DH;
      *reinterpret_cast<floatx4*>(xs + k) = oa_merge_coherent(prs, hh * S * ps * 4, S, ps, e);
    }
  }
  __syncthreads();
  ct = 0; cr = 0;
  for (int g = 0; g < n2; ++g) {
    consume(w, ta, true);
    if (g + 1 < n2) request(w, g + 1, 0, ta);
  }
  if (lane < nrows) reinterpret_cast<float*>(a.out)[row0 + lane] = mine + pre_add;
}

template <typename T>
int dispatch(const gemv_args& a, hipStream_t s) {
  constexpr int U = 8;
  const bool full = a.K % (U * 64 * chunk<T>::EPC) == 0;
  if (a.am_work) return full ? launch<T, U, true, false, true>(a, s) : launch<T, U, false, false, true>(a, s);
  if (a.am.partials) return full ? launch<T, U, true, true>(a, s) : launch<T, U, false, true>(a, s);
  return full ? launch<T, U, true, false>(a, s) : launch<T, U, false, false>(a, s);
}

}  // namespace

extern "C" int mtj_gemv(const float* x, const float* ln_scale, const float* ln_offset, const void* W,
                        const float* bias, int64_t N, int64_t K, int dtype, int epi, void* out, int out_dtype,
                        const mtj_inproj* ip, const mtj_attn_merge* am, void* stream) {
  MTJ_REQUIRE(x && W, MTJ_EINVAL, "mtj_gemv: null pointer");
  MTJ_REQUIRE(N > 0 && K > 0 && K % 8 == 0, MTJ_EINVAL, "mtj_gemv: K=%lld must be a positive multiple of 8", (long long)K);
  MTJ_REQUIRE(K * 4 <= 160 * 1024 - 512, MTJ_ELIMIT, "mtj_gemv: K=%lld floats do not fit LDS", (long long)K);
  MTJ_REQUIRE(mtj_aligned16(x) && mtj_aligned16(W), MTJ_EALIGN, "mtj_gemv: x and W must be 16-byte aligned");
  MTJ_REQUIRE((ln_scale == nullptr) == (ln_offset == nullptr), MTJ_EINVAL, "mtj_gemv: ln_scale/ln_offset go together");
  gemv_args a{};
  a.x = x; a.ln_scale = ln_scale; a.ln_offset = ln_offset; a.W = W; a.bias = bias;
  a.N = N; a.K = K; a.epi = epi; a.out = out; a.out_dtype = out_dtype;
  if (epi == MTJ_EPI_INPROJ) {
    MTJ_REQUIRE(ip && bias, MTJ_EINVAL, "mtj_gemv: INPROJ needs ip and the fc_in bias");
    a.ip = *ip;
    const int64_t d = (int64_t)ip->n_heads * ip->d_head;
    MTJ_REQUIRE((int64_t)ip->n_heads * ip->Tcap * ip->d_head < (1ll << 31) && N < (1ll << 31) && ip->ld_act < (1ll << 31), MTJ_ELIMIT,
                "mtj_gemv: n_heads * Tcap * d_head, N and ld_act must be below 2^31");
    MTJ_REQUIRE(ip->Tp == 1 && N > 3 * d && N % 2 == 0 && ip->rotary_dims % 2 == 0 && ip->rotary_dims <= ip->d_head &&
                    ip->Tcap > 0 && ip->max_pos > 0 && ip->pos0 && ip->sin_tab && ip->cos_tab && ip->q && ip->k_cache &&
                    ip->v_cache && ip->act && ip->ld_act >= N - 2 * d &&
                    mtj_is_dtype(ip->act_dtype) && mtj_is_dtype(ip->q_dtype) && mtj_is_dtype(ip->kv_dtype),
                MTJ_EINVAL, "mtj_gemv: inconsistent INPROJ geometry");
    a.ip.v_t = nullptr;
  } else if (epi == MTJ_EPI_STORE) {
    MTJ_REQUIRE(out && mtj_is_dtype(out_dtype), MTJ_EINVAL, "mtj_gemv: STORE needs out");
  } else if (epi == MTJ_EPI_RESID) {
    MTJ_REQUIRE(out && out != (const void*)x, MTJ_EINVAL, "mtj_gemv: RESID needs out distinct from x");
  } else {
    return mtj_fail(MTJ_EINVAL, "mtj_gemv: epilogue %d", epi);
  }
  if (am) {
    const int64_t dm = (int64_t)am->n_heads * am->d_head;
    MTJ_REQUIRE(!ln_scale && am->partials && mtj_aligned16(am->partials) && am->n_heads > 0 && am->d_head > 0 &&
                    am->d_head % 4 == 0 && dm <= K && am->splits >= 1 && am->splits <= MTJ_DEC_MAXS,
                MTJ_EINVAL, "mtj_gemv: attention partials need 1..%d ranges, d_head a multiple of 4, H*dh <= K and no LayerNorm",
                MTJ_DEC_MAXS);
    a.am = *am;
  }
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTJ_F32) return dispatch<float>(a, s);
  if (dtype == MTJ_BF16) return dispatch<bf16_t>(a, s);
  if (dtype == MTJ_F16) return dispatch<f16_t>(a, s);
  return mtj_fail(MTJ_EDTYPE, "mtj_gemv: dtype %d", dtype);
}

extern "C" int mtj_gemv_greedy(const float* x, const float* ln_scale, const float* ln_offset, const void* W,
                               const float* bias, int64_t N, int64_t K, int dtype, float* logits, int32_t* tok,
                               int32_t* out_tokens, int64_t ld_tokens, int32_t* pos, const int32_t* pos_start,
                               const mtj_next_embed* next, void* work, void* stream) {
  (void)ld_tokens;
  MTJ_REQUIRE(x && W && logits && tok && pos && pos_start && work, MTJ_EINVAL, "mtj_gemv_greedy: null pointer");
  MTJ_REQUIRE(N > 0 && N < (1ll << 31) && K > 0 && K % 8 == 0, MTJ_EINVAL,
              "mtj_gemv_greedy: K=%lld must be a positive multiple of 8, N below 2^31", (long long)K);
  MTJ_REQUIRE(K * 4 <= 160 * 1024 - 512, MTJ_ELIMIT, "mtj_gemv_greedy: K=%lld floats do not fit LDS", (long long)K);
  MTJ_REQUIRE(mtj_aligned16(x) && mtj_aligned16(W), MTJ_EALIGN, "mtj_gemv_greedy: x and W must be 16-byte aligned");
  MTJ_REQUIRE((reinterpret_cast<uintptr_t>(work) & 255u) == 0, MTJ_EALIGN, "mtj_gemv_greedy: work must be 256-byte aligned");
  MTJ_REQUIRE((ln_scale == nullptr) == (ln_offset == nullptr), MTJ_EINVAL, "mtj_gemv_greedy: ln_scale/ln_offset go together");
  gemv_args a{};
  a.x = x; a.ln_scale = ln_scale; a.ln_offset = ln_offset; a.W = W; a.bias = bias;
  a.N = N; a.K = K; a.epi = MTJ_EPI_STORE; a.out = logits; a.out_dtype = MTJ_F32;
  a.am_work = reinterpret_cast<unsigned long long*>(work);
  a.tok = tok; a.out_tokens = out_tokens; a.pos = pos; a.pos_start = pos_start;   // one row: ld_tokens plays no part
  a.ne = mtj_next_embed{nullptr, nullptr, nullptr, 0, 0};
  if (next && next->w) {
    MTJ_REQUIRE(next->bias && next->x_next && next->d > 0 && (next->dtype == MTJ_F32 || next->dtype == MTJ_BF16), MTJ_EINVAL,
                "mtj_gemv_greedy: incomplete next-step embedding");
    a.ne = *next;
  }
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTJ_F32) return dispatch<float>(a, s);
  if (dtype == MTJ_BF16) return dispatch<bf16_t>(a, s);
  if (dtype == MTJ_F16) return dispatch<f16_t>(a, s);
  return mtj_fail(MTJ_EDTYPE, "mtj_gemv_greedy: dtype %d", dtype);
}

// ------------------------------------------------------------------------------------------------ fused out projection
namespace {

constexpr int OA_TILE_BYTES = 8 * 64 * 16;     // one tile of 8 wavefront loads

struct outatt_plan {
  int grid, S;
};

// The fused kernel needs whole tiles on both sides of the attention/rest boundary and every workgroup resident at once.
bool outatt_plan_for(int64_t N, int64_t K, int dtype, int64_t H, int64_t dh, int kv_dtype, int64_t Tcap, outatt_plan* plan) {
  if (dtype != MTJ_F32 && dtype != MTJ_BF16) return false;
  if (kv_dtype != (dtype == MTJ_F32 ? MTJ_F32 : MTJ_F16) || (dh != 64 && dh != 256) || H <= 0 || N <= 0) return false;
  const int64_t tile = OA_TILE_BYTES / mtj_elem_size(dtype), dm = H * dh;
  if (K % tile || dm % tile || dm >= K || K * 4 + 24 * 1024 > 160 * 1024) return false;
  int64_t grid = 256;
  if (grid > (N + 15) / 16) grid = (N + 15) / 16;
  if ((N + grid * 16 - 1) / (grid * 16) > 62) return false;
  static std::atomic<int> cus[MTJ_MAX_DEVICES];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MTJ_MAX_DEVICES) return false;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return false;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  if (grid > n) return false;
  int64_t S = grid / H;
  if (S > MTJ_DEC_MAXS) S = MTJ_DEC_MAXS;
  if (S > (Tcap + 15) / 16) S = (Tcap + 15) / 16;
  if (S < 1) return false;
  plan->grid = (int)grid;
  plan->S = (int)S;
  return true;
}

template <typename T, typename TKV, int DH>
int launch_outatt(const outatt_args& oa, int grid, hipStream_t s) {
  const size_t lds = (size_t)oa.g.K * sizeof(float);
  static mtj_device_once once;
  if (int rc = mtj_allow_lds(once, "mtj_gemv_attn", &gemv_outatt_kernel<T, TKV, DH>, 160 * 1024 - 24 * 1024)) return rc;
  gemv_outatt_kernel<T, TKV, DH><<<(unsigned)grid, 1024, lds, s>>>(oa);
  return mtj_check_launch("mtj_gemv_attn");
}

}  // namespace

extern "C" int mtj_gemv_attn_supported(int64_t N, int64_t K, int dtype, int64_t H, int64_t dh, int kv_dtype, int64_t Tcap) {
  outatt_plan plan;
  return outatt_plan_for(N, K, dtype, H, dh, kv_dtype, Tcap, &plan) ? 1 : 0;
}

extern "C" int64_t mtj_gemv_attn_work_bytes(int64_t H, int64_t dh) {
  if (H <= 0 || dh <= 0) return 0;
  return (OA_HEAD + H * MTJ_DEC_MAXS * ((dh + MTJ_DEC_PAD + 31) / 32 * 32)) * (int64_t)sizeof(float);
}

extern "C" int mtj_gemv_attn(const float* x, const void* W, const float* bias, int64_t N, int64_t K, int dtype, float* out,
                             const float* q, const void* k_cache, const void* v_cache, const int32_t* pos, int64_t H,
                             int64_t Tcap, int64_t dh, int kv_dtype, void* work, void* stream) {
  MTJ_REQUIRE(x && W && out && q && k_cache && v_cache && pos && work, MTJ_EINVAL, "mtj_gemv_attn: null pointer");
  MTJ_REQUIRE(out != x, MTJ_EINVAL, "mtj_gemv_attn: out must be distinct from x");
  MTJ_REQUIRE(mtj_aligned16(x) && mtj_aligned16(W) && mtj_aligned16(q) && mtj_aligned16(k_cache) && mtj_aligned16(v_cache) &&
                  (reinterpret_cast<uintptr_t>(work) & 127u) == 0,
              MTJ_EALIGN, "mtj_gemv_attn: x, W, q and the caches must be 16-byte aligned, work 128-byte aligned");
  outatt_plan plan;
  MTJ_REQUIRE(Tcap > 0 && outatt_plan_for(N, K, dtype, H, dh, kv_dtype, Tcap, &plan), MTJ_ELIMIT,
              "mtj_gemv_attn: shape N=%lld K=%lld H=%lld dh=%lld is not covered by the fused kernel (see "
              "mtj_gemv_attn_supported); use mtj_attn_decode_partials + mtj_gemv",
              (long long)N, (long long)K, (long long)H, (long long)dh);
  outatt_args oa{};
  oa.g.x = x; oa.g.W = W; oa.g.bias = bias; oa.g.N = N; oa.g.K = K; oa.g.epi = MTJ_EPI_RESID; oa.g.out = out;
  oa.g.out_dtype = MTJ_F32;
  oa.g.upb = (int)(N / plan.grid); oa.g.upb_rem = (int)(N % plan.grid);
  oa.q = q; oa.kc = k_cache; oa.vc = v_cache; oa.pos = pos; oa.H = (int)H; oa.Tcap = (int)Tcap; oa.S = plan.S;
  oa.work = reinterpret_cast<float*>(work);
  hipStream_t s = (hipStream_t)stream;
#define MTJ_OA(WD, TW, KD, TK, DHV) \
  if (dtype == WD && kv_dtype == KD && dh == DHV) return launch_outatt<TW, TK, DHV>(oa, plan.grid, s);
  MTJ_OA(MTJ_BF16, bf16_t, MTJ_F16, f16_t, 256)
  MTJ_OA(MTJ_BF16, bf16_t, MTJ_F16, f16_t, 64)
  MTJ_OA(MTJ_F32, float, MTJ_F32, float, 256)
  MTJ_OA(MTJ_F32, float, MTJ_F32, float, 64)
#undef MTJ_OA
  return mtj_fail(MTJ_ELIMIT, "mtj_gemv_attn: no kernel for weight dtype %d with K/V dtype %d", dtype, kv_dtype);
}


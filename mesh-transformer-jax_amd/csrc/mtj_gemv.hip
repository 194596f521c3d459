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
};

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
template <typename T, int U, bool FULL, bool MERGE>
__global__ __launch_bounds__(1024) void gemv_kernel(const gemv_args a) {
  extern __shared__ __align__(16) float xs[];
  __shared__ float red[2][16];
  constexpr int EPC = chunk<T>::EPC;
  constexpr int STEP = 64 * EPC;  // elements one wavefront covers per load
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const int K = (int)a.K;
  const T* __restrict__ W = reinterpret_cast<const T*>(a.W);

  const bool pairs = a.epi == MTJ_EPI_INPROJ;
  const int64_t upw = pairs ? 2 : 1;
  const int64_t units = a.N / upw;
  // The units of a workgroup (an equal contiguous share of all) go to its wavefronts in contiguous runs, the odd
  // ones to the FIRST wavefronts: under a saturated memory system the wavefronts of a SIMD are served oldest
  // first and the youngest finish last, so they should be the ones with less to do.
  const int64_t ub0 = units * blockIdx.x / gridDim.x, ub1 = units * (blockIdx.x + 1) / gridDim.x;
  const int cnt = (int)(ub1 - ub0), per = cnt / nwaves, rem = cnt % nwaves;
  const int64_t row0 = (ub0 + (int64_t)wave * per + (wave < rem ? wave : rem)) * upw;
  const int nrows = (per + (wave < rem ? 1 : 0)) * (int)upw;   // <= 64 (the host sizes the grid for that)

  // ---- x first (4 values per thread while K <= 4096; the general loop below covers the rest) ...
  const bool ln = a.ln_scale != nullptr;
  floatx4 xv = {0.f, 0.f, 0.f, 0.f};
  const bool fast_x = ln && K == 4 * (int)blockDim.x;
  if (fast_x) xv = *reinterpret_cast<const floatx4*>(a.x + 4 * tid);
  // ---- ... then the epilogue operands of "my" row (lane j finishes row row0 + j) ...
  inproj_pre pre;
  pre.kind = -1;
  float pre_add = 0.f;
  if (lane < nrows) {
    const int64_t n = row0 + lane;
    if (pairs) pre = inproj_prepare(a.ip, a.bias, 0, n);
    else {
      pre_add = a.bias ? a.bias[n] : 0.f;
      if (a.epi == MTJ_EPI_RESID) pre_add += reinterpret_cast<const float*>(a.out)[n];
    }
  }
  // ---- ... then the first tile of weights
  uint32x4 w[U];
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

  // ---- stage x (with LayerNorm if asked) into LDS
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
          mtj_merge_partials(a.am.partials + (int64_t)h * a.am.splits * (a.am.d_head + MTJ_DEC_PAD), a.am.splits, a.am.d_head, e);
    }
    for (int k = dm + tid * 4; k < K; k += blockDim.x * 4)
      *reinterpret_cast<floatx4*>(xs + k) = *reinterpret_cast<const floatx4*>(a.x + k);
  }
  __syncthreads();

  // ---- stream my rows; lane r keeps the sum of row r
  const int tpr = (K + STEP * U - 1) / (STEP * U);          // tiles per row
  float mine = 0.f;
  if (FULL) {
    constexpr int TILE = STEP * U;
    const T* base = W + row0 * a.K + lane * EPC;            // tile g of this wavefront starts at base + g * TILE
    const int ntiles = nrows * tpr;
    uint32x4 w2[U];
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
    if (lane < nrows) inproj_finish(a.ip, pre, mine, partner);
  } else if (lane < nrows) {
    const int64_t n = row0 + lane;
    if (a.epi == MTJ_EPI_STORE) store_as(a.out, n, mine + pre_add, a.out_dtype);
    else reinterpret_cast<float*>(a.out)[n] = mine + pre_add;
  }
}

template <typename T, int U, bool FULL, bool MERGE>
int launch(const gemv_args& a, hipStream_t s) {
  const size_t lds = (size_t)a.K * sizeof(float);
  const int64_t units = a.epi == MTJ_EPI_INPROJ ? a.N / 2 : a.N;
  int64_t grid = 256;                                       // one workgroup per CU
  if (grid > (units + 15) / 16) grid = (units + 15) / 16;   // at least one unit per wavefront
  if (grid < 1) grid = 1;
  const int64_t upw = a.epi == MTJ_EPI_INPROJ ? 2 : 1;
  while ((units + grid * 16 - 1) / (grid * 16) * upw > 62) grid *= 2;   // a lane per row: <= 64 rows per wavefront
  static mtj_device_once once;
  if (int rc = mtj_allow_lds(once, "mtj_gemv", &gemv_kernel<T, U, FULL, MERGE>, 160 * 1024 - 256)) return rc;
  gemv_kernel<T, U, FULL, MERGE><<<(unsigned)grid, 1024, lds, s>>>(a);
  return mtj_check_launch("mtj_gemv");
}

template <typename T>
int dispatch(const gemv_args& a, hipStream_t s) {
  constexpr int U = 8;
  const bool full = a.K % (U * 64 * chunk<T>::EPC) == 0;
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

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
  int kv_dtype;
  mtj_inproj ip;
};

// R rows per wavefront, U 16-byte loads in flight per row.
template <typename T, int R, int U>
__global__ __launch_bounds__(1024) void gemv_kernel(const gemv_args a) {
  extern __shared__ __align__(16) float xs[];
  __shared__ float red[2][16];
  constexpr int EPC = chunk<T>::EPC;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const int K = (int)a.K;

  // ---- stage x (with LayerNorm if asked) into LDS
  if (a.ln_scale) {
    float s = 0.f;
    for (int k = tid; k < K; k += blockDim.x) {
      const float v = a.x[k];
      xs[k] = v;
      s += v;
    }
    s = wave_sum(s);
    if (lane == 0) red[0][wave] = s;
    __syncthreads();
    float tot = 0.f;
    for (int w = 0; w < nwaves; ++w) tot += red[0][w];
    const float mean = tot / (float)K;
    float q = 0.f;
    for (int k = tid; k < K; k += blockDim.x) {
      const float t = xs[k] - mean;
      q += t * t;
    }
    q = wave_sum(q);
    if (lane == 0) red[1][wave] = q;
    __syncthreads();
    float var = 0.f;
    for (int w = 0; w < nwaves; ++w) var += red[1][w];
    const float inv = rsqrtf(var / (float)K + 1e-5f);
    for (int k = tid; k < K; k += blockDim.x)
      xs[k] = (a.ln_scale[k] * inv) * (xs[k] - mean) + a.ln_offset[k];
  } else {
    for (int k = tid * 4; k < K; k += blockDim.x * 4)
      *reinterpret_cast<floatx4*>(xs + k) = *reinterpret_cast<const floatx4*>(a.x + k);
  }
  __syncthreads();

  // ---- stream the rows of this wavefront
  const int64_t n0 = ((int64_t)blockIdx.x * nwaves + wave) * R;
  if (n0 >= a.N) return;
  const T* __restrict__ W = reinterpret_cast<const T*>(a.W);
  const T* rows[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t n = (n0 + r < a.N) ? n0 + r : a.N - 1;  // clamp: duplicates are never stored
    rows[r] = W + n * a.K;
  }
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;

  const int step = 64 * EPC;            // elements one wavefront covers per load
  const int kfull = (K / (step * U)) * (step * U);
  int k = lane * EPC;
  for (; k < kfull; k += step * U) {
    uint32x4 w[U][R];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < R; ++r)
        w[u][r] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(rows[r] + k + u * step));
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < R; ++r) chunk<T>::fma(w[u][r], xs + k + u * step, acc[r]);
  }
  for (; k < K; k += step) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32x4 w = *reinterpret_cast<const uint32x4*>(rows[r] + k);
      chunk<T>::fma(w, xs + k, acc[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);

  // ---- epilogue: lane r finishes row n0 + r
  if (lane < R) {
    float own = acc[0], partner = acc[0];
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (lane == r) {
        own = acc[r];
        partner = acc[(r ^ 1) < R ? (r ^ 1) : r];
      }
    const int64_t n = n0 + lane;
    if (n < a.N) {
      if (a.epi == MTJ_EPI_STORE) {
        store_as(a.out, n, own + (a.bias ? a.bias[n] : 0.f), a.out_dtype);
      } else if (a.epi == MTJ_EPI_RESID) {
        float* o = reinterpret_cast<float*>(a.out);
        o[n] += own + (a.bias ? a.bias[n] : 0.f);
      } else {
        inproj_store(a.ip, a.bias, a.kv_dtype, 0, n, own, partner);
      }
    }
  }
}

template <typename T, int R, int U>
int launch(const gemv_args& a, int waves, hipStream_t s) {
  const int64_t rows_per_block = (int64_t)waves * R;
  const unsigned grid = (unsigned)((a.N + rows_per_block - 1) / rows_per_block);
  const size_t lds = (size_t)a.K * sizeof(float);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_kernel<T, R, U>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256);
    if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "mtj_gemv: hipFuncSetAttribute: %s", hipGetErrorString(e));
    attr_set = true;
  }
  gemv_kernel<T, R, U><<<grid, waves * 64, lds, s>>>(a);
  return mtj_check_launch("mtj_gemv");
}

template <typename T>
int dispatch(const gemv_args& a, hipStream_t s) {
  // Small K (x fits LDS many times over): 4 wavefronts x 4 rows, so thousands of workgroups.
  // Large K (the 80 KiB out|fc_out input): one 16-wavefront workgroup per CU, the rows split evenly.
  if (a.K * 4 <= 40 * 1024) {
    if (a.N >= 16 * 1024) return launch<T, 4, 4>(a, 4, s);
    return launch<T, 2, 8>(a, 4, s);
  }
  if (a.epi == MTJ_EPI_INPROJ) return launch<T, 2, 8>(a, 16, s);
  if (a.N >= 16 * 512) return launch<T, 2, 8>(a, 16, s);
  return launch<T, 1, 8>(a, 16, s);
}

}  // namespace

extern "C" int mtj_gemv(const float* x, const float* ln_scale, const float* ln_offset, const void* W,
                        const float* bias, int64_t N, int64_t K, int dtype, int epi, void* out, int out_dtype,
                        const mtj_inproj* ip, void* stream) {
  MTJ_REQUIRE(x && W, MTJ_EINVAL, "mtj_gemv: null pointer");
  MTJ_REQUIRE(N > 0 && K > 0 && K % 8 == 0, MTJ_EINVAL, "mtj_gemv: K=%lld must be a positive multiple of 8", (long long)K);
  MTJ_REQUIRE(K * 4 <= 160 * 1024 - 512, MTJ_ELIMIT, "mtj_gemv: K=%lld floats do not fit LDS", (long long)K);
  MTJ_REQUIRE(mtj_aligned16(x) && mtj_aligned16(W), MTJ_EALIGN, "mtj_gemv: x and W must be 16-byte aligned");
  MTJ_REQUIRE((ln_scale == nullptr) == (ln_offset == nullptr), MTJ_EINVAL, "mtj_gemv: ln_scale/ln_offset go together");
  gemv_args a{};
  a.x = x; a.ln_scale = ln_scale; a.ln_offset = ln_offset; a.W = W; a.bias = bias;
  a.N = N; a.K = K; a.epi = epi; a.out = out; a.out_dtype = out_dtype; a.kv_dtype = dtype;
  if (epi == MTJ_EPI_INPROJ) {
    MTJ_REQUIRE(ip && bias, MTJ_EINVAL, "mtj_gemv: INPROJ needs ip and the fc_in bias");
    a.ip = *ip;
    const int64_t d = (int64_t)ip->n_heads * ip->d_head;
    MTJ_REQUIRE(ip->Tp == 1 && N > 3 * d && N % 2 == 0 && ip->rotary_dims % 2 == 0 && ip->rotary_dims <= ip->d_head &&
                    ip->Tcap > 0 && ip->max_pos > 0 && ip->pos0 && ip->sin_tab && ip->cos_tab && ip->q && ip->k_cache &&
                    ip->v_cache && ip->act && ip->ld_act >= N - 2 * d &&
                    (ip->act_dtype == MTJ_F32 || ip->act_dtype == MTJ_BF16) &&
                    (ip->q_dtype == MTJ_F32 || ip->q_dtype == MTJ_BF16),
                MTJ_EINVAL, "mtj_gemv: inconsistent INPROJ geometry");
    a.ip.v_t = nullptr;
  } else if (epi == MTJ_EPI_STORE) {
    MTJ_REQUIRE(out && (out_dtype == MTJ_F32 || out_dtype == MTJ_BF16), MTJ_EINVAL, "mtj_gemv: STORE needs out");
  } else if (epi == MTJ_EPI_RESID) {
    MTJ_REQUIRE(out && out != (const void*)x, MTJ_EINVAL, "mtj_gemv: RESID needs out distinct from x");
  } else {
    return mtj_fail(MTJ_EINVAL, "mtj_gemv: epilogue %d", epi);
  }
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTJ_F32) return dispatch<float>(a, s);
  if (dtype == MTJ_BF16) return dispatch<bf16_t>(a, s);
  return mtj_fail(MTJ_EDTYPE, "mtj_gemv: dtype %d", dtype);
}

// MFMA GEMM for prefill and batched decode: C[M, N] = A[M, K] x W[N, K]^T with fused epilogues.
// Both operands are K-contiguous, are staged global -> registers -> LDS (padded rows, so that the
// 16-byte fragment reads of a 32x32 MFMA hit 64 distinct banks) and double-buffered; accumulation is
// float32.  bf16 uses v_mfma_f32_32x32x16_bf16, float32 uses v_mfma_f32_32x32x2_f32 (true fp32).
#include "mtj_common.h"

namespace {

template <typename T> struct mma;
template <> struct mma<bf16_t> {
  static constexpr int EPC = 8;  // elements per 16-byte chunk
  struct frag { bf16x8 v; };
  __device__ static __forceinline__ frag load(const bf16_t* p) {
    frag f;
    f.v = *reinterpret_cast<const bf16x8*>(p);
    return f;
  }
  __device__ static __forceinline__ void run(floatx16& c, const frag& a, const frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
  }
};
template <> struct mma<float> {
  static constexpr int EPC = 4;
  struct frag { floatx4 lo, hi; };
  __device__ static __forceinline__ frag load(const float* p) {
    frag f;
    f.lo = *reinterpret_cast<const floatx4*>(p);
    f.hi = *reinterpret_cast<const floatx4*>(p + 4);
    return f;
  }
  __device__ static __forceinline__ void run(floatx16& c, const frag& a, const frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.lo.x, b.lo.x, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.lo.y, b.lo.y, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.lo.z, b.lo.z, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.lo.w, b.lo.w, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.hi.x, b.hi.x, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.hi.y, b.hi.y, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.hi.z, b.hi.z, c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.hi.w, b.hi.w, c, 0, 0, 0);
  }
};

struct gemm_args {
  const void* A;
  int64_t lda;
  const void* W;
  const float* bias;
  int M, N, K;
  int epi;
  void* out;
  int64_t ldo;
  int out_dtype;
  int kv_dtype;
  mtj_inproj ip;
};

// Workgroup tile (WAVES_M*WM*32) x (WAVES_N*WN*32), K step BK elements.
template <typename T, int WAVES_M, int WAVES_N, int WM, int WN, int BK>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_kernel(const gemm_args a) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
  constexpr int EPC = mma<T>::EPC;
  constexpr int CPR = BK / EPC;          // 16-byte chunks per tile row
  constexpr int LDS_ROW = BK + EPC;      // padded row, elements (row stride 144 B for both types)
  constexpr int A_CHUNKS = BM * CPR / NT, B_CHUNKS = BN * CPR / NT;
  static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0, "tile does not divide over threads");
  static_assert(BK % 16 == 0, "BK must hold whole MFMA k-steps");

  extern __shared__ __align__(16) unsigned char smem[];
  T* As = reinterpret_cast<T*>(smem);                    // [2][BM][LDS_ROW]
  T* Bs = As + 2 * BM * LDS_ROW;                         // [2][BN][LDS_ROW]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int fr = lane & 31, fg = lane >> 5;

  // ---- tile id: give each XCD (workgroups are dealt round-robin over 8 XCDs) a contiguous range of
  // tiles, then walk that range in groups of 8 row-tiles so one XCD's L2 sees few distinct W panels.
  const int tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
  const int nblk = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int per = nblk / 8;
    if (pid < per * 8) pid = (pid % 8) * per + pid / 8;
  }
  constexpr int GM = 8;
  const int group = pid / (GM * tiles_n);
  const int first_m = group * GM;
  const int gsz = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
  const int tm = first_m + (pid % (GM * tiles_n)) % gsz;
  const int tn = (pid % (GM * tiles_n)) / gsz;
  const int m0 = tm * BM, n0 = tn * BN;

  const T* __restrict__ A = reinterpret_cast<const T*>(a.A);
  const T* __restrict__ W = reinterpret_cast<const T*>(a.W);

  uint32x4 ra[A_CHUNKS], rb[B_CHUNKS];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = i * NT + tid, row = c / CPR, cc = c % CPR;
      const int m = m0 + row;
      ra[i] = (m < a.M) ? *reinterpret_cast<const uint32x4*>(A + (int64_t)m * a.lda + k0 + cc * EPC)
                        : uint32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
      const int c = i * NT + tid, row = c / CPR, cc = c % CPR;
      const int n = n0 + row;
      rb[i] = (n < a.N) ? *reinterpret_cast<const uint32x4*>(W + (int64_t)n * a.K + k0 + cc * EPC)
                        : uint32x4{0, 0, 0, 0};
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = i * NT + tid, row = c / CPR, cc = c % CPR;
      *reinterpret_cast<uint32x4*>(As + (buf * BM + row) * LDS_ROW + cc * EPC) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
      const int c = i * NT + tid, row = c / CPR, cc = c % CPR;
      *reinterpret_cast<uint32x4*>(Bs + (buf * BN + row) * LDS_ROW + cc * EPC) = rb[i];
    }
  };

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int KT = a.K / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) load_global((kt + 1) * BK);
    const T* as = As + (buf * BM + wm * WM * 32 + fr) * LDS_ROW + fg * 8;
    const T* bs = Bs + (buf * BN + wn * WN * 32 + fr) * LDS_ROW + fg * 8;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      typename mma<T>::frag fa[WM], fb[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i) fa[i] = mma<T>::load(as + i * 32 * LDS_ROW + ks * 16);
#pragma unroll
      for (int j = 0; j < WN; ++j) fb[j] = mma<T>::load(bs + j * 32 * LDS_ROW + ks * 16);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) mma<T>::run(acc[i][j], fa[i], fb[j]);
    }
    if (kt + 1 < KT) store_lds(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue.  Accumulator register v of lane l holds C[8*(v/4) + 4*(l/32) + v%4][l%32].
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int n = n0 + (wn * WN + j) * 32 + fr;
      const float bias = (a.bias && a.epi != MTJ_EPI_INPROJ && n < a.N) ? a.bias[n] : 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + (wm * WM + i) * 32 + 8 * (v / 4) + 4 * fg + (v % 4);
        const float own = acc[i][j][v];
        if (a.epi == MTJ_EPI_INPROJ) {
          const float partner = __shfl_xor(own, 1);
          if (m < a.M && n < a.N) inproj_store(a.ip, a.bias, a.kv_dtype, m, n, own, partner);
        } else if (m < a.M && n < a.N) {
          const int64_t idx = (int64_t)m * a.ldo + n;
          if (a.epi == MTJ_EPI_STORE) {
            store_as(a.out, idx, own + bias, a.out_dtype);
          } else {
            float* o = reinterpret_cast<float*>(a.out);
            o[idx] += own + bias;
          }
        }
      }
    }
}

template <typename T, int WAVES_M, int WAVES_N, int WM, int WN, int BK>
int launch(const gemm_args& a, hipStream_t s) {
  constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
  constexpr size_t lds = 2 * (size_t)(BM + BN) * (BK + mma<T>::EPC) * sizeof(T);
  static_assert(lds <= 160 * 1024, "tile does not fit LDS");
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<T, WAVES_M, WAVES_N, WM, WN, BK>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "mtj_gemm: hipFuncSetAttribute: %s", hipGetErrorString(e));
    attr_set = true;
  }
  const int tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  gemm_kernel<T, WAVES_M, WAVES_N, WM, WN, BK><<<tiles, WAVES_M * WAVES_N * 64, lds, s>>>(a);
  return mtj_check_launch("mtj_gemm");
}

template <typename T, int BK>
int dispatch(const gemm_args& a, hipStream_t s) {
  if (a.M <= 32) return launch<T, 1, 4, 1, 2, BK>(a, s);    // 32 x 256: batched decode, weights stream once
  if (a.M <= 64) return launch<T, 1, 4, 2, 2, BK>(a, s);    // 64 x 256
  return launch<T, 2, 2, 2, 2, BK>(a, s);                   // 128 x 128
}

}  // namespace

extern "C" int mtj_gemm(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N, int64_t K,
                        int dtype, int epi, void* out, int64_t ldo, int out_dtype, const mtj_inproj* ip,
                        void* stream) {
  MTJ_REQUIRE(A && W, MTJ_EINVAL, "mtj_gemm: null pointer");
  MTJ_REQUIRE(dtype == MTJ_F32 || dtype == MTJ_BF16, MTJ_EDTYPE, "mtj_gemm: dtype %d", dtype);
  const int bk = dtype == MTJ_BF16 ? 64 : 32;
  const int esz = dtype == MTJ_BF16 ? 2 : 4;
  MTJ_REQUIRE(M > 0 && N > 0 && K > 0 && K % bk == 0 && lda >= K, MTJ_EINVAL,
              "mtj_gemm: bad shape M=%lld N=%lld K=%lld lda=%lld (K must be a multiple of %d)", (long long)M,
              (long long)N, (long long)K, (long long)lda, bk);
  MTJ_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), MTJ_ELIMIT, "mtj_gemm: dimension too large");
  MTJ_REQUIRE(mtj_aligned16(A) && mtj_aligned16(W) && (lda * esz) % 16 == 0, MTJ_EALIGN,
              "mtj_gemm: A, W and the row stride of A must be 16-byte aligned");
  gemm_args a{};
  a.A = A; a.lda = lda; a.W = W; a.bias = bias; a.M = (int)M; a.N = (int)N; a.K = (int)K;
  a.epi = epi; a.out = out; a.ldo = ldo; a.out_dtype = out_dtype; a.kv_dtype = dtype;
  if (epi == MTJ_EPI_INPROJ) {
    MTJ_REQUIRE(ip && bias, MTJ_EINVAL, "mtj_gemm: INPROJ needs ip and the fc_in bias");
    a.ip = *ip;
    const int64_t d = (int64_t)ip->n_heads * ip->d_head;
    MTJ_REQUIRE(ip->Tp > 0 && M % ip->Tp == 0 && N > 3 * d && N % 2 == 0 && ip->rotary_dims % 2 == 0 &&
                    ip->rotary_dims <= ip->d_head && ip->Tcap > 0 && ip->max_pos > 0 && ip->pos0 && ip->sin_tab &&
                    ip->cos_tab && ip->q && ip->k_cache && ip->v_cache && ip->act && ip->ld_act >= N - 2 * d &&
                    (ip->act_dtype == MTJ_F32 || ip->act_dtype == MTJ_BF16) &&
                    (ip->q_dtype == MTJ_F32 || ip->q_dtype == MTJ_BF16) && (!ip->v_t || ip->ldvt >= ip->Tp),
                MTJ_EINVAL, "mtj_gemm: inconsistent INPROJ geometry");
  } else if (epi == MTJ_EPI_STORE) {
    MTJ_REQUIRE(out && ldo >= N && (out_dtype == MTJ_F32 || out_dtype == MTJ_BF16), MTJ_EINVAL,
                "mtj_gemm: STORE needs out with ldo >= N");
  } else if (epi == MTJ_EPI_RESID) {
    MTJ_REQUIRE(out && ldo >= N, MTJ_EINVAL, "mtj_gemm: RESID needs out with ldo >= N");
  } else {
    return mtj_fail(MTJ_EINVAL, "mtj_gemm: epilogue %d", epi);
  }
  hipStream_t s = (hipStream_t)stream;
  return dtype == MTJ_BF16 ? dispatch<bf16_t, 64>(a, s) : dispatch<float, 32>(a, s);
}

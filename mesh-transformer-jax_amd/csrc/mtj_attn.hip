// Attention: MFMA flash-style prefill over a left-padded rectangle, and one-token decode over the K/V window.
#include "mtj_common.h"
#include <type_traits>

namespace {

template <typename T> struct mma;
template <> struct mma<bf16_t> {
  static constexpr int EPC = 8;
  typedef uint16_t raw_t;
  struct frag { bf16x8 v; };
  __device__ static __forceinline__ frag load(const bf16_t* p) {
    frag f;
    f.v = *reinterpret_cast<const bf16x8*>(p);
    return f;
  }
  __device__ static __forceinline__ void pin(frag& f) { asm volatile("" : "+v"(f.v)); }
  __device__ static __forceinline__ frag from_floats(const float* p) {  // 8 probabilities -> operand
    frag f;
    uint32x4 u;
    u.x = pack_bf16x2(p[0], p[1]);
    u.y = pack_bf16x2(p[2], p[3]);
    u.z = pack_bf16x2(p[4], p[5]);
    u.w = pack_bf16x2(p[6], p[7]);
    f.v = *reinterpret_cast<bf16x8*>(&u);
    return f;
  }
  __device__ static __forceinline__ void run(floatx16& c, const frag& a, const frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
  }
  __device__ static __forceinline__ floatx16 first(const frag& a, const frag& b) {   // product alone: C is the constant 0
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, floatx16{}, 0, 0, 0);
  }
  // The same instruction spelled out, with the accumulator tied to vector registers (_v) or held in accumulation
  // registers that are named here and nowhere else (_fixed), for a kernel that fills the whole register file and cannot
  // leave the placement of its accumulators (and the copies it can entail) to the compiler.  The compiler does not know these are matrix instructions: the caller inserts the
  // wait states before other instructions read the result.
  __device__ static __forceinline__ void first_v(floatx16& c, const frag& a, const frag& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a.v), "v"(b.v));   // the result must not overlap an operand
  }
  __device__ static __forceinline__ void run_v(floatx16& c, const frag& a, const frag& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a.v), "v"(b.v));
  }
  // accumulator in the sixteen accumulation registers from a[BASE] on, which the compiler never sees
  template <int BASE> __device__ static __forceinline__ void run_fixed(const frag& a, const frag& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 a[%c2:%c2+15], %0, %1, a[%c2:%c2+15]" : : "v"(a.v), "v"(b.v), "n"(BASE));
  }
};
template <> struct mma<f16_t> {
  static constexpr int EPC = 8;
  typedef uint16_t raw_t;
  struct frag { f16x8 v; };
  __device__ static __forceinline__ frag load(const f16_t* p) {
    frag f;
    f.v = *reinterpret_cast<const f16x8*>(p);
    return f;
  }
  __device__ static __forceinline__ void pin(frag& f) { asm volatile("" : "+v"(f.v)); }
  // 8 probabilities -> operand; they lie in [0, 64], so the conversion needs no clamp to the float16 range
  __device__ static __forceinline__ frag from_floats(const float* p) {
    frag f;
#pragma unroll
    for (int j = 0; j < 8; ++j) f.v[j] = (f16_t)p[j];
    return f;
  }
  __device__ static __forceinline__ void run(floatx16& c, const frag& a, const frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.v, b.v, c, 0, 0, 0);
  }
  __device__ static __forceinline__ floatx16 first(const frag& a, const frag& b) {   // product alone: C is the constant 0
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a.v, b.v, floatx16{}, 0, 0, 0);
  }
  // The same instruction spelled out, with the accumulator tied to vector registers (_v) or held in accumulation
  // registers that are named here and nowhere else (_fixed), for a kernel that fills the whole register file and cannot
  // leave the placement of its accumulators (and the copies it can entail) to the compiler.  The compiler does not know these are matrix instructions: the caller inserts the
  // wait states before other instructions read the result.
  __device__ static __forceinline__ void first_v(floatx16& c, const frag& a, const frag& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a.v), "v"(b.v));   // the result must not overlap an operand
  }
  __device__ static __forceinline__ void run_v(floatx16& c, const frag& a, const frag& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a.v), "v"(b.v));
  }
  // accumulator in the sixteen accumulation registers from a[BASE] on, which the compiler never sees
  template <int BASE> __device__ static __forceinline__ void run_fixed(const frag& a, const frag& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 a[%c2:%c2+15], %0, %1, a[%c2:%c2+15]" : : "v"(a.v), "v"(b.v), "n"(BASE));
  }
};
template <> struct mma<float> {
  static constexpr int EPC = 4;
  typedef uint32_t raw_t;
  struct frag { float v[8]; };
  __device__ static __forceinline__ frag load(const float* p) {
    frag f;
    const floatx4 lo = *reinterpret_cast<const floatx4*>(p), hi = *reinterpret_cast<const floatx4*>(p + 4);
    f.v[0] = lo.x; f.v[1] = lo.y; f.v[2] = lo.z; f.v[3] = lo.w;
    f.v[4] = hi.x; f.v[5] = hi.y; f.v[6] = hi.z; f.v[7] = hi.w;
    return f;
  }
  __device__ static __forceinline__ void pin(frag&) {}
  __device__ static __forceinline__ frag from_floats(const float* p) {
    frag f;
#pragma unroll
    for (int j = 0; j < 8; ++j) f.v[j] = p[j];
    return f;
  }
  __device__ static __forceinline__ void run(floatx16& c, const frag& a, const frag& b) {
#pragma unroll
    for (int j = 0; j < 8; ++j) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[j], b.v[j], c, 0, 0, 0);
  }
};

// ------------------------------------------------------------------------------------------------
// Prefill.  Everything is computed transposed so that one lane owns one query: S^T = K Q^T gives each
// lane (query = lane % 32) sixteen keys of a 32-key block, the online-softmax state is lane-local, and
// O^T = V^T P^T is rescaled without any cross-lane traffic.  K rows are fetched in a permuted order so
// that the sixteen keys a lane ends up with are 8 consecutive ones per MFMA k-step - exactly the
// operand layout the second MFMA wants for P^T - and V comes pre-transposed ([dh][keys]).
//
// Workgroup: NW wavefronts x 32 queries; K / V^T tiles of BKV keys are staged global -> registers -> LDS,
// double-buffered (the loads of tile kt+1 are in flight while tile kt is multiplied).  The softmax runs in
// the exp2 domain with the hardware exponential; the accumulator is rescaled only when some lane's running
// maximum actually moved.
template <typename T, int DH, int NW, int BKV>
__global__ __launch_bounds__(NW * 64) void attn_prefill_kernel(const T* __restrict__ q, const T* __restrict__ kc,
                                                               const T* __restrict__ vt, const int32_t* __restrict__ pos0,
                                                               int H, int Tp, int Tcap, int64_t ldvt, T* __restrict__ out,
                                                               int64_t ld_out, int nseq, int nqblk,
                                                               const int32_t* __restrict__ key_limit) {
  constexpr int NT = NW * 64;
  constexpr int BQ = NW * 32;
  constexpr int EPC = mma<T>::EPC;
  using raw_t = typename mma<T>::raw_t;
  constexpr int KROW = DH + EPC;     // padded K row (elements)
  constexpr int VROW = BKV + EPC;    // padded V^T row
  constexpr int KS = DH / 16;        // MFMA k-steps over the head dim
  constexpr int NBLK = DH / 32;      // 32-wide blocks of the head dim in O^T
  constexpr int KB = BKV / 32;       // 32-key blocks per tile
  constexpr int CPRK = DH / EPC, CPRV = BKV / EPC;
  constexpr int K_CHUNKS = BKV * CPRK / NT, V_CHUNKS = DH * CPRV / NT;
  static_assert(BKV * CPRK % NT == 0 && DH * CPRV % NT == 0, "tile does not divide over threads");
  extern __shared__ __align__(16) unsigned char smem[];
  T* Ks = reinterpret_cast<T*>(smem);              // [2][BKV][KROW]
  T* Vs = Ks + 2 * BKV * KROW;                     // [2][DH][VROW]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int fr = lane & 31, fg = lane >> 5;
  // Workgroups are dispatched in blockIdx.x order: the head / sequence index varies fastest and the query block
  // slowest, latest block first, so that the longest workgroups of ALL heads start first and the tail of the
  // launch consists of short ones.
  const int hb = blockIdx.x % (H * nseq), qblk = blockIdx.x / (H * nseq);
  const int h = hb % H, b = hb / H;
  const int qt0 = (nqblk - 1 - qblk) * BQ;
  const int p0 = pos0[b];                       // <= 0: minus the number of padding rows
  const int t = qt0 + wave * 32 + fr;           // this lane's query (rectangle index)
  const int qpos = (t < Tp) ? t + p0 : -1;      // its position; < 0 = padding / out of range
  // last key this query may see: itself, or an earlier position when the caller masks the tail of the sequence
  const int klim = key_limit ? key_limit[b] : 0x7fffffff;
  const int qsee = qpos < klim ? qpos : klim;
  const int last_t = (qt0 + BQ - 1 < Tp - 1) ? qt0 + BQ - 1 : Tp - 1;
  const int kmax = last_t + p0;                 // last key any query of this workgroup may see
  const int klast = Tp - 1 + p0;                // last key position that exists for this sequence
  const int wave_last = qt0 + wave * 32 + 31 + p0;   // last key this wavefront may see
  // first query position of this wavefront if all 32 of its queries are real, else -1 (always mask)
  const int wave_first0 = (qt0 + wave * 32 + 31 < Tp) ? qt0 + wave * 32 + p0 : -1;
  const int wave_first = wave_first0 < klim ? wave_first0 : klim;
  const int64_t bh = (int64_t)b * H + h;

  // Q fragments (B operand of S^T): lane (query fr, half fg) holds Q[t][ks*16 + fg*8 .. +8)
  typename mma<T>::frag qf[KS];
  {
    const int tq = (t < Tp) ? t : Tp - 1;
    const T* qp = q + (bh * Tp + tq) * DH + fg * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = mma<T>::load(qp + ks * 16);
      mma<T>::pin(qf[ks]);   // or the compiler re-loads Q from global memory inside the key loop
    }
  }
  // row fr of an S^T block is key krow: rows {0-3, 4-7, 8-11, 12-15} <- keys {0-3, 8-11, 4-7, 12-15} (+16)
  const int krow = 16 * (fr >> 4) + 8 * ((fr >> 2) & 1) + 4 * ((fr >> 3) & 1) + (fr & 3);

  floatx16 o[NBLK];
#pragma unroll
  for (int i = 0; i < NBLK; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[i][v] = 0.f;
  float mrun = -INFINITY, lrun = 0.f;           // running max (log2 units) and sum
  const float sc2 = rsqrtf((float)DH) * 1.4426950408889634f;   // 1/sqrt(dh) * log2(e)

  // ---- staging
  uint32x4 rk[K_CHUNKS], rv[V_CHUNKS];
  // Loads are unconditional: K rows beyond the last key are clamped to it (the causal mask removes them), and a
  // V^T row is ldvt >= round_up(Tp, BKV) long, so the chunk exists; what it holds beyond the last key is zeroed
  // in LDS by fix_last_tile (0 x garbage must not become NaN).
  // Per-thread bases, so that a tile costs one scalar offset and no per-chunk address arithmetic: chunk i of the K
  // tile is row i * (NT / CPRK) + tid / CPRK, chunk i of the V^T tile is row i * (NT / CPRV) + tid / CPRV.
  static_assert(NT % CPRK == 0 && NT % CPRV == 0, "chunks of one pass start in the same column");
  const int k_row0 = tid / CPRK;
  const T* k_base = kc + bh * Tcap * DH + (tid % CPRK) * EPC;
  const T* v_base = vt + (bh * DH + tid / CPRV) * ldvt + (tid % CPRV) * EPC;
  const int64_t v_pass = (int64_t)(NT / CPRV) * ldvt;
  auto load_tile = [&](int kt) {
    const int key0 = kt * BKV;
    if (key0 + BKV - 1 <= klast) {             // workgroup-uniform: every row of the tile exists
      const T* kp = k_base + (int64_t)(key0 + k_row0) * DH;
#pragma unroll
      for (int i = 0; i < K_CHUNKS; ++i) rk[i] = *reinterpret_cast<const uint32x4*>(kp + i * (NT / CPRK) * DH);
    } else {
#pragma unroll
      for (int i = 0; i < K_CHUNKS; ++i) {
        const int row = key0 + k_row0 + i * (NT / CPRK);
        rk[i] = *reinterpret_cast<const uint32x4*>(k_base + (int64_t)(row <= klast ? row : klast) * DH);
      }
    }
    const T* vp = v_base + key0;
#pragma unroll
    for (int i = 0; i < V_CHUNKS; ++i) rv[i] = *reinterpret_cast<const uint32x4*>(vp + i * v_pass);
  };
  auto fix_last_tile = [&](int kt, int buf) {     // workgroup-uniform caller; runs between the store and the barrier
    const int key0 = kt * BKV;
    const int nbad = key0 + BKV - 1 - klast;       // columns klast+1-key0 .. BKV-1 of V^T do not exist
    if (nbad <= 0) return;
    raw_t* vs = reinterpret_cast<raw_t*>(Vs + buf * DH * VROW);
    for (int c = tid; c < DH * nbad; c += NT) vs[(c / nbad) * VROW + (BKV - nbad) + (c % nbad)] = (raw_t)0;
  };
  T* ks_dst = Ks + k_row0 * KROW + (tid % CPRK) * EPC;
  T* vs_dst = Vs + (tid / CPRV) * VROW + (tid % CPRV) * EPC;
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < K_CHUNKS; ++i)
      *reinterpret_cast<uint32x4*>(ks_dst + (buf * BKV + i * (NT / CPRK)) * KROW) = rk[i];
#pragma unroll
    for (int i = 0; i < V_CHUNKS; ++i)
      *reinterpret_cast<uint32x4*>(vs_dst + (buf * DH + i * (NT / CPRV)) * VROW) = rv[i];
  };

  const int ntiles = (kmax >= 0) ? kmax / BKV + 1 : 0;
  if (ntiles > 0) {
    load_tile(0);
    store_tile(0);
    __syncthreads();
    fix_last_tile(0, 0);
  }
  __syncthreads();
  for (int kt = 0; kt < ntiles; ++kt) {
    const int buf = kt & 1;
    const int key0 = kt * BKV;
    if (kt + 1 < ntiles) load_tile(kt + 1);
    if (key0 <= wave_last) {      // wave-uniform: tiles entirely above this wavefront's last query are skipped
      // ---- S^T blocks: rows = (permuted) keys, columns = queries.  The K fragments of k-steps
      // ks+G .. ks+2G-1 are read from LDS while the MFMAs of k-steps ks .. ks+G-1 run; the KB key blocks
      // give KB independent accumulation chains.
      floatx16 s[KB];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) s[kb][v] = 0.f;
      {
        constexpr int G = 2;                       // k-steps per group
        const T* kp = Ks + (buf * BKV + krow) * KROW + fg * 8;
        typename mma<T>::frag kf[2][KB][G];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int g = 0; g < G; ++g) kf[0][kb][g] = mma<T>::load(kp + kb * 32 * KROW + g * 16);
#pragma unroll
        for (int k0 = 0; k0 < KS; k0 += G) {
          const int cur = (k0 / G) & 1, nxt = cur ^ 1;
          if (k0 + G < KS) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
              for (int g = 0; g < G; ++g) kf[nxt][kb][g] = mma<T>::load(kp + kb * 32 * KROW + (k0 + G + g) * 16);
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int g = 0; g < G; ++g)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) mma<T>::run(s[kb], kf[cur][kb][g], qf[k0 + g]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // register v of block kb is key key0 + kb*32 + 16*(v/8) + 8*fg + v%8
      float mt = -INFINITY;
      if (key0 + BKV - 1 <= wave_first) {   // wave-uniform: the whole tile is below the diagonal for every lane
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            s[kb][v] *= sc2;
            mt = fmaxf(mt, s[kb][v]);
          }
      } else {
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = key0 + kb * 32 + 16 * (v / 8) + 8 * fg + (v % 8);
            s[kb][v] = (key <= qsee) ? s[kb][v] * sc2 : -INFINITY;
            mt = fmaxf(mt, s[kb][v]);
          }
      }
      mt = fmaxf(mt, __shfl_xor(mt, 32));
      // The running maximum only moves when a lane's tile maximum exceeds it by more than 2^6: the
      // probabilities then stay below 64 (harmless in float32 / bf16) and the rescale of the whole
      // accumulator, which costs as much as the MFMAs of a tile, happens in the first tiles only.
      if (__any(mt > mrun + 6.0f)) {
        const float mnew = fmaxf(mrun, mt);
        const float alpha = (mnew == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(mrun - mnew);   // mrun = -inf -> 0
        lrun *= alpha;
        // The accumulators live in the accumulation registers, which only the matrix instructions and copies can
        // address; the empty asm statements tie each block to those registers on both sides of its multiplication,
        // so that the copies out and back stay inside this rarely taken branch instead of the head of the key loop.
#pragma unroll
        for (int i = 0; i < NBLK; ++i) {
          if constexpr (sizeof(T) == 2) asm volatile("" : "+a"(o[i]));
#pragma unroll
          for (int v = 0; v < 16; ++v) o[i][v] *= alpha;
          if constexpr (sizeof(T) == 2) asm volatile("" : "+a"(o[i]));
        }
        mrun = mnew;
      }
      const float msafe = (mrun == -INFINITY) ? 0.f : mrun;
      float lt = 0.f;
      typename mma<T>::frag pf[KB][2];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        float p[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          p[v] = __builtin_amdgcn_exp2f(s[kb][v] - msafe);          // masked -> exp2(-inf) = 0
          lt += p[v];
        }
        pf[kb][0] = mma<T>::from_floats(p);
        pf[kb][1] = mma<T>::from_floats(p + 8);
      }
      lt += __shfl_xor(lt, 32);
      lrun += lt;
      // ---- O^T += V^T P^T : A = V^T rows (head-dim), B = P^T (keys x queries).  One 16-key k-step at a
      // time over all NBLK head-dim blocks (NBLK independent accumulators), fragments one k-step ahead.
      {
        constexpr int HB = NBLK > 4 ? 4 : NBLK;   // head-dim blocks per pass (bounds the live fragments)
        const T* vp = Vs + (buf * DH + fr) * VROW + fg * 8;
#pragma unroll
        for (int i0 = 0; i0 < NBLK; i0 += HB) {
          typename mma<T>::frag vf[2][HB];
#pragma unroll
          for (int i = 0; i < HB; ++i) vf[0][i] = mma<T>::load(vp + (i0 + i) * 32 * VROW);
#pragma unroll
          for (int st = 0; st < 2 * KB; ++st) {     // k-step st covers keys st*16 .. st*16+15 of the tile
            const int cur = st & 1, nxt = cur ^ 1;
            if (st + 1 < 2 * KB) {
#pragma unroll
              for (int i = 0; i < HB; ++i) vf[nxt][i] = mma<T>::load(vp + (i0 + i) * 32 * VROW + (st + 1) * 16);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < HB; ++i) mma<T>::run(o[i0 + i], vf[cur][i], pf[st / 2][st % 2]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
    }
    if (kt + 1 < ntiles) {
      store_tile(buf ^ 1);
      if ((kt + 2) * BKV - 1 > klast) {     // only the last tile of a sequence can be partial
        __syncthreads();
        fix_last_tile(kt + 1, buf ^ 1);
      }
    }
    __syncthreads();
  }

  // ---- write O: register v of block i is head-dim i*32 + 8*(v/4) + 4*fg + v%4 of query t
  if (t < Tp) {
    const float inv = (qpos >= 0 && lrun > 0.f) ? 1.0f / lrun : 0.f;
    T* op = out + ((int64_t)b * Tp + t) * ld_out + (int64_t)h * DH;
#pragma unroll
    for (int i = 0; i < NBLK; ++i)
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const int e = i * 32 + 8 * v4 + 4 * fg;
        if constexpr (sizeof(T) == 2) {
          uint32x2 pk;
          pk.x = pack2<T>(o[i][v4 * 4] * inv, o[i][v4 * 4 + 1] * inv);
          pk.y = pack2<T>(o[i][v4 * 4 + 2] * inv, o[i][v4 * 4 + 3] * inv);
          *reinterpret_cast<uint32x2*>(op + e) = pk;
        } else {
          *reinterpret_cast<floatx4*>(op + e) =
              floatx4{o[i][v4 * 4] * inv, o[i][v4 * 4 + 1] * inv, o[i][v4 * 4 + 2] * inv, o[i][v4 * 4 + 3] * inv};
        }
      }
  }
}

// ------------------------------------------------------------------------------------------------
// Prefill for 16-bit types at d_head 256: the same mathematics and the same lane layout as attn_prefill_kernel (one
// lane owns one query, S^T = K Q^T, O^T = V^T P^T, K rows permuted so that the scores land in the operand layout of the
// second product), but each block of 32 queries is worked on by a PAIR of wavefronts that share a SIMD (wave w and
// w + 4 of an 8-wavefront workgroup, 128 queries per workgroup):
//   the score wavefront (w < 4) holds Q and computes the scores of key tile i, their running maximum and the rescale
//     factor, and hands score - maximum to its partner through LDS;
//   the value wavefront (w + 4) holds the output accumulator and the running sum, turns the scores of tile i-1 into
//     probabilities (the exponentials) and multiplies them with V^T; it also issues every global -> LDS load.
// An iteration is two phases separated by workgroup barriers: [scores of tile i | exponentials of tile i-1], then
// [maximum of tile i | P V of tile i-1], so the two wavefronts of a SIMD take turns on the matrix pipe and each one's
// vector arithmetic runs under the other's MFMAs; with one wavefront per SIMD doing all of it in sequence the matrix
// pipe was busy a quarter of the time.  K and V^T tiles of 32 keys go global -> LDS without passing through registers
// (buffer_load ... lds), four stages each, requested three (K) and two (V^T) tiles ahead; rows are unpadded and the
// 16-byte chunks of a row are xor-swizzled (K: low four bits of the chunk index with the row, V^T: the two bits with
// (row / 4) % 4) so that the fragment reads of 16 consecutive rows hit 16 distinct bank groups.  Loads beyond the last
// tile re-read the last tile (into a stage nobody reads again), which keeps the wait count the same in every iteration.
constexpr int PP_STAGES = 4, PP_KTILE = 32 * 256 * 2, PP_VTILE = 256 * 32 * 2;
constexpr int PP_LDS_K = 0, PP_LDS_V = PP_STAGES * PP_KTILE, PP_LDS_S = PP_LDS_V + PP_STAGES * PP_VTILE;
constexpr int PP_LDS_A = PP_LDS_S + 4 * 4096, PP_LDS_F = PP_LDS_A + 4 * 512, PP_LDS_BYTES = PP_LDS_F + 64;

// sum of eight 16-bit probabilities as the second product will see them (after rounding), added to acc
template <typename T> struct psum;
template <> struct psum<f16_t> {
  __device__ static __forceinline__ float run(const typename mma<f16_t>::frag& f, float acc) {
    const f16x2 one = {(f16_t)1.f, (f16_t)1.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_fdot2(f16x2{f.v[2 * j], f.v[2 * j + 1]}, one, acc, false);
    return acc;
  }
};
template <> struct psum<bf16_t> {
  __device__ static __forceinline__ float run(const typename mma<bf16_t>::frag& f, float acc) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc += (float)f.v[j];
    return acc;
  }
};

template <typename T>
__global__ __launch_bounds__(512) void attn_prefill_pair_kernel(const T* __restrict__ q, const T* __restrict__ kc,
                                                                const T* __restrict__ vt, const int32_t* __restrict__ pos0,
                                                                int H, int Tp, int Tcap, int64_t ldvt, T* __restrict__ out,
                                                                int64_t ld_out, int nseq, int nqblk,
                                                                const int32_t* __restrict__ key_limit) {
  static_assert(sizeof(T) == 2, "16-bit types");
  constexpr int DH = 256, BKV = 32, BQ = 128, KS = DH / 16, NBLK = DH / 32;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pw = wave & 3;                      // which 32 queries of the workgroup
  const bool value_role = wave >= 4;
  const int fr = lane & 31, fg = lane >> 5;
  const int hb = blockIdx.x % (H * nseq), qblk = blockIdx.x / (H * nseq);
  const int h = hb % H, b = hb / H;
  const int qt0 = (nqblk - 1 - qblk) * BQ;      // longest workgroups first
  const int t = qt0 + pw * 32 + fr;             // this lane's query (rectangle index)
  const int64_t bh = (int64_t)b * H + h;

  float* sx = reinterpret_cast<float*>(smem + PP_LDS_S + pw * 4096) + lane * 4;   // + v4 * 256 floats
  float* ax = reinterpret_cast<float*>(smem + PP_LDS_A + pw * 512) + lane;        // rescale factor, + 64: minus the maximum
  int* fx = reinterpret_cast<int*>(smem + PP_LDS_F) + pw;
  const float sc2 = rsqrtf((float)DH) * 1.4426950408889634f;   // 1/sqrt(dh) * log2(e): probabilities are 2^(s*sc2 - max)

  // Requests that do not depend on the sequence's padding go out before it is known: Q, and the first three K tiles and
  // two V^T tiles (a row or column index beyond the buffers is clamped into them; such a tile is never read).
  typename mma<T>::frag qf[KS];
  const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(kc + bh * Tcap * DH), 0, (int)((int64_t)Tcap * DH * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(vt + bh * DH * ldvt), 0, (int)((int64_t)DH * ldvt * 2), 0x00020000);
  // global -> LDS loads.  K tile: 32 rows x 512 bytes = 16 wavefront loads of 2 rows, load j = 4*wb + jj; lane l fills
  // position l % 32 of row 2j + l / 32 with chunk (p & 16) | ((p & 15) ^ (row & 15)).  V^T tile: 256 rows x 64 bytes =
  // 16 loads of 16 rows; lane l fills position l % 4 of row 16j + l / 4 with chunk (l % 4) ^ ((row / 4) % 4).
  const int wb = wave & 3;
  int k_row[4], k_chunk[4], k_off[4], v_off[4];
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    const int j = 4 * wb + jj;
    k_row[jj] = 2 * j + (lane >> 5);
    const int kp_l = lane & 31;
    k_chunk[jj] = ((kp_l & 16) | ((kp_l & 15) ^ (k_row[jj] & 15))) * 16;
    k_off[jj] = k_row[jj] * 512 + k_chunk[jj];
    const int vrow_l = 16 * j + (lane >> 2);
    v_off[jj] = (int)((int64_t)vrow_l * ldvt * 2) + (((lane & 3) ^ ((vrow_l >> 2) & 3)) * 16);
  }
  auto issue_k1 = [&](int stage_tile, int tile, auto JJ_) {
    constexpr int jj = decltype(JJ_)::value;
    unsigned char* dst = smem + PP_LDS_K + (stage_tile & (PP_STAGES - 1)) * PP_KTILE + wb * 4096 + jj * 1024;
    // rows beyond the last key are masked by their readers; rows beyond the window repeat its last row
    if (tile * BKV + BKV <= Tcap) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (lds_ptr)dst, 16, k_off[jj] + tile * (BKV * 512), 0, 0, 0);
    } else {
      const int row = tile * BKV + k_row[jj];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (lds_ptr)dst, 16, (row < Tcap ? row : Tcap - 1) * 512 + k_chunk[jj], 0, 0, 0);
    }
  };
  auto issue_v1 = [&](int stage_tile, int tile, auto JJ_) {
    constexpr int jj = decltype(JJ_)::value;
    unsigned char* dst = smem + PP_LDS_V + (stage_tile & (PP_STAGES - 1)) * PP_VTILE + wb * 4096 + jj * 1024;
    const int col = (int64_t)tile * BKV + BKV <= ldvt ? tile * BKV : (int)ldvt - BKV;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (lds_ptr)dst, 16, v_off[jj] + col * 2, 0, 0, 0);
  };
  using J0 = std::integral_constant<int, 0>;
  using J1 = std::integral_constant<int, 1>;
  using J2 = std::integral_constant<int, 2>;
  using J3 = std::integral_constant<int, 3>;
  auto issue_k = [&](int st, int tile) { issue_k1(st, tile, J0{}); issue_k1(st, tile, J1{}); issue_k1(st, tile, J2{}); issue_k1(st, tile, J3{}); };
  auto issue_v = [&](int st, int tile) { issue_v1(st, tile, J0{}); issue_v1(st, tile, J1{}); issue_v1(st, tile, J2{}); issue_v1(st, tile, J3{}); };
  if (value_role) {
    issue_k(0, 0); issue_v(0, 0); issue_k(1, 1); issue_v(1, 1); issue_k(2, 2);
  } else {
    const int tq = (t < Tp) ? t : Tp - 1;
    const T* qp = q + (bh * Tp + tq) * DH + fg * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = mma<T>::load(qp + ks * 16);
  }

  const int p0 = pos0[b];                       // <= 0: minus the number of padding rows
  const int qpos = (t < Tp) ? t + p0 : -1;      // its position; < 0 = padding / out of range
  const int klim = key_limit ? key_limit[b] : 0x7fffffff;
  const int qsee = qpos < klim ? qpos : klim;   // last key this query may see
  const int last_t = (qt0 + BQ - 1 < Tp - 1) ? qt0 + BQ - 1 : Tp - 1;
  const int kmax = last_t + p0;                 // last key any query of this workgroup may see
  const int klast = Tp - 1 + p0;                // last key position that exists for this sequence
  const int wave_last = qt0 + pw * 32 + 31 + p0;     // last key this pair may see
  const int wave_first0 = (qt0 + pw * 32 + 31 < Tp) ? qt0 + pw * 32 + p0 : -1;
  const int wave_first = wave_first0 < klim ? wave_first0 : klim;
  const int ntiles = (kmax >= 0) ? kmax / BKV + 1 : 0;

  if (!value_role) {
    // ---------------- score wavefront
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) mma<T>::pin(qf[ks]);   // pinned, or Q is re-loaded inside the key loop
    // row fr of an S^T block is key krow: rows {0-3, 4-7, 8-11, 12-15} <- keys {0-3, 8-11, 4-7, 12-15} (+16)
    const int krow = 16 * (fr >> 4) + 8 * ((fr >> 2) & 1) + 4 * ((fr >> 3) & 1) + (fr & 3);
    const int kx = (krow & 15) ^ fg;            // chunk 2*ks + fg of row krow sits at ((2*(ks%8)) ^ kx) + 16*(ks/8)
    float mrun = -INFINITY;                     // running maximum of s * sc2
    typename mma<T>::frag kf[KS];
    int kxo[8];                                 // byte offset of chunk 2*k + fg of my row inside a 256-byte half row
#pragma unroll
    for (int k = 0; k < 8; ++k) kxo[k] = krow * 512 + (((2 * k) ^ kx) * 16);
    auto read_k = [&](int tile, int ks_lo, int ks_hi) {
      const unsigned char* kp = smem + PP_LDS_K + (tile & (PP_STAGES - 1)) * PP_KTILE;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        if (ks >= ks_lo && ks < ks_hi) kf[ks] = mma<T>::load(reinterpret_cast<const T*>(kp + kxo[ks & 7] + (ks >> 3) * 256));
    };
    __builtin_amdgcn_s_barrier();               // tile 0 has landed (the value wavefronts waited for it)
    if (ntiles > 0) read_k(0, 0, 8);
    for (int i = 0; i <= ntiles; ++i) {
      const int key0 = i * BKV;
      const bool active = i < ntiles && key0 <= wave_last;
      floatx16 s;
      if (active) {
        // one accumulation chain (dependent MFMAs of one shape issue back to back); the fragments of k-steps 0-7 were
        // fetched in the previous phase, those of k-steps 8-15 arrive under the first eight MFMAs
        read_k(i, 8, 16);
        __builtin_amdgcn_sched_barrier(0);
        s = mma<T>::first(kf[0], qf[0]);
#pragma unroll
        for (int ks = 1; ks < KS; ++ks) mma<T>::run(s, kf[ks], qf[ks]);
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_barrier();
      if (active) {
        // register v is key key0 + 16*(v/8) + 8*fg + v%8
        if (key0 + BKV - 1 > wave_first) {      // the diagonal crosses the tile: hide what a query may not see
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = key0 + 16 * (v / 8) + 8 * fg + (v % 8);
            s[v] = (key <= qsee) ? s[v] : -INFINITY;
          }
        }
        float mt = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
        for (int v = 3; v < 15; v += 2) mt = fmaxf(fmaxf(mt, s[v]), s[v + 1]);
        mt = fmaxf(mt, s[15]) * sc2;            // sc2 > 0
        mt = max_halves(mt);
        // the running maximum only moves when some lane's tile maximum exceeds it by more than 2^6 (probabilities stay
        // below 64), so the partner rescales its accumulator in the first tiles only
        const bool moved = __any(mt > mrun + 6.0f);
        if (moved) {
          const float mnew = fmaxf(mrun, mt);
          *ax = (mnew == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(mrun - mnew);   // mrun = -inf -> 0
          mrun = mnew;
          ax[64] = (mrun == -INFINITY) ? 0.f : -mrun;
        }
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4)
          *reinterpret_cast<floatx4*>(sx + v4 * 256) = floatx4{s[4 * v4], s[4 * v4 + 1], s[4 * v4 + 2], s[4 * v4 + 3]};
        if (lane == 0) *fx = moved ? 1 : 0;
      }
      // K tile i+1 has landed (the value wavefronts waited for it before the barrier above)
      if (i + 1 < ntiles && key0 + BKV <= wave_last) read_k(i + 1, 0, 8);
      __builtin_amdgcn_s_barrier();
    }
    return;
  }

  // ---------------- value wavefront
  floatx16 o[NBLK];
#pragma unroll
  for (int i = 0; i < NBLK; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[i][v] = 0.f;
  float lrun = 0.f, mneg = 0.f;
  __builtin_amdgcn_s_waitcnt(wait_vmcnt(12));               // tile 0 of K and V^T
  __builtin_amdgcn_s_barrier();

  const int vx = (fr >> 2) & 3;
  const unsigned char* vbase = smem + PP_LDS_V + fr * 64;
  const int vpos0 = ((0 + fg) ^ vx) * 16, vpos1 = ((2 + fg) ^ vx) * 16;
  const int last = ntiles > 0 ? ntiles - 1 : 0;
  for (int i = 0; i <= ntiles; ++i) {
    // ---- phase 1: the probabilities of tile i-1 and its V^T fragments
    const int tk3 = i + 3 < last ? i + 3 : last, tv2 = i + 2 < last ? i + 2 : last;   // the tiles requested in phase 2
    const int tv = i - 1;
    const bool active = tv >= 0 && tv * BKV <= wave_last;
    typename mma<T>::frag pf[2], vf[2][NBLK];
    if (active) {
      const unsigned char* vp = vbase + (tv & (PP_STAGES - 1)) * PP_VTILE;
      // the last tile of a sequence can be partial: what V^T holds beyond the last key must not reach the product
      // (0 x garbage may be NaN).  Every value wavefront clears all of it before its own reads (LDS operations of one
      // wavefront stay in order), so no barrier is needed.
      const int nbad = tv * BKV + BKV - 1 - klast;
      if (nbad > 0) {
        uint16_t* vs = reinterpret_cast<uint16_t*>(smem + PP_LDS_V + (tv & (PP_STAGES - 1)) * PP_VTILE);
        for (int c = lane; c < DH * nbad; c += 64) {
          const int row = c / nbad, col = BKV - nbad + (c % nbad);
          vs[row * 32 + (((col >> 3) ^ ((row >> 2) & 3)) * 8) + (col & 7)] = (uint16_t)0;
        }
      }
      float p[16];
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const floatx4 sv = *reinterpret_cast<const floatx4*>(sx + v4 * 256);
        p[4 * v4] = sv.x; p[4 * v4 + 1] = sv.y; p[4 * v4 + 2] = sv.z; p[4 * v4 + 3] = sv.w;
      }
      const int moved = *fx;
#pragma unroll
      for (int n = 0; n < NBLK; ++n) vf[0][n] = mma<T>::load(reinterpret_cast<const T*>(vp + n * 2048 + vpos0));
#pragma unroll
      for (int n = 0; n < NBLK; ++n) vf[1][n] = mma<T>::load(reinterpret_cast<const T*>(vp + n * 2048 + vpos1));
      if (moved) {
        const float alpha = *ax;
        mneg = ax[64];
        lrun *= alpha;
#pragma unroll
        for (int n = 0; n < NBLK; ++n)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[n][v] *= alpha;
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) p[v] = __builtin_amdgcn_exp2f(fmaf(p[v], sc2, mneg));   // masked -> exp2(-inf) = 0
      pf[0] = mma<T>::from_floats(p);
      pf[1] = mma<T>::from_floats(p + 8);
      float lt = psum<T>::run(pf[1], psum<T>::run(pf[0], 0.f));
      lrun += sum_halves(lt);
    }
    __builtin_amdgcn_s_waitcnt(wait_vmcnt(8));              // K of tile i+1 and V^T of tile i have landed
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase 2: O^T += V^T P^T, and the requests for K tile i+3 and V^T tile i+2 (their stages were last read in
    // iteration i-1), one per two MFMAs.  (Issued by the score wavefronts instead, whose second phase is the longer
    // one, the kernel is 5 % slower.)
    if (active) {
      mma<T>::run(o[0], vf[0][0], pf[0]); mma<T>::run(o[1], vf[0][1], pf[0]);
      __builtin_amdgcn_sched_barrier(0); issue_k1(i + 3, tk3, J0{}); __builtin_amdgcn_sched_barrier(0);
      mma<T>::run(o[2], vf[0][2], pf[0]); mma<T>::run(o[3], vf[0][3], pf[0]);
      __builtin_amdgcn_sched_barrier(0); issue_k1(i + 3, tk3, J1{}); __builtin_amdgcn_sched_barrier(0);
      mma<T>::run(o[4], vf[0][4], pf[0]); mma<T>::run(o[5], vf[0][5], pf[0]);
      __builtin_amdgcn_sched_barrier(0); issue_k1(i + 3, tk3, J2{}); __builtin_amdgcn_sched_barrier(0);
      mma<T>::run(o[6], vf[0][6], pf[0]); mma<T>::run(o[7], vf[0][7], pf[0]);
      __builtin_amdgcn_sched_barrier(0); issue_k1(i + 3, tk3, J3{}); __builtin_amdgcn_sched_barrier(0);
      mma<T>::run(o[0], vf[1][0], pf[1]); mma<T>::run(o[1], vf[1][1], pf[1]);
      __builtin_amdgcn_sched_barrier(0); issue_v1(i + 2, tv2, J0{}); __builtin_amdgcn_sched_barrier(0);
      mma<T>::run(o[2], vf[1][2], pf[1]); mma<T>::run(o[3], vf[1][3], pf[1]);
      __builtin_amdgcn_sched_barrier(0); issue_v1(i + 2, tv2, J1{}); __builtin_amdgcn_sched_barrier(0);
      mma<T>::run(o[4], vf[1][4], pf[1]); mma<T>::run(o[5], vf[1][5], pf[1]);
      __builtin_amdgcn_sched_barrier(0); issue_v1(i + 2, tv2, J2{}); __builtin_amdgcn_sched_barrier(0);
      mma<T>::run(o[6], vf[1][6], pf[1]); mma<T>::run(o[7], vf[1][7], pf[1]);
      __builtin_amdgcn_sched_barrier(0); issue_v1(i + 2, tv2, J3{}); __builtin_amdgcn_sched_barrier(0);
    } else {
      issue_k(i + 3, tk3);
      issue_v(i + 2, tv2);
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));                // the surplus loads land before the LDS is given away

  // ---- write O: register v of block n is head-dim n*32 + 8*(v/4) + 4*fg + v%4 of query t
  if (t < Tp) {
    const float inv = (qpos >= 0 && lrun > 0.f) ? 1.0f / lrun : 0.f;
    T* op = out + ((int64_t)b * Tp + t) * ld_out + (int64_t)h * DH;
#pragma unroll
    for (int n = 0; n < NBLK; ++n)
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const int e = n * 32 + 8 * v4 + 4 * fg;
        uint32x2 pk;
        pk.x = pack2<T>(o[n][v4 * 4] * inv, o[n][v4 * 4 + 1] * inv);
        pk.y = pack2<T>(o[n][v4 * 4 + 2] * inv, o[n][v4 * 4 + 3] * inv);
        *reinterpret_cast<uint32x2*>(op + e) = pk;
      }
  }
}

// ------------------------------------------------------------------------------------------------
// Prefill for 16-bit types at d_head 256, long prompts: ONE wavefront per SIMD that owns 64 queries (two blocks of 32)
// and does everything for them, four wavefronts = 256 queries per workgroup.  With 32 queries per wavefront (the pair
// kernel above) every 1 KiB K or V^T fragment read from LDS feeds one matrix instruction, and LDS traffic (~200 KB per
// 32-key tile and CU for 1024 matrix-pipe cycles) is what bounds that kernel; here a fragment feeds two, one per query
// block, for the price of the register budget of a whole SIMD: Q 128 registers, the output accumulator 256, scores 32,
// probabilities of two tiles 32.  The matrix pipe and the vector unit overlap inside the wavefront instead of across
// a pair: iteration i first computes the scores of tile i (K Q^T), then issues the products V^T P^T of tile i-1
// together with the softmax arithmetic of tile i, which the matrix instructions (32 cycles apiece, asynchronous) hide.
// Same lane layout, K row permutation, LDS stages, xor swizzles and global -> LDS loads as the pair kernel; one
// workgroup barrier per tile.
constexpr int Q64_LDS_BYTES = PP_STAGES * (PP_KTILE + PP_VTILE);

// The output accumulator of attn_prefill_q64_kernel lives in all 256 accumulation registers, addressed by number from
// inline assembly only: block (qb, n) - 32 head dims x 32 queries - is a[(qb * 8 + n) * 16 .. + 15].  The clobber list
// names every one of them once, which takes them out of the compiler's hands for good (it uses accumulation registers
// that the function does not mention as spill space for vector registers).
#define Q64_A8(n) "a" #n "0", "a" #n "1", "a" #n "2", "a" #n "3", "a" #n "4", "a" #n "5", "a" #n "6", "a" #n "7", "a" #n "8", "a" #n "9"
#define Q64_ALL_ACC                                                                                                      \
  "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", Q64_A8(1), Q64_A8(2), Q64_A8(3), Q64_A8(4), Q64_A8(5),     \
      Q64_A8(6), Q64_A8(7), Q64_A8(8), Q64_A8(9), Q64_A8(10), Q64_A8(11), Q64_A8(12), Q64_A8(13), Q64_A8(14), Q64_A8(15), \
      Q64_A8(16), Q64_A8(17), Q64_A8(18), Q64_A8(19), Q64_A8(20), Q64_A8(21), Q64_A8(22), Q64_A8(23), Q64_A8(24),         \
      "a250", "a251", "a252", "a253", "a254", "a255"
__device__ __forceinline__ void acc_zero_all() {
  asm volatile(".set mtj_r, 0\n\t.rept 256\n\tv_accvgpr_write_b32 a[mtj_r], 0\n\t.set mtj_r, mtj_r+1\n\t.endr" : : : Q64_ALL_ACC);
}
template <int BASE> __device__ __forceinline__ void acc_scale16(float f) {        // a[BASE .. BASE+15] *= f
  float tmp;
  asm volatile(".set mtj_r, %c2\n\t.rept 16\n\tv_accvgpr_read_b32 %0, a[mtj_r]\n\tv_mul_f32 %0, %0, %1\n\t"
               "v_accvgpr_write_b32 a[mtj_r], %0\n\t.set mtj_r, mtj_r+1\n\t.endr"
               : "=&v"(tmp) : "v"(f), "n"(BASE));
}
template <int R> __device__ __forceinline__ float acc_read() {
  float t;
  asm volatile("v_accvgpr_read_b32 %0, a[%c1]" : "=v"(t) : "n"(R));
  return t;
}
// max(a, b, c) in one instruction; the operands come out of matrix instructions, where the compiler would first
// canonicalise each of them
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// two probabilities -> one word of 16-bit operands, no clamp: they are at most 64 wherever the result is used
template <typename T> __device__ __forceinline__ uint32_t pack_prob(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack_prob<bf16_t>(float lo, float hi) { return pack_bf16x2(lo, hi); }
template <> __device__ __forceinline__ uint32_t pack_prob<f16_t>(float lo, float hi) {
  const f16x2 r = {(f16_t)lo, (f16_t)hi};
  return __builtin_bit_cast(uint32_t, r);
}
// f(integral_constant<int, K>) for K = 0 .. N-1, in order
template <int N, int K = 0, class F> __device__ __forceinline__ void static_for(F&& f) {
  if constexpr (K < N) {
    f(std::integral_constant<int, K>{});
    static_for<N, K + 1>(f);
  }
}


template <typename T>
__global__ __launch_bounds__(256) void attn_prefill_q64_kernel(const T* __restrict__ q, const T* __restrict__ kc,
                                                               const T* __restrict__ vt, const int32_t* __restrict__ pos0,
                                                               int H, int Tp, int Tcap, int64_t ldvt, T* __restrict__ out,
                                                               int64_t ld_out, int nseq, int nqblk,
                                                               const int32_t* __restrict__ key_limit) {
  static_assert(sizeof(T) == 2, "16-bit types");
  constexpr int DH = 256, BKV = 32, BQ = 256, KS = DH / 16, NBLK = DH / 32;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int fr = lane & 31, fg = lane >> 5;
  // A workgroup takes query block nqblk-1-j of a (sequence, head) and then block j: under the causal mask block k costs
  // k+1 units, so every workgroup costs the same (no longest-first dispatch, no tail), and the workgroups of one
  // (sequence, head) start together and walk the key tiles of their long blocks in step.  They are also given to ONE
  // XCD (workgroups are handed to the XCDs round robin), so that a K / V^T tile is fetched from memory once and found in
  // that XCD's L2 by the others: fetched per query block from wherever it lies, the tiles were what bounded the kernel
  // (1.2 GB per layer at 8 x 2048 tokens, ~5 TB/s).
  const int nq2 = (nqblk + 1) / 2, npair = H * nseq;
  int hb, j;
  if (npair % 8 == 0) {
    const int x = blockIdx.x & 7, r = blockIdx.x >> 3;
    hb = (r / nq2) * 8 + x;
    j = r % nq2;
  } else {
    hb = blockIdx.x % npair;
    j = blockIdx.x / npair;
  }
  const int h = hb % H, b = hb / H;
  const int64_t bh = (int64_t)b * H + h;
  const float sc2 = rsqrtf((float)DH) * 1.4426950408889634f;   // 1/sqrt(dh) * log2(e): probabilities are 2^(s*sc2 - max)
  const int nparts = (nqblk - 1 - j == j) ? 1 : 2;
#pragma nounroll
  for (int part = 0; part < nparts; ++part) {
  const int qt0 = (part == 0 ? nqblk - 1 - j : j) * BQ;

  // Q fragments of my two query blocks (B operand of S^T): lane (query fr, half fg) holds Q[t][ks*16 + fg*8 .. +8)
  typename mma<T>::frag qf[2][KS];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int t = qt0 + wave * 64 + qb * 32 + fr;
    const T* qp = q + (bh * Tp + (t < Tp ? t : Tp - 1)) * DH + fg * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[qb][ks] = mma<T>::load(qp + ks * 16);
  }
  const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(kc + bh * Tcap * DH), 0, (int)((int64_t)Tcap * DH * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(vt + bh * DH * ldvt), 0, (int)((int64_t)DH * ldvt * 2), 0x00020000);
  // global -> LDS loads: a K tile is 16 wavefront loads of 2 rows (lane l fills position l % 32 of row 2j + l / 32 with
  // chunk (p & 16) | ((p & 15) ^ (row & 15))), a V^T tile 16 loads of 16 rows (lane l fills position l % 4 of row
  // 16j + l / 4 with chunk (l % 4) ^ ((row / 4) % 4)).  Wavefront w issues K loads j = 4jj + w and V^T loads j = 4w + jj,
  // jj = 0 .. 3: the per-lane part of the address then depends on jj through one bit for K (row & 8) and not at all for
  // V^T, and the rest is a scalar offset - three address registers instead of sixteen in a kernel that has none to spare.
  const int k_row0 = 2 * wave + (lane >> 5);                                   // row of load jj: k_row0 + 8 jj
  const int k_lo = k_row0 * 512 + (((lane & 16) | ((lane & 15) ^ (k_row0 & 15))) * 16);
  const int v_lo = (int)((int64_t)(64 * wave + (lane >> 2)) * ldvt * 2) + (((lane & 3) ^ ((lane >> 4) & 3)) * 16);
  const int v_step = (int)(ldvt * 32);                                         // 16 rows of V^T
  auto issue_k1 = [&](int stage_tile, int tile, int jj) {
    unsigned char* dst = smem + PP_LDS_K + (stage_tile & (PP_STAGES - 1)) * PP_KTILE + jj * 4096 + wave * 1024;
    const int lo = (jj & 1) ? (k_lo ^ 128) : k_lo;
    if (tile * BKV + BKV <= Tcap) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (lds_ptr)dst, 16, lo, tile * (BKV * 512) + jj * 4096, 0, 0);
    } else {      // rows beyond the window repeat its last row; their readers mask them
      const int row = tile * BKV + k_row0 + 8 * jj;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (lds_ptr)dst, 16, (row < Tcap ? row : Tcap - 1) * 512 + (lo & 511), 0, 0, 0);
    }
  };
  auto issue_v1 = [&](int stage_tile, int tile, int jj) {
    const int col = (int64_t)tile * BKV + BKV <= ldvt ? tile * BKV : (int)ldvt - BKV;
    unsigned char* dst = smem + PP_LDS_V + (stage_tile & (PP_STAGES - 1)) * PP_VTILE + wave * 4096 + jj * 1024;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (lds_ptr)dst, 16, v_lo, col * 2 + jj * v_step, 0, 0);
  };
  auto issue_k = [&](int stage_tile, int tile) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) issue_k1(stage_tile, tile, jj);
  };
  auto issue_v = [&](int stage_tile, int tile) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) issue_v1(stage_tile, tile, jj);
  };
  // tiles 0 .. 2 of K and 0 .. 1 of V^T go out before the sequence's padding is known (indices beyond the buffers are
  // clamped into them; such a tile is never read)
  issue_k(0, 0); issue_v(0, 0); issue_k(1, 1); issue_v(1, 1); issue_k(2, 2);
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) mma<T>::pin(qf[qb][ks]);   // pinned, or Q is re-loaded inside the key loop

  const int p0 = pos0[b];                       // <= 0: minus the number of padding rows
  const int klim = key_limit ? key_limit[b] : 0x7fffffff;
  int qsee[2], wave_first[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int t = qt0 + wave * 64 + qb * 32 + fr;
    const int qpos = (t < Tp) ? t + p0 : -1;    // this lane's position in block qb; < 0 = padding / out of range
    qsee[qb] = qpos < klim ? qpos : klim;       // last key this query may see
    const int wf0 = (qt0 + wave * 64 + qb * 32 + 31 < Tp) ? qt0 + wave * 64 + qb * 32 + p0 : -1;
    wave_first[qb] = wf0 < klim ? wf0 : klim;   // a tile that ends at or below this needs no mask in block qb
  }
  const int last_t = (qt0 + BQ - 1 < Tp - 1) ? qt0 + BQ - 1 : Tp - 1;
  const int kmax = last_t + p0;                 // last key any query of this workgroup may see
  const int klast = Tp - 1 + p0;                // last key position that exists for this sequence
  const int wave_last = qt0 + wave * 64 + 63 + p0;   // last key this wavefront may see
  const int ntiles = (kmax >= 0) ? kmax / BKV + 1 : 0;
  const int last = ntiles > 0 ? ntiles - 1 : 0;

  // row fr of an S^T block is key krow: rows {0-3, 4-7, 8-11, 12-15} <- keys {0-3, 8-11, 4-7, 12-15} (+16)
  const int krow = 16 * (fr >> 4) + 8 * ((fr >> 2) & 1) + 4 * ((fr >> 3) & 1) + (fr & 3);
  const int kx = (krow & 15) ^ fg;              // chunk 2*ks + fg of row krow sits at ((2*(ks%8)) ^ kx) + 16*(ks/8)
  const int kbase = krow * 512;
  // worked out at every read: the score phase has vector-unit slots to spare, the register file has nothing
  auto kxo = [&](int k) { return kbase + (((2 * k) ^ kx) << 4); };
  const int vx = (fr >> 2) & 3;
  const unsigned char* vbase = smem + PP_LDS_V + fr * 64;
  const int vpos[2] = {((0 + fg) ^ vx) * 16, ((2 + fg) ^ vx) * 16};

  acc_zero_all();                               // the output accumulator: a[0:255], see above
  float mrun[2] = {-INFINITY, -INFINITY}, lrun[2] = {0.f, 0.f};
  typename mma<T>::frag pf[2][2];               // probabilities of the previous tile: [query block][16-key half]
  bool prev_active = false;

  for (int i = 0; i <= ntiles; ++i) {
    const int key0 = i * BKV;
    // K tile i and V^T tile i-1 have landed once at most the 16 loads of the last two iterations are outstanding; the
    // barrier also says that every wavefront is done with the stages that are requested next
    __builtin_amdgcn_s_waitcnt(wait_vmcnt(16));
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    const int tk3 = i + 3 < last ? i + 3 : last, tv2 = i + 2 < last ? i + 2 : last;   // the tiles requested in this iteration
    const bool active = i < ntiles && key0 <= wave_last;
    floatx16 s[2];
    if (active) {
      // ---- scores of tile i: every K fragment feeds both query blocks
      const unsigned char* kp = smem + PP_LDS_K + (i & (PP_STAGES - 1)) * PP_KTILE;
      // with one wavefront per SIMD nothing but this wavefront's own earlier requests hides the LDS latency: the
      // fragments of a pair of steps are requested while the pair before it multiplies (four matrix instructions)
      typename mma<T>::frag kf[4];
#pragma unroll
      for (int j = 0; j < 2; ++j) kf[j] = mma<T>::load(reinterpret_cast<const T*>(kp + kxo(j)));
      // Two k-steps at a time, both into s[0], then both into s[1]: a matrix instruction whose accumulator is the
      // result of the one right before it starts without delay (the result is forwarded), while one that accumulates
      // onto the result of the instruction before last waits for the write-back - alternating s[0], s[1] per k-step
      // ran at 50 cycles per instruction instead of 32.
#pragma unroll
      for (int ks = 0; ks < KS; ks += 2) {
#pragma unroll
        for (int d = 2; d < 4; ++d)
          if (ks + d < KS)
            kf[(ks + d) & 3] = mma<T>::load(reinterpret_cast<const T*>(kp + kxo((ks + d) & 7) + ((ks + d) >> 3) * 256));
        // the eight global -> LDS requests of this iteration, one per pair of steps, under the matrix instructions
        if (ks < 8) issue_k1(i + 3, tk3, ks / 2);
        else issue_v1(i + 2, tv2, ks / 2 - 4);
        __builtin_amdgcn_sched_barrier(0);
        if (ks == 0) mma<T>::first_v(s[0], kf[0], qf[0][0]);
        else mma<T>::run_v(s[0], kf[ks & 3], qf[0][ks]);
        mma<T>::run_v(s[0], kf[(ks + 1) & 3], qf[0][ks + 1]);
        if (ks == 0) mma<T>::first_v(s[1], kf[0], qf[1][0]);
        else mma<T>::run_v(s[1], kf[ks & 3], qf[1][ks]);
        mma<T>::run_v(s[1], kf[(ks + 1) & 3], qf[1][ks + 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
      asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");   // wait states between the last score MFMA and the first read of s
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        // register v is key key0 + 16*(v/8) + 8*fg + v%8
        if (key0 + BKV - 1 > wave_first[qb]) {    // the diagonal crosses the tile: hide what a query may not see
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = key0 + 16 * (v / 8) + 8 * fg + (v % 8);
            s[qb][v] = (key <= qsee[qb]) ? s[qb][v] : -INFINITY;
          }
        }
      }
    }
    if (!active) {
      issue_k(i + 3, tk3);
      issue_v(i + 2, tv2);
    }
    if (prev_active) {
      // the last tile of a sequence can be partial: what V^T holds beyond the last key must not reach the product
      // (0 x garbage may be NaN).  Every wavefront clears all of it before its own reads (LDS operations of one
      // wavefront stay in order), so no barrier is needed.
      const int tv = i - 1;
      const int nbad = tv * BKV + BKV - 1 - klast;
      if (nbad > 0) {
        uint16_t* vs = reinterpret_cast<uint16_t*>(smem + PP_LDS_V + (tv & (PP_STAGES - 1)) * PP_VTILE);
        for (int c = lane; c < DH * nbad; c += 64) {
          const int row = c / nbad, col = BKV - nbad + (c % nbad);
          vs[row * 32 + (((col >> 3) ^ ((row >> 2) & 3)) * 8) + (col & 7)] = (uint16_t)0;
        }
      }
    }
    // ---- V^T P^T of tile i-1 on the matrix pipe with the exponentials of tile i on the vector unit between its
    // instructions.  The exponentials are taken against the running maximum of the EARLIER tiles, so that nothing in
    // this region waits for the maximum of tile i; that maximum is worked out alongside, and only if it lies more than
    // 2^6 above the running one (probabilities would pass 64; after the first tiles it never does) the tile is redone
    // below against the new maximum and the accumulator rescaled.
    typename mma<T>::frag pn[2][2];
    float mt[2] = {-INFINITY, -INFINITY}, lt[2] = {0.f, 0.f};
    const float mneg[2] = {mrun[0] == -INFINITY ? 0.f : -mrun[0], mrun[1] == -INFINITY ? 0.f : -mrun[1]};
    const unsigned char* vp = vbase + ((i - 1) & (PP_STAGES - 1)) * PP_VTILE;
    float pe[2];                                  // the even-numbered probability of the pair being packed
    auto exp_step = [&](auto K_) {                // step K of 32: probability K % 16 of query block K / 16
      constexpr int k = decltype(K_)::value, qb = k / 16, v = k % 16;
      const float p = __builtin_amdgcn_exp2f(fmaf(s[qb][v], sc2, mneg[qb]));   // masked -> exp2(-inf) = 0
      if constexpr (v % 2 == 0) {
        pe[qb] = p;
      } else {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        u32x4 w = __builtin_bit_cast(u32x4, pn[qb][v / 8].v);
        w[(v % 8) / 2] = pack_prob<T>(pe[qb], p);
        pn[qb][v / 8].v = __builtin_bit_cast(decltype(pn[qb][v / 8].v), w);
      }
      if constexpr (v % 4 == 3) mt[qb] = max3(max3(mt[qb], s[qb][v - 3], s[qb][v - 2]), s[qb][v - 1], s[qb][v]);
      if constexpr (v % 8 == 7) lt[qb] = psum<T>::run(pn[qb][v / 8], lt[qb]);
    };
    __builtin_amdgcn_sched_barrier(0);
    if (prev_active && active) {
      typename mma<T>::frag vf[4];             // the V^T fragment of step j + 3 is requested while step j multiplies
#pragma unroll
      for (int j = 0; j < 3; ++j) vf[j] = mma<T>::load(reinterpret_cast<const T*>(vp + j * 2048 + vpos[0]));
      static_for<16>([&](auto J_) {
        constexpr int j = decltype(J_)::value, kh = j / 8, n = j % 8;
        if constexpr (j + 3 < 16)
          vf[(j + 3) & 3] = mma<T>::load(reinterpret_cast<const T*>(vp + ((j + 3) % 8) * 2048 + vpos[(j + 3) / 8]));
        __builtin_amdgcn_sched_barrier(0);
        mma<T>::template run_fixed<n * 16>(vf[j & 3], pf[0][kh]);
        exp_step(std::integral_constant<int, 2 * j>{});
        __builtin_amdgcn_sched_barrier(0);
        mma<T>::template run_fixed<(8 + n) * 16>(vf[j & 3], pf[1][kh]);
        exp_step(std::integral_constant<int, 2 * j + 1>{});
        __builtin_amdgcn_sched_barrier(0);
      });
    } else if (prev_active) {
      typename mma<T>::frag vf[4];
#pragma unroll
      for (int j = 0; j < 3; ++j) vf[j] = mma<T>::load(reinterpret_cast<const T*>(vp + j * 2048 + vpos[0]));
      static_for<16>([&](auto J_) {
        constexpr int j = decltype(J_)::value, kh = j / 8, n = j % 8;
        if constexpr (j + 3 < 16)
          vf[(j + 3) & 3] = mma<T>::load(reinterpret_cast<const T*>(vp + ((j + 3) % 8) * 2048 + vpos[(j + 3) / 8]));
        __builtin_amdgcn_sched_barrier(0);
        mma<T>::template run_fixed<n * 16>(vf[j & 3], pf[0][kh]);
        mma<T>::template run_fixed<(8 + n) * 16>(vf[j & 3], pf[1][kh]);
        __builtin_amdgcn_sched_barrier(0);
      });
    } else if (active) {
      static_for<32>(exp_step);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (active) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const float mtile = max_halves(mt[qb] * sc2);            // sc2 > 0
        if (__any(mtile > mrun[qb] + 6.0f)) {
          // rare: redo the tile against the new maximum and bring the accumulator (tiles 0 .. i-1) to it
          const float mnew = fmaxf(mrun[qb], mtile);
          const float alpha = (mnew == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(mrun[qb] - mnew);   // mrun = -inf -> 0
          const float mn = (mnew == -INFINITY) ? 0.f : -mnew;
          mrun[qb] = mnew;
          float p[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) p[v] = __builtin_amdgcn_exp2f(fmaf(s[qb][v], sc2, mn));
          pn[qb][0] = mma<T>::from_floats(p);
          pn[qb][1] = mma<T>::from_floats(p + 8);
          lt[qb] = psum<T>::run(pn[qb][1], psum<T>::run(pn[qb][0], 0.f));
          lrun[qb] *= alpha;
          asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");     // the last MFMA into the accumulator may still be in flight
          if (qb == 0) static_for<NBLK>([&](auto N_) { acc_scale16<decltype(N_)::value * 16>(alpha); });
          else static_for<NBLK>([&](auto N_) { acc_scale16<(8 + decltype(N_)::value) * 16>(alpha); });
        }
        lrun[qb] += sum_halves(lt[qb]);
        pf[qb][0] = pn[qb][0];
        pf[qb][1] = pn[qb][1];
      }
    }
    prev_active = active;
  }
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");           // the last MFMAs into the accumulator drain
  // ---- write O.  Register v of block n is head-dim n*32 + 8*(v/4) + 4*fg + v%4 of the lane's query: stored from
  // there, a store instruction would put 16 bytes into each of 32 rows.  The tiles are done with, so every wavefront
  // turns its 64 rows round in its own 32 KiB of LDS (16-byte chunks xor-swizzled with the row) and writes whole rows.
  __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));                // my surplus loads have landed ...
  __builtin_amdgcn_s_barrier();                             // ... and so have everybody's; nobody reads a tile any more
  unsigned char* ob = smem + wave * 32768;
  static_for<2>([&](auto QB_) {
    constexpr int qb = decltype(QB_)::value;
    const int t = qt0 + wave * 64 + qb * 32 + fr;
    const float inv = (t < Tp && t + p0 >= 0 && lrun[qb] > 0.f) ? 1.0f / lrun[qb] : 0.f;
    static_for<NBLK * 4>([&](auto I_) {
      constexpr int c = decltype(I_)::value, r = (qb * 8 + c / 4) * 16 + (c % 4) * 4;   // c: 16-byte chunk n*4 + v4 of the row
      uint32x2 pk;
      pk.x = pack2<T>(acc_read<r>() * inv, acc_read<r + 1>() * inv);
      pk.y = pack2<T>(acc_read<r + 2>() * inv, acc_read<r + 3>() * inv);
      *reinterpret_cast<uint32x2*>(ob + (qb * 32 + fr) * 512 + ((c ^ fr) << 4) + fg * 8) = pk;
    });
  });
  // (a wavefront's LDS operations stay in order: no barrier between its own writes and reads)
#pragma unroll 4
  for (int it = 0; it < 32; ++it) {
    const int row = 2 * it + fg, t = qt0 + wave * 64 + row;
    const uint32x4 v = *reinterpret_cast<const uint32x4*>(ob + row * 512 + ((fr ^ (row & 31)) << 4));
    if (t < Tp) *reinterpret_cast<uint32x4*>(out + ((int64_t)b * Tp + t) * ld_out + (int64_t)h * DH + fr * 8) = v;
  }
  __builtin_amdgcn_s_barrier();                             // the next part's tiles go where these rows were
  }
}

// ------------------------------------------------------------------------------------------------
// Decode.  Grid (S, H, B): the valid part of a (sequence, head) window is cut into S equal key ranges (the cut
// follows the position read from device memory, so every workgroup has work whatever the fill), and each
// 4-wavefront workgroup reduces its range to a partial (max, sum, weighted V).  A wavefront owns every fourth
// group of KPL keys and keeps its own online-softmax state in registers: LPK lanes cover one key row with 16-byte
// loads, the score of a key is reduced over those lanes by shuffles, and the probability-weighted V rows are
// accumulated per lane, so nothing crosses wavefronts until the end of the range.  All K and V rows of one
// 64-key step are requested before the first is used and the next step's rows before the current step is
// reduced; rows beyond the range are clamped to its last key and masked, so no load is conditional.
//
// Partials: work[((b*H + h)*S + s) * (DH + 4)] = {max, sum, -, -, V[DH]}.  With S == 1 and `out` given the normalised
// result goes straight to `out`; otherwise attn_combine_kernel (or the prologue of the out-projection GEMV) merges them.
constexpr int DEC_NI = 8;            // K (and V) loads per lane and step
constexpr int DEC_PAD = MTJ_DEC_PAD;  // floats in front of the vector of a partial

template <typename T, int DH>
__global__ __launch_bounds__(256) void attn_decode_kernel(const float* __restrict__ q, const T* __restrict__ kc,
                                                          const T* __restrict__ vc, const int32_t* __restrict__ pos,
                                                          int H, int Tcap, float* __restrict__ work, void* __restrict__ out,
                                                          int64_t ld_out, int out_dtype) {
  constexpr int EPC = kvrow<T>::EPC;
  constexpr int LPK = DH / EPC;      // lanes per key row
  constexpr int KPL = 64 / LPK;      // keys per wavefront load
  constexpr int NI = DEC_NI;
  constexpr int STEP = 4 * NI * KPL; // keys per workgroup step
  static_assert(LPK <= 64 && 64 % LPK == 0, "head dim does not map onto a wavefront");
  __shared__ float part[4][DH];
  __shared__ float stat[4][2];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z, S = gridDim.x;
  const int64_t bh = (int64_t)b * H + h;
  const int p = pos[b];
  const int nvalid = (p + 1 < Tcap) ? p + 1 : Tcap;
  const int per = (nvalid + S - 1) / S;                       // keys per range
  const int k0 = split * per;
  const int nk = (k0 + per <= nvalid) ? per : nvalid - k0;     // <= 0: an empty range (fewer keys than ranges)
  const int sub = lane / LPK, el = (lane % LPK) * EPC;

  float m_run = -INFINITY, l_run = 0.f;                        // l_run and acc are per lane (their key subgroup)
  float acc[EPC];
#pragma unroll
  for (int j = 0; j < EPC; ++j) acc[j] = 0.f;

  if (nk > 0) {
    const T* kbase = kc + (bh * Tcap + k0) * DH + el;
    const T* vbase = vc + (bh * Tcap + k0) * DH + el;
    uint32x4 kr[2][NI], vr[2][NI];
    auto request = [&](int buf, int base) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        int kk = base + (i * 4 + wave) * KPL + sub;
        kk = kk < nk ? kk : nk - 1;
        // streaming loads: the window is read once per step and never again, and kept in the caches it only displaces
        // itself (32 sequences x 2004 keys: 155.6 us against 177.6 with ordinary loads)
        kr[buf][i] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(kbase + (int64_t)kk * DH));
        vr[buf][i] = __builtin_nontemporal_load(reinterpret_cast<const uint32x4*>(vbase + (int64_t)kk * DH));
      }
    };
    float qv[EPC];
    request(0, 0);
#pragma unroll
    for (int j = 0; j < EPC; ++j) qv[j] = q[bh * DH + el + j];
    const float scale = rsqrtf((float)DH);
    auto reduce = [&](int buf, int base) {
      float sc[NI];
      float mt = -INFINITY;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        float kf[EPC];
        kvrow<T>::get(kr[buf][i], kf);
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < EPC; ++j) d = fmaf(kf[j], qv[j], d);
#pragma unroll
        for (int o = LPK / 2; o > 0; o >>= 1) d += __shfl_xor(d, o);
        const int kk = base + (i * 4 + wave) * KPL + sub;
        sc[i] = kk < nk ? d * scale : -INFINITY;
        mt = fmaxf(mt, sc[i]);
      }
#pragma unroll
      for (int o = 32; o >= LPK; o >>= 1) mt = fmaxf(mt, __shfl_xor(mt, o));
      const float m_new = fmaxf(m_run, mt);                    // finite: the first key group of a wavefront's step 0 ...
      if (m_new == -INFINITY) return;                          // ... unless this wavefront has no key in this step
      const float alpha = __expf(m_run - m_new);               // m_run = -inf -> 0
      l_run *= alpha;
#pragma unroll
      for (int j = 0; j < EPC; ++j) acc[j] *= alpha;
      m_run = m_new;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const float pr = __expf(sc[i] - m_new);                // masked -> 0
        l_run += pr;
        float vf[EPC];
        kvrow<T>::get(vr[buf][i], vf);
#pragma unroll
        for (int j = 0; j < EPC; ++j) acc[j] = fmaf(pr, vf[j], acc[j]);
      }
    };
    int base = 0;
    for (; base + 2 * STEP < nk + STEP; base += 2 * STEP) {    // steps base and base + STEP both exist
      request(1, base + STEP);
      reduce(0, base);
      if (base + 2 * STEP < nk) request(0, base + 2 * STEP);
      reduce(1, base + STEP);
    }
    if (base < nk) reduce(0, base);
  }
  // ---- key subgroups of a wavefront, then the four wavefronts
#pragma unroll
  for (int o = 32; o >= LPK; o >>= 1) {
    l_run += __shfl_xor(l_run, o);
#pragma unroll
    for (int j = 0; j < EPC; ++j) acc[j] += __shfl_xor(acc[j], o);
  }
  if (lane < LPK) {
#pragma unroll
    for (int j = 0; j < EPC; ++j) part[wave][el + j] = acc[j];
  }
  if (lane == 0) { stat[wave][0] = m_run; stat[wave][1] = l_run; }
  __syncthreads();
  const float m0 = stat[0][0], m1 = stat[1][0], m2 = stat[2][0], m3 = stat[3][0];
  const float mm = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));
  const bool any = mm != -INFINITY;
  const float f0 = any ? __expf(m0 - mm) : 0.f, f1 = any ? __expf(m1 - mm) : 0.f;
  const float f2 = any ? __expf(m2 - mm) : 0.f, f3 = any ? __expf(m3 - mm) : 0.f;
  const float lt = (f0 * stat[0][1] + f1 * stat[1][1]) + (f2 * stat[2][1] + f3 * stat[3][1]);
  float* wout = work + (bh * S + split) * (DH + DEC_PAD);
  for (int e = tid; e < DH; e += 256) {
    const float v = (f0 * part[0][e] + f1 * part[1][e]) + (f2 * part[2][e] + f3 * part[3][e]);
    if (S == 1 && out) store_as(out, (int64_t)b * ld_out + h * DH + e, lt > 0.f ? v / lt : 0.f, out_dtype);
    else wout[DEC_PAD + e] = v;
  }
  if (!(S == 1 && out) && tid == 0) { wout[0] = mm; wout[1] = lt; }
}

// Merge of the S partials of one (sequence, head), four elements per thread (the out-projection GEMV does the same
// while it stages its input).
template <int DH>
__global__ __launch_bounds__(DH / 4) void attn_combine_kernel(const float* __restrict__ work, int S, int H,
                                                              void* __restrict__ out, int64_t ld_out, int out_dtype) {
  const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int64_t bh = (int64_t)b * H + h;
  const floatx4 a = mtj_merge_partials(work + bh * S * (DH + DEC_PAD), S, DH + DEC_PAD, 4 * tid);
  const int64_t o = (int64_t)b * ld_out + h * DH + 4 * tid;
  store_as(out, o, a.x, out_dtype);
  store_as(out, o + 1, a.y, out_dtype);
  store_as(out, o + 2, a.z, out_dtype);
  store_as(out, o + 3, a.w, out_dtype);
}

// key ranges per (sequence, head): about one workgroup per CU when the batch alone does not fill the chip; a range
// never starts out shorter than 16 keys at the full window
int decode_splits(int64_t B, int64_t H, int64_t Tcap) {
  int64_t S = 256 / (B * H);
  if (S > (Tcap + 15) / 16) S = (Tcap + 15) / 16;
  if (S > MTJ_DEC_MAXS) S = MTJ_DEC_MAXS;
  if (S < 1) S = 1;
  return (int)S;
}

}  // namespace

extern "C" int mtj_attn_prefill(const void* q, const void* k_cache, const void* v_t, const int32_t* pos0, int64_t B,
                                int64_t H, int64_t Tp, int64_t Tcap, int64_t dh, int64_t ldvt, void* out,
                                int64_t ld_out, int dtype, const int32_t* key_limit, void* stream) {
  MTJ_REQUIRE(q && k_cache && v_t && pos0 && out, MTJ_EINVAL, "mtj_attn_prefill: null pointer");
  MTJ_REQUIRE(B > 0 && H > 0 && Tp > 0 && Tp <= Tcap && ld_out >= H * dh && B < 65536 && H < 65536, MTJ_EINVAL,
              "mtj_attn_prefill: bad shape B=%lld H=%lld Tp=%lld Tcap=%lld", (long long)B, (long long)H,
              (long long)Tp, (long long)Tcap);
  MTJ_REQUIRE(mtj_is_dtype(dtype), MTJ_EDTYPE, "mtj_attn_prefill: dtype %d", dtype);
  const int esz = mtj_elem_size(dtype);
  MTJ_REQUIRE(ldvt >= (Tp + 63) / 64 * 64 && (ldvt * esz) % 16 == 0 && (ld_out * esz) % 16 == 0, MTJ_EALIGN,
              "mtj_attn_prefill: ldvt must be >= Tp rounded up to a multiple of 64, rows 16-byte aligned");
  MTJ_REQUIRE(mtj_aligned16(q) && mtj_aligned16(k_cache) && mtj_aligned16(v_t) && mtj_aligned16(out), MTJ_EALIGN,
              "mtj_attn_prefill: pointers must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
#define MTJ_PREFILL(T, DH, NW, BKV)                                                                                  \
  do {                                                                                                               \
    constexpr size_t lds = 2 * ((size_t)BKV * (DH + mma<T>::EPC) + (size_t)DH * (BKV + mma<T>::EPC)) * sizeof(T);    \
    static_assert(lds <= 160 * 1024, "attention tiles do not fit LDS");                                              \
    static mtj_device_once once;                                                                                     \
    if (int rc = mtj_allow_lds(once, "mtj_attn_prefill", &attn_prefill_kernel<T, DH, NW, BKV>, lds)) return rc;      \
    const int64_t nqblk = (Tp + NW * 32 - 1) / (NW * 32);                                                            \
    MTJ_REQUIRE(nqblk * H * B < (1ll << 31), MTJ_ELIMIT, "mtj_attn_prefill: too many workgroups");                    \
    attn_prefill_kernel<T, DH, NW, BKV><<<(unsigned)(nqblk * H * B), NW * 64, lds, s>>>(                              \
        (const T*)q, (const T*)k_cache, (const T*)v_t, pos0, (int)H, (int)Tp, (int)Tcap, ldvt, (T*)out, ld_out,      \
        (int)B, (int)nqblk, key_limit);                                                                                       \
  } while (0)
#define MTJ_PREFILL_PAIR(T)                                                                                          \
  do {                                                                                                               \
    static_assert(PP_LDS_BYTES <= 160 * 1024, "attention tiles do not fit LDS");                                     \
    static mtj_device_once once;                                                                                     \
    if (int rc = mtj_allow_lds(once, "mtj_attn_prefill", &attn_prefill_pair_kernel<T>, PP_LDS_BYTES)) return rc;     \
    const int64_t nqblk = (Tp + 127) / 128;                                                                          \
    MTJ_REQUIRE(nqblk * H * B < (1ll << 31), MTJ_ELIMIT, "mtj_attn_prefill: too many workgroups");                    \
    MTJ_REQUIRE(Tcap * 512 < (1ll << 31) && 512 * ldvt < (1ll << 31), MTJ_ELIMIT, "mtj_attn_prefill: window too long"); \
    attn_prefill_pair_kernel<T><<<(unsigned)(nqblk * H * B), 512, PP_LDS_BYTES, s>>>(                                 \
        (const T*)q, (const T*)k_cache, (const T*)v_t, pos0, (int)H, (int)Tp, (int)Tcap, ldvt, (T*)out, ld_out,      \
        (int)B, (int)nqblk, key_limit);                                                                              \
  } while (0)
#define MTJ_PREFILL_Q64(T)                                                                                           \
  do {                                                                                                               \
    static_assert(Q64_LDS_BYTES <= 160 * 1024, "attention tiles do not fit LDS");                                    \
    static mtj_device_once once;                                                                                     \
    if (int rc = mtj_allow_lds(once, "mtj_attn_prefill", &attn_prefill_q64_kernel<T>, Q64_LDS_BYTES)) return rc;     \
    const int64_t nqblk = (Tp + 255) / 256;                                                                          \
    MTJ_REQUIRE(nqblk * H * B < (1ll << 31), MTJ_ELIMIT, "mtj_attn_prefill: too many workgroups");                    \
    MTJ_REQUIRE(Tcap * 512 < (1ll << 31) && 512 * ldvt < (1ll << 31), MTJ_ELIMIT, "mtj_attn_prefill: window too long"); \
    attn_prefill_q64_kernel<T><<<(unsigned)((nqblk + 1) / 2 * H * B), 256, Q64_LDS_BYTES, s>>>(                                 \
        (const T*)q, (const T*)k_cache, (const T*)v_t, pos0, (int)H, (int)Tp, (int)Tcap, ldvt, (T*)out, ld_out,      \
        (int)B, (int)nqblk, key_limit);                                                                              \
  } while (0)
  // 256-query blocks, two per workgroup, when that still makes two workgroups per CU (measured on 16 heads x 2048 tokens:
  // 472 us against 529 for 8 sequences, 796 against 1069 for 16, but 225 against 208 for 4); shorter problems keep the
  // 128-query workgroups
  const bool q64 = dh == 256 && B * H * ((Tp + 255) / 256) >= 1024;
  if (dtype == MTJ_BF16 && q64) MTJ_PREFILL_Q64(bf16_t);
  else if (dtype == MTJ_F16 && q64) MTJ_PREFILL_Q64(f16_t);
  else if (dtype == MTJ_BF16 && dh == 256) MTJ_PREFILL_PAIR(bf16_t);
  else if (dtype == MTJ_BF16 && dh == 64) MTJ_PREFILL(bf16_t, 64, 8, 64);
  else if (dtype == MTJ_F16 && dh == 256) MTJ_PREFILL_PAIR(f16_t);
  else if (dtype == MTJ_F16 && dh == 64) MTJ_PREFILL(f16_t, 64, 8, 64);
  else if (dtype == MTJ_F32 && dh == 256) MTJ_PREFILL(float, 256, 4, 32);
  else if (dtype == MTJ_F32 && dh == 64) MTJ_PREFILL(float, 64, 4, 32);
  else return mtj_fail(MTJ_EINVAL, "mtj_attn_prefill: unsupported dtype %d / d_head %lld (64 or 256)", dtype, (long long)dh);
#undef MTJ_PREFILL
#undef MTJ_PREFILL_PAIR
#undef MTJ_PREFILL_Q64
  return mtj_check_launch("mtj_attn_prefill");
}

extern "C" int mtj_attn_decode_splits(int64_t B, int64_t H, int64_t Tcap) {
  if (B <= 0 || H <= 0 || Tcap <= 0) return 0;
  return decode_splits(B, H, Tcap);
}

extern "C" int64_t mtj_attn_decode_work_bytes(int64_t B, int64_t H, int64_t dh, int64_t Tcap) {
  if (B <= 0 || H <= 0 || Tcap <= 0 || dh <= 0) return 0;
  return B * H * (int64_t)decode_splits(B, H, Tcap) * (dh + DEC_PAD) * (int64_t)sizeof(float);
}

namespace {

// merge = false: only the partials are produced (the caller merges them, see mtj_attn_merge), out may be NULL
int attn_decode_impl(const char* who, const float* q, const void* k_cache, const void* v_cache, const int32_t* pos,
                     int64_t B, int64_t H, int64_t Tcap, int64_t dh, void* out, int64_t ld_out, int out_dtype, int dtype,
                     void* work, bool merge, void* stream) {
  MTJ_REQUIRE(q && k_cache && v_cache && pos && work && (out || !merge), MTJ_EINVAL, "%s: null pointer", who);
  MTJ_REQUIRE(B > 0 && H > 0 && Tcap > 0 && B < 65536 && H < 65536 && Tcap < (1ll << 30), MTJ_EINVAL, "%s: bad shape", who);
  MTJ_REQUIRE(mtj_aligned16(q) && mtj_aligned16(k_cache) && mtj_aligned16(v_cache) && mtj_aligned16(work), MTJ_EALIGN,
              "%s: pointers must be 16-byte aligned", who);
  if (merge) {
    MTJ_REQUIRE(ld_out >= H * dh, MTJ_EINVAL, "%s: ld_out < H * dh", who);
    MTJ_REQUIRE(mtj_is_dtype(out_dtype), MTJ_EDTYPE, "%s: out_dtype %d", who, out_dtype);
  }
  const int S = decode_splits(B, H, Tcap);
  float* partials = reinterpret_cast<float*>(work);
  dim3 grid((unsigned)S, (unsigned)H, (unsigned)B);
  hipStream_t s = (hipStream_t)stream;
#define MTJ_DECODE(T, DH)                                                                                         \
  do {                                                                                                            \
    attn_decode_kernel<T, DH><<<grid, 256, 0, s>>>(q, (const T*)k_cache, (const T*)v_cache, pos, (int)H, (int)Tcap, \
                                                   partials, out, ld_out, out_dtype);                             \
    if (merge && S > 1)                                                                                           \
      attn_combine_kernel<DH><<<dim3((unsigned)H, (unsigned)B), DH / 4, 0, s>>>(partials, S, (int)H, out, ld_out,  \
                                                                                 out_dtype);                      \
  } while (0)
  if (dtype == MTJ_BF16 && dh == 256) MTJ_DECODE(bf16_t, 256);
  else if (dtype == MTJ_BF16 && dh == 64) MTJ_DECODE(bf16_t, 64);
  else if (dtype == MTJ_F16 && dh == 256) MTJ_DECODE(f16_t, 256);
  else if (dtype == MTJ_F16 && dh == 64) MTJ_DECODE(f16_t, 64);
  else if (dtype == MTJ_F32 && dh == 256) MTJ_DECODE(float, 256);
  else if (dtype == MTJ_F32 && dh == 64) MTJ_DECODE(float, 64);
  else return mtj_fail(MTJ_EINVAL, "%s: unsupported dtype %d / d_head %lld (64 or 256)", who, dtype, (long long)dh);
#undef MTJ_DECODE
  return mtj_check_launch(who);
}

}  // namespace

extern "C" int mtj_attn_decode(const float* q, const void* k_cache, const void* v_cache, const int32_t* pos, int64_t B,
                               int64_t H, int64_t Tcap, int64_t dh, void* out, int64_t ld_out, int out_dtype, int dtype,
                               void* work, void* stream) {
  return attn_decode_impl("mtj_attn_decode", q, k_cache, v_cache, pos, B, H, Tcap, dh, out, ld_out, out_dtype, dtype, work,
                          true, stream);
}

extern "C" int mtj_attn_decode_partials(const float* q, const void* k_cache, const void* v_cache, const int32_t* pos,
                                        int64_t B, int64_t H, int64_t Tcap, int64_t dh, int dtype, void* work,
                                        mtj_attn_merge* merge, void* stream) {
  MTJ_REQUIRE(merge, MTJ_EINVAL, "mtj_attn_decode_partials: null pointer");
  const int rc = attn_decode_impl("mtj_attn_decode_partials", q, k_cache, v_cache, pos, B, H, Tcap, dh, nullptr, 0, MTJ_F32,
                                  dtype, work, false, stream);
  if (rc) return rc;
  const int S = decode_splits(B, H, Tcap);
  merge->partials = reinterpret_cast<const float*>(work);
  merge->n_heads = (int32_t)H;
  merge->d_head = (int32_t)dh;
  merge->splits = S;
  return MTJ_OK;
}

// ------------------------------------------------------------------------------------------------
// The same launches with the partial results kept in a device array that lives in the code object, for
// callers that cannot allocate (or pass) a workspace.  Every device that loads the library holds its own copy of
// `scratch` at its own address: the address is looked up once per device (hipGetSymbolAddress with that device
// current) and that pointer, never the array's name, is what host code hands to the kernels.  Nothing in
// `scratch` has to start at zero: the merge kernel reads only the partials that the first kernel of the same
// call has written.  All calls on one device share the array, so calls that overlap on one device race.
static __device__ __align__(256) unsigned char scratch[MTJ_ATTN_DECODE_STATIC_BYTES];

namespace {
mtj_device_once scratch_once;
void* scratch_ptr[MTJ_MAX_DEVICES];

int scratch_address(void** p) {
  int dev = 0;
  const int rc = mtj_once_per_device(scratch_once, "mtj_attn_decode_static", [&](int d) {
    void* sym = nullptr;
    const hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !sym)
      return mtj_fail(MTJ_EHIP, "mtj_attn_decode_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    scratch_ptr[d] = sym;
    return (int)MTJ_OK;
  });
  if (rc) return rc;
  const hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return mtj_fail(MTJ_EHIP, "mtj_attn_decode_static: hipGetDevice: %s", hipGetErrorString(e));
  *p = scratch_ptr[dev];
  return MTJ_OK;
}
}  // namespace

// Also the set-up call: it looks the array's address up on the current device (a symbol lookup may load the code object
// and must not happen inside a stream capture), so that mtj_attn_decode_static itself only launches.
extern "C" int64_t mtj_attn_decode_static_max_bytes(void) {
  void* p = nullptr;
  (void)scratch_address(&p);          // without a usable device the size is still the answer; the entry point reports it
  return MTJ_ATTN_DECODE_STATIC_BYTES;
}

extern "C" int mtj_attn_decode_static(const float* q, const void* k_cache, const void* v_cache, const int32_t* pos,
                                      int64_t B, int64_t H, int64_t Tcap, int64_t dh, void* out, int64_t ld_out,
                                      int out_dtype, int dtype, void* stream) {
  MTJ_REQUIRE(B > 0 && H > 0 && Tcap > 0 && dh > 0, MTJ_EINVAL, "mtj_attn_decode_static: bad shape");
  const int64_t need = mtj_attn_decode_work_bytes(B, H, dh, Tcap);
  MTJ_REQUIRE(need <= MTJ_ATTN_DECODE_STATIC_BYTES, MTJ_ELIMIT,
              "mtj_attn_decode_static: B=%lld H=%lld Tcap=%lld dh=%lld needs %lld bytes of partial results, the built-in "
              "array holds %lld; use mtj_attn_decode with a caller-provided workspace",
              (long long)B, (long long)H, (long long)Tcap, (long long)dh, (long long)need,
              (long long)MTJ_ATTN_DECODE_STATIC_BYTES);
  void* work = nullptr;
  if (int rc = scratch_address(&work)) return rc;
  return attn_decode_impl("mtj_attn_decode_static", q, k_cache, v_cache, pos, B, H, Tcap, dh, out, ld_out, out_dtype,
                          dtype, work, true, stream);
}

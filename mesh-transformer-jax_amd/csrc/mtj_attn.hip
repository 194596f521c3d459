// Attention: MFMA flash-style prefill over a left-padded rectangle, and one-token decode over the K/V window.
#include "mtj_common.h"

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
  auto load_tile = [&](int kt) {
    const int key0 = kt * BKV;
#pragma unroll
    for (int i = 0; i < K_CHUNKS; ++i) {
      const int c = i * NT + tid, row = c / CPRK, cc = c % CPRK;
      const int key = (key0 + row <= klast) ? key0 + row : klast;
      rk[i] = *reinterpret_cast<const uint32x4*>(kc + (bh * Tcap + key) * DH + cc * EPC);
    }
#pragma unroll
    for (int i = 0; i < V_CHUNKS; ++i) {
      const int c = i * NT + tid, row = c / CPRV, cc = c % CPRV;
      rv[i] = *reinterpret_cast<const uint32x4*>(vt + (bh * DH + row) * ldvt + key0 + cc * EPC);
    }
  };
  auto fix_last_tile = [&](int kt, int buf) {     // workgroup-uniform caller; runs between the store and the barrier
    const int key0 = kt * BKV;
    const int nbad = key0 + BKV - 1 - klast;       // columns klast+1-key0 .. BKV-1 of V^T do not exist
    if (nbad <= 0) return;
    raw_t* vs = reinterpret_cast<raw_t*>(Vs + buf * DH * VROW);
    for (int c = tid; c < DH * nbad; c += NT) vs[(c / nbad) * VROW + (BKV - nbad) + (c % nbad)] = (raw_t)0;
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < K_CHUNKS; ++i) {
      const int c = i * NT + tid, row = c / CPRK, cc = c % CPRK;
      *reinterpret_cast<uint32x4*>(Ks + (buf * BKV + row) * KROW + cc * EPC) = rk[i];
    }
#pragma unroll
    for (int i = 0; i < V_CHUNKS; ++i) {
      const int c = i * NT + tid, row = c / CPRV, cc = c % CPRV;
      *reinterpret_cast<uint32x4*>(Vs + (buf * DH + row) * VROW + cc * EPC) = rv[i];
    }
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
#pragma unroll
        for (int i = 0; i < NBLK; ++i)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[i][v] *= alpha;
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
        if (sizeof(T) == 2) {
          uint32x2 pk;
          pk.x = pack_bf16x2(o[i][v4 * 4] * inv, o[i][v4 * 4 + 1] * inv);
          pk.y = pack_bf16x2(o[i][v4 * 4 + 2] * inv, o[i][v4 * 4 + 3] * inv);
          *reinterpret_cast<uint32x2*>(op + e) = pk;
        } else {
          *reinterpret_cast<floatx4*>(op + e) =
              floatx4{o[i][v4 * 4] * inv, o[i][v4 * 4 + 1] * inv, o[i][v4 * 4 + 2] * inv, o[i][v4 * 4 + 3] * inv};
        }
      }
  }
}

// ------------------------------------------------------------------------------------------------
// Decode.  Grid (splits, H, B); each workgroup reduces 64 window slots to a partial (max, sum, weighted V)
// and attn_combine_kernel merges the non-empty partials of a (sequence, head).  (Merging in the same launch,
// by the last workgroup to arrive, needs a device-scope fence per workgroup; on this multi-die GPU that
// fence writes back the L2 and made the kernel 6x slower than the two launches.)  16-byte loads: LPK lanes
// cover one key row; all K and V loads of a workgroup are requested up front (V does not depend on the
// scores).
constexpr int DEC_CHUNK = 64;

template <typename T, int DH>
__global__ __launch_bounds__(256) void attn_decode_kernel(const float* __restrict__ q, const T* __restrict__ kc,
                                                          const T* __restrict__ vc, const int32_t* __restrict__ pos,
                                                          int H, int Tcap, float* __restrict__ work) {
  constexpr int EPC = 16 / sizeof(T);
  constexpr int LPK = DH / EPC;      // lanes per key row
  constexpr int KPL = 64 / LPK;      // keys per wavefront load
  constexpr int NI = DEC_CHUNK / (4 * KPL);   // loads per lane for K (and for V)
  static_assert(LPK <= 64 && 64 % LPK == 0 && NI >= 1, "head dim does not map onto a wavefront");
  __shared__ float sc[DEC_CHUNK];
  __shared__ float part[4][DH];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z, S = gridDim.x;
  const int64_t bh = (int64_t)b * H + h;
  const int nvalid = (pos[b] + 1 < Tcap) ? pos[b] + 1 : Tcap;
  const int k0 = split * DEC_CHUNK;
  const int nk = (k0 + DEC_CHUNK < nvalid) ? DEC_CHUNK : nvalid - k0;     // <= 0: nothing in this range
  float* wout = work + (bh * S + split) * (DH + 2);
  const int sub = lane / LPK, el = (lane % LPK) * EPC;

  if (nk > 0) {
    // ---- request every K and V row of the range
    uint32x4 kr[NI], vr[NI];
    const T* kbase = kc + (bh * Tcap + k0) * DH + el;
    const T* vbase = vc + (bh * Tcap + k0) * DH + el;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int kk = (i * 4 + wave) * KPL + sub;
      if (kk < nk) {
        kr[i] = *reinterpret_cast<const uint32x4*>(kbase + (int64_t)kk * DH);
        vr[i] = *reinterpret_cast<const uint32x4*>(vbase + (int64_t)kk * DH);
      }
    }
    float qv[EPC];
#pragma unroll
    for (int j = 0; j < EPC; ++j) qv[j] = q[bh * DH + el + j];
    const float scale = rsqrtf((float)DH);
    // ---- scores
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int kk = (i * 4 + wave) * KPL + sub;
      float d = 0.f;
      if (kk < nk) {
        const uint32x4 w = kr[i];
        if (sizeof(T) == 2) {
          d = bf16_lo(w.x) * qv[0] + bf16_hi(w.x) * qv[1 % EPC] + bf16_lo(w.y) * qv[2 % EPC] + bf16_hi(w.y) * qv[3 % EPC] +
              bf16_lo(w.z) * qv[4 % EPC] + bf16_hi(w.z) * qv[5 % EPC] + bf16_lo(w.w) * qv[6 % EPC] + bf16_hi(w.w) * qv[7 % EPC];
        } else {
          d = __uint_as_float(w.x) * qv[0] + __uint_as_float(w.y) * qv[1] + __uint_as_float(w.z) * qv[2] +
              __uint_as_float(w.w) * qv[3];
        }
      }
#pragma unroll
      for (int o = LPK / 2; o > 0; o >>= 1) d += __shfl_xor(d, o);
      if (kk < nk && (lane % LPK) == 0) sc[kk] = d * scale;
    }
    __syncthreads();
    // ---- softmax statistics of the range (64 scores: one wavefront's worth, every wavefront redoes it)
    const float sv = (lane < nk) ? sc[lane] : -INFINITY;
    const float m = wave_max(sv);
    const float pv = (lane < nk) ? expf(sv - m) : 0.f;
    const float l = wave_sum(pv);
    // ---- weighted V from the registers
    float acc[EPC];
#pragma unroll
    for (int j = 0; j < EPC; ++j) acc[j] = 0.f;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int kk = (i * 4 + wave) * KPL + sub;
      const float p = __shfl(pv, kk < nk ? kk : 0);
      if (kk < nk) {
        const uint32x4 w = vr[i];
        if (sizeof(T) == 2) {
          acc[0] += p * bf16_lo(w.x); acc[1 % EPC] += p * bf16_hi(w.x);
          acc[2 % EPC] += p * bf16_lo(w.y); acc[3 % EPC] += p * bf16_hi(w.y);
          acc[4 % EPC] += p * bf16_lo(w.z); acc[5 % EPC] += p * bf16_hi(w.z);
          acc[6 % EPC] += p * bf16_lo(w.w); acc[7 % EPC] += p * bf16_hi(w.w);
        } else {
          acc[0] += p * __uint_as_float(w.x); acc[1] += p * __uint_as_float(w.y);
          acc[2] += p * __uint_as_float(w.z); acc[3] += p * __uint_as_float(w.w);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < EPC; ++j)
#pragma unroll
      for (int o = 32; o >= LPK; o >>= 1) acc[j] += __shfl_xor(acc[j], o);
    if (lane < LPK)
#pragma unroll
      for (int j = 0; j < EPC; ++j) part[wave][el + j] = acc[j];
    __syncthreads();
    for (int e = tid; e < DH; e += 256) wout[2 + e] = (part[0][e] + part[1][e]) + (part[2][e] + part[3][e]);
    if (tid == 0) { wout[0] = m; wout[1] = l; }
  }

}

// Grid (H, B): merge the partials of the non-empty splits.
template <int DH>
__global__ __launch_bounds__(256) void attn_combine_kernel(const float* __restrict__ work, const int32_t* __restrict__ pos,
                                                           int S, int H, int Tcap, void* __restrict__ out, int64_t ld_out,
                                                           int out_dtype) {
  __shared__ float wgt[64];
  const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int64_t bh = (int64_t)b * H + h;
  const int nvalid = (pos[b] + 1 < Tcap) ? pos[b] + 1 : Tcap;
  const int ns = (nvalid + DEC_CHUNK - 1) / DEC_CHUNK;    // non-empty splits (<= S <= 64)
  const float* wb = work + bh * S * (DH + 2);
  // The partial vectors do not depend on the weights: thread e requests element e of the first 16 partials before
  // the barrier behind which the weights are visible, so the merge costs one memory round trip after the weights'
  // own, not one per four splits.  (d_head <= 256: one element per thread.)
  static_assert(DH <= 256, "one element per thread");
  constexpr int G = 16;
  const int e = tid;
  float pv[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int s2 = g < ns ? g : ns - 1;                      // beyond the last split: a valid address, weight 0 below
    pv[g] = (e < DH) ? wb[(int64_t)s2 * (DH + 2) + 2 + e] : 0.f;
  }
  if (tid < 64) {
    const float ms = (tid < ns) ? wb[(int64_t)tid * (DH + 2)] : -INFINITY;
    const float ls = (tid < ns) ? wb[(int64_t)tid * (DH + 2) + 1] : 0.f;
    const float mm = wave_max(ms);
    const float f = (tid < ns) ? expf(ms - mm) : 0.f;
    const float lt = wave_sum(f * ls);
    wgt[tid] = f / lt;
  }
  __syncthreads();
  if (e < DH) {
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    for (int s0 = 0; s0 < ns; s0 += G) {
      if (s0 > 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int s2 = s0 + g < ns ? s0 + g : ns - 1;
          pv[g] = wb[(int64_t)s2 * (DH + 2) + 2 + e];
        }
      }
#pragma unroll
      for (int g = 0; g < G; g += 4) {
        a0 += (s0 + g < ns ? wgt[s0 + g] : 0.f) * pv[g];
        a1 += (s0 + g + 1 < ns ? wgt[s0 + g + 1] : 0.f) * pv[g + 1];
        a2 += (s0 + g + 2 < ns ? wgt[s0 + g + 2] : 0.f) * pv[g + 2];
        a3 += (s0 + g + 3 < ns ? wgt[s0 + g + 3] : 0.f) * pv[g + 3];
      }
    }
    store_as(out, (int64_t)b * ld_out + h * DH + e, (a0 + a1) + (a2 + a3), out_dtype);
  }
}

int decode_splits(int64_t Tcap) { return (int)((Tcap + DEC_CHUNK - 1) / DEC_CHUNK); }

}  // namespace

extern "C" int mtj_attn_prefill(const void* q, const void* k_cache, const void* v_t, const int32_t* pos0, int64_t B,
                                int64_t H, int64_t Tp, int64_t Tcap, int64_t dh, int64_t ldvt, void* out,
                                int64_t ld_out, int dtype, const int32_t* key_limit, void* stream) {
  MTJ_REQUIRE(q && k_cache && v_t && pos0 && out, MTJ_EINVAL, "mtj_attn_prefill: null pointer");
  MTJ_REQUIRE(B > 0 && H > 0 && Tp > 0 && Tp <= Tcap && ld_out >= H * dh && B < 65536 && H < 65536, MTJ_EINVAL,
              "mtj_attn_prefill: bad shape B=%lld H=%lld Tp=%lld Tcap=%lld", (long long)B, (long long)H,
              (long long)Tp, (long long)Tcap);
  const int esz = dtype == MTJ_BF16 ? 2 : 4;
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
  if (dtype == MTJ_BF16 && dh == 256) MTJ_PREFILL(bf16_t, 256, 4, 32);
  else if (dtype == MTJ_BF16 && dh == 64) MTJ_PREFILL(bf16_t, 64, 8, 64);
  else if (dtype == MTJ_F32 && dh == 256) MTJ_PREFILL(float, 256, 4, 32);
  else if (dtype == MTJ_F32 && dh == 64) MTJ_PREFILL(float, 64, 4, 32);
  else return mtj_fail(MTJ_EINVAL, "mtj_attn_prefill: unsupported dtype %d / d_head %lld (64 or 256)", dtype, (long long)dh);
#undef MTJ_PREFILL
  return mtj_check_launch("mtj_attn_prefill");
}

extern "C" int64_t mtj_attn_decode_work_bytes(int64_t B, int64_t H, int64_t dh, int64_t Tcap) {
  return B * H * (int64_t)decode_splits(Tcap) * (dh + 2) * (int64_t)sizeof(float);
}

namespace {

int attn_decode_impl(const char* who, const float* q, const void* k_cache, const void* v_cache, const int32_t* pos,
                     int64_t B, int64_t H, int64_t Tcap, int64_t dh, void* out, int64_t ld_out, int out_dtype, int dtype,
                     void* work, void* stream) {
  MTJ_REQUIRE(q && k_cache && v_cache && pos && out && work, MTJ_EINVAL, "%s: null pointer", who);
  MTJ_REQUIRE(B > 0 && H > 0 && Tcap > 0 && ld_out >= H * dh && B < 65536 && H < 65536, MTJ_EINVAL, "%s: bad shape", who);
  MTJ_REQUIRE(out_dtype == MTJ_F32 || out_dtype == MTJ_BF16, MTJ_EDTYPE, "%s: out_dtype %d", who, out_dtype);
  MTJ_REQUIRE(mtj_aligned16(q) && mtj_aligned16(k_cache) && mtj_aligned16(v_cache) && mtj_aligned16(work), MTJ_EALIGN,
              "%s: pointers must be 16-byte aligned", who);
  const int S = decode_splits(Tcap);
  MTJ_REQUIRE(S <= 64, MTJ_ELIMIT, "%s: window of %lld slots exceeds %d", who, (long long)Tcap, 64 * DEC_CHUNK);
  float* partials = reinterpret_cast<float*>(work);
  dim3 grid((unsigned)S, (unsigned)H, (unsigned)B);
  hipStream_t s = (hipStream_t)stream;
#define MTJ_DECODE(T, DH)                                                                                         \
  do {                                                                                                            \
    attn_decode_kernel<T, DH><<<grid, 256, 0, s>>>(q, (const T*)k_cache, (const T*)v_cache, pos, (int)H, (int)Tcap, \
                                                   partials);                                                     \
    attn_combine_kernel<DH><<<dim3((unsigned)H, (unsigned)B), 256, 0, s>>>(partials, pos, S, (int)H, (int)Tcap, out, \
                                                                           ld_out, out_dtype);                    \
  } while (0)
  if (dtype == MTJ_BF16 && dh == 256) MTJ_DECODE(bf16_t, 256);
  else if (dtype == MTJ_BF16 && dh == 64) MTJ_DECODE(bf16_t, 64);
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
                          stream);
}

// ------------------------------------------------------------------------------------------------
// The same two launches with the partial results kept in a device array that lives in the code object, for
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

extern "C" int64_t mtj_attn_decode_static_max_bytes(void) { return MTJ_ATTN_DECODE_STATIC_BYTES; }

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
                          dtype, work, stream);
}

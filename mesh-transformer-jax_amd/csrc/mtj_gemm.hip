// MFMA GEMM for prefill and batched decode: C[M, N] = A[M, K] x W[N, K]^T with fused epilogues.
// Both operands are K-contiguous and accumulation is float32; bf16 uses v_mfma_f32_32x32x16_bf16, float32 uses
// v_mfma_f32_32x32x2_f32 (true fp32).  Two kernels share the epilogues:
//   gemm_kernel      any dtype and shape: global -> registers -> LDS (padded rows, so that the 16-byte fragment
//                    reads of a 32x32 MFMA hit distinct banks), LDS double-buffered;
//   gemm_dma_kernel  large bf16 problems: 256x256x64 tiles written straight into LDS by the memory pipeline
//                    (buffer_load ... lds), rows xor-swizzled instead of padded, no staging registers.
#include "mtj_common.h"
#include <type_traits>

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
  __device__ static __forceinline__ void run16(floatx4& c, const frag& a, const frag& b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
  }
};
template <> struct mma<f16_t> {
  static constexpr int EPC = 8;
  struct frag { f16x8 v; };
  __device__ static __forceinline__ frag load(const f16_t* p) {
    frag f;
    f.v = *reinterpret_cast<const f16x8*>(p);
    return f;
  }
  __device__ static __forceinline__ void run(floatx16& c, const frag& a, const frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.v, b.v, c, 0, 0, 0);
  }
  __device__ static __forceinline__ void run16(floatx4& c, const frag& a, const frag& b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.v, b.v, c, 0, 0, 0);
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
  void* out;
  int64_t ldo;
  int out_dtype;
  float alpha;            // multiplies the accumulator first (undoes a power-of-two scale of the packed weights)
  int splits;             // > 1: blockIdx.y owns a K range and stores a raw float32 partial at out + y * split_stride
  int64_t split_stride;
  mtj_inproj ip;
  // MTJ_EPI_XENT: the product is never stored; per (row, column tile) the maximum and the sum of exp(logit - maximum)
  const int32_t* target;  // [M]
  float* pmax;            // [tiles_n, M]
  float* psum;            // [tiles_n, M]
  float* tlogit;          // [M]: the logit of the target column (written by the one tile that holds it)
};

constexpr int MTJ_EPI_XENT = 3;   // internal: logits + cross entropy (ProjectionShard.loss, layers.py:569-593)

// 16 consecutive elements, 16-byte vector stores (idx is a multiple of 16 elements, base 16-byte aligned)
__device__ __forceinline__ void store16(void* base, int64_t idx, const float* v, int dtype) {
  if (dtype == MTJ_F32) {
    floatx4* p = reinterpret_cast<floatx4*>(reinterpret_cast<float*>(base) + idx);
#pragma unroll
    for (int q = 0; q < 4; ++q) p[q] = floatx4{v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
  } else {
    uint32x4* p = reinterpret_cast<uint32x4*>(reinterpret_cast<uint16_t*>(base) + idx);
#pragma unroll
    for (int q = 0; q < 2; ++q)
      p[q] = uint32x4{pack_16x2(v[8 * q], v[8 * q + 1], dtype), pack_16x2(v[8 * q + 2], v[8 * q + 3], dtype),
                      pack_16x2(v[8 * q + 4], v[8 * q + 5], dtype), pack_16x2(v[8 * q + 6], v[8 * q + 7], dtype)};
  }
}

// compile-time loop over the accumulator tiles (i, j) of a wavefront: the indices must be constants for the
// accumulators to stay in registers
template <int I, int J, int WM, int WN, class F>
__device__ __forceinline__ void for_tiles(F&& f) {
  f(std::integral_constant<int, I>{}, std::integral_constant<int, J>{});
  if constexpr (I + 1 < WM) for_tiles<I + 1, J, WM, WN>(f);
  else if constexpr (J + 1 < WN) for_tiles<0, J + 1, WM, WN>(f);
}

template <int S, int NS, class F>
__device__ __forceinline__ void for_stages(F&& f) {
  f(std::integral_constant<int, S>{});
  if constexpr (S + 1 < NS) for_stages<S + 1, NS>(f);
}

// per-tile operands of the fused input-projection epilogue, fetched one tile ahead of their use:
// fc_in columns: 16 bias values; rotary q/k columns: 8 sines then 8 cosines
struct epi_ops { floatx4 o[4]; };

// Epilogue of a workgroup tile whose wavefront (wm, wn) holds WM x WN accumulator tiles of 32x32.  `smem` (the
// operand staging area, no longer needed) must hold 2*BM ints and one 32x36 float patch per wavefront.
// Two accumulator layouts:
//   MI16 false  acc is floatx16[WM][WN] from 32x32 MFMAs: register v of lane l holds C[8*(v/4) + 4*(l/32) + v%4][l%32];
//   MI16 true   acc is floatx4[2*WM][2*WN] from 16x16x32 MFMAs issued with the WEIGHT fragment as the first operand:
//               register v of lane l of block (i, j) holds C[16*i + l%16][16*j + 4*(l/16) + v], four consecutive
//               columns of one row, so stores are 8 or 16 bytes per lane.
template <int EPI, int WAVES_M, int WAVES_N, int WM, int WN, bool MI16 = false, class ACC>
__device__ __forceinline__ void epilogue(const gemm_args& a, void* out, ACC& acc, unsigned char* smem, int m0, int n0) {
  constexpr int NT = WAVES_M * WAVES_N * 64, BM = WAVES_M * WM * 32;
  constexpr int PS = 36;   // patch row stride in floats: 16-byte aligned rows, and 16-byte reads of 8 lanes hit distinct banks
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int fr = lane & 31, fg = lane >> 5;
  if (EPI == MTJ_EPI_XENT) {
    // Row statistics of this workgroup's column tile: accumulator register v of lane (fr, fg) is row 8*(v/4) + 4*fg +
    // v%4, column fr of a 32x32 tile, so a row is reduced over the WN tiles in registers, then over the 32 lanes
    // with the same fg by shuffles, then over the WAVES_N wavefronts through LDS.
    constexpr int BN = WAVES_N * WN * 32;
    __syncthreads();                                       // every wavefront is done with the operand tiles
    float* red = reinterpret_cast<float*>(smem);           // [WAVES_N][BM][2]
    if constexpr (MI16) {
      // a lane holds 4 columns of each of the 2*WN column blocks of its row; a row is completed by the four lanes
      // l%16 + 16*q, then by the WAVES_N wavefronts through LDS
      const int r16 = lane & 15, q16 = lane >> 4;
      float bias[2 * WN][4];
      bool ok[2 * WN][4];
#pragma unroll
      for (int j = 0; j < 2 * WN; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int n = n0 + (wn * WN * 2 + j) * 16 + 4 * q16 + v;
          ok[j][v] = n < a.N;
          bias[j][v] = (a.bias && ok[j][v]) ? a.bias[n] : 0.f;
        }
      for_tiles<0, 0, 2 * WM, 1>([&](auto I_, auto) {
        constexpr int i = decltype(I_)::value;
        const int r = (wm * WM * 2 + i) * 16 + r16;
        const int m = m0 + r;
        float val[2 * WN][4];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 2 * WN; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            val[j][v] = ok[j][v] ? acc[i][j][v] * a.alpha + bias[j][v] : -INFINITY;
            mx = fmaxf(mx, val[j][v]);
          }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        float sm = 0.f;
        if (mx != -INFINITY) {
#pragma unroll
          for (int j = 0; j < 2 * WN; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) sm += __expf(val[j][v] - mx);      // exp(-inf) = 0 for columns beyond N
        }
        sm += __shfl_xor(sm, 16);
        sm += __shfl_xor(sm, 32);
        if (m < a.M) {
          const int t = a.target[m];
#pragma unroll
          for (int j = 0; j < 2 * WN; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v)
              if (n0 + (wn * WN * 2 + j) * 16 + 4 * q16 + v == t) a.tlogit[m] = val[j][v];
        }
        if (q16 == 0) {
          red[(wn * BM + r) * 2] = mx;
          red[(wn * BM + r) * 2 + 1] = sm;
        }
      });
    } else
    for_tiles<0, 0, WM, 1>([&](auto I_, auto) {
      constexpr int i = decltype(I_)::value;
      float val[WN][16];
      int col[WN];
      for_tiles<0, 0, 1, WN>([&](auto, auto J_) {
        constexpr int j = decltype(J_)::value;
        const int n = n0 + (wn * WN + j) * 32 + fr;
        col[j] = n;
        const bool n_ok = n < a.N;
        const float bias = (a.bias && n_ok) ? a.bias[n] : 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) val[j][v] = n_ok ? acc[i][j][v] * a.alpha + bias : -INFINITY;
      });
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = (wm * WM + i) * 32 + 8 * (v / 4) + 4 * fg + (v % 4);
        const int m = m0 + r;
        float mx = val[0][v];
#pragma unroll
        for (int j = 1; j < WN; ++j) mx = fmaxf(mx, val[j][v]);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        float sm = 0.f;
        if (mx != -INFINITY) {
#pragma unroll
          for (int j = 0; j < WN; ++j) sm += __expf(val[j][v] - mx);      // exp(-inf) = 0 for columns beyond N
        }
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) sm += __shfl_xor(sm, o);
        if (m < a.M) {
          const int t = a.target[m];
#pragma unroll
          for (int j = 0; j < WN; ++j)
            if (col[j] == t) a.tlogit[m] = val[j][v];
        }
        if (fr == 0) {
          red[(wn * BM + r) * 2] = mx;
          red[(wn * BM + r) * 2 + 1] = sm;
        }
      }
    });
    __syncthreads();
    const int tn = n0 / BN;
    for (int r = tid; r < BM; r += NT) {
      const int m = m0 + r;
      if (m >= a.M) continue;
      float mx = -INFINITY;
#pragma unroll
      for (int w = 0; w < WAVES_N; ++w) mx = fmaxf(mx, red[(w * BM + r) * 2]);
      float sm = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES_N; ++w) {
        const float pm = red[(w * BM + r) * 2];
        sm += pm == -INFINITY ? 0.f : __expf(pm - mx) * red[(w * BM + r) * 2 + 1];
      }
      a.pmax[(int64_t)tn * a.M + m] = mx;
      a.psum[(int64_t)tn * a.M + m] = sm;
    }
  } else if (EPI == MTJ_EPI_INPROJ) {
    // Each 32x32 accumulator tile goes through a private LDS patch of its wavefront and comes back with one
    // lane owning 16 consecutive columns of one row: rotary pairs are then lane-local and every destination
    // (q, K/V window, gelu(fc_in)) gets 32- or 64-byte stores.
    __syncthreads();                                       // every wavefront is done with the operand tiles
    int* row_b = reinterpret_cast<int*>(smem);
    int* row_pos = row_b + BM;
    float* patch = reinterpret_cast<float*>(smem) + 2 * BM + wave * (32 * PS);
    for (int r = tid; r < BM; r += NT) {
      const int m = m0 + r;
      int b = 0, pos = -1;
      if (m < a.M) {
        b = m / a.ip.Tp;
        pos = a.ip.pos0[b] + (m - b * a.ip.Tp);
      }
      row_b[r] = b;
      row_pos[r] = pos;
    }
    __syncthreads();
    const int d = a.ip.n_heads * a.ip.d_head, dh = a.ip.d_head, rd = a.ip.rotary_dims, Tp = a.ip.Tp;
    const int prow = lane >> 1, pcol = (lane & 1) * 16;     // my row / first column inside a tile

    // tile-uniform facts of accumulator tile column j, and my first column inside its segment
    struct col_info { bool is_fc, n_ok; int seg, c0, h, e0; };
    auto column = [&](int j) {
      col_info c;
      const int nb = n0 + (wn * WN + j) * 32;               // first column of the tile
      c.is_fc = nb >= 3 * d;
      c.seg = c.is_fc ? 3 : nb / d;                         // 0 q, 1 v, 2 k
      c.c0 = nb - c.seg * d + pcol;
      c.h = c.c0 / dh;
      c.e0 = c.c0 - c.h * dh;
      c.n_ok = nb + pcol < a.N;                             // N is a multiple of 16 columns here
      return c;
    };
    auto load_ops = [&](int i, int j) {
      epi_ops p;
#pragma unroll
      for (int q = 0; q < 4; ++q) p.o[q] = floatx4{0.f, 0.f, 0.f, 0.f};
      const col_info c = column(j);
      if (!c.n_ok) return p;
      if (c.is_fc) {
        const floatx4* bp = reinterpret_cast<const floatx4*>(a.bias + c.c0);   // c0 is a multiple of 16
#pragma unroll
        for (int q = 0; q < 4; ++q) p.o[q] = bp[q];
      } else if (c.seg != 1 && c.e0 < rd) {                 // rd is a multiple of 16 (checked on the host)
        const int pos = row_pos[(wm * WM + i) * 32 + prow];
        if (pos >= 0) {
          const int pp = pos < a.ip.max_pos ? pos : a.ip.max_pos - 1;
          const floatx4* sp = reinterpret_cast<const floatx4*>(a.ip.sin_tab + (int64_t)pp * (rd / 2) + (c.e0 >> 1));
          const floatx4* cp = reinterpret_cast<const floatx4*>(a.ip.cos_tab + (int64_t)pp * (rd / 2) + (c.e0 >> 1));
          p.o[0] = sp[0]; p.o[1] = sp[1]; p.o[2] = cp[0]; p.o[3] = cp[1];
        }
      }
      return p;
    };
    epi_ops cur = load_ops(0, 0);
    for_tiles<0, 0, WM, WN>([&](auto I_, auto J_) {
      constexpr int i = decltype(I_)::value, j = decltype(J_)::value;
      constexpr int ni = i + 1 < WM ? i + 1 : 0, nj = i + 1 < WM ? j : j + 1;
      epi_ops nxt = cur;
      if constexpr (nj < WN) nxt = load_ops(ni, nj);
      const col_info c = column(j);
      if constexpr (MI16) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj)
            *reinterpret_cast<floatx4*>(patch + (ii * 16 + (lane & 15)) * PS + jj * 16 + 4 * (lane >> 4)) =
                acc[2 * i + ii][2 * j + jj] * a.alpha;
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) patch[(8 * (v / 4) + 4 * fg + (v % 4)) * PS + fr] = acc[i][j][v] * a.alpha;
      }
      __builtin_amdgcn_wave_barrier();
      float val[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const floatx4 t = *reinterpret_cast<const floatx4*>(patch + prow * PS + pcol + 4 * q);
        val[4 * q] = t.x; val[4 * q + 1] = t.y; val[4 * q + 2] = t.z; val[4 * q + 3] = t.w;
      }
      __builtin_amdgcn_wave_barrier();
      const int r = (wm * WM + i) * 32 + prow;
      const int m = m0 + r;
      if (m < a.M && c.n_ok) {
        if (c.is_fc) {
#pragma unroll
          for (int k = 0; k < 16; ++k) val[k] = gelu_tanh(val[k] + cur.o[k >> 2][k & 3]);
          store16(a.ip.act, (int64_t)m * a.ip.ld_act + d + c.c0, val, a.ip.act_dtype);
        } else {
          const int pos = row_pos[r];
          if (pos >= 0) {
            const int b = row_b[r];
            if (c.seg != 1 && c.e0 < rd) {
#pragma unroll
              for (int k = 0; k < 16; k += 2) {
                const float sn = cur.o[k >> 3][(k >> 1) & 3], cs = cur.o[2 + (k >> 3)][(k >> 1) & 3];
                const float x0 = val[k], x1 = val[k + 1];
                val[k] = x0 * cs - x1 * sn;
                val[k + 1] = x1 * cs + x0 * sn;
              }
            }
            const int64_t bh = (int64_t)b * a.ip.n_heads + c.h;
            if (c.seg == 0) {
              store16(a.ip.q, (bh * Tp + (m - b * Tp)) * dh + c.e0, val, a.ip.q_dtype);
            } else {
              const int slot = pos % a.ip.Tcap;
              store16(c.seg == 1 ? a.ip.v_cache : a.ip.k_cache, (bh * a.ip.Tcap + slot) * dh + c.e0, val, a.ip.kv_dtype);
              if (c.seg == 1 && a.ip.v_t && pos < a.ip.ldvt) {
#pragma unroll
                for (int k = 0; k < 16; ++k) store_as(a.ip.v_t, (bh * dh + c.e0 + k) * a.ip.ldvt + pos, val[k], a.ip.kv_dtype);
              }
            }
          }
        }
      }
      cur = nxt;
    });
  } else if constexpr (MI16) {
    // four consecutive columns per lane: 16-byte (float32) or 8-byte (16-bit) accesses when the rows of `out` allow it
    const int r16 = lane & 15, q16 = lane >> 4;
    const int esz = (EPI == MTJ_EPI_RESID || a.out_dtype == MTJ_F32) ? 4 : 2;
    const bool vec = a.ldo % 4 == 0 && (reinterpret_cast<uintptr_t>(out) % (4 * esz)) == 0;
    for_tiles<0, 0, 1, 2 * WN>([&](auto, auto J_) {
      constexpr int j = decltype(J_)::value;
      const int nb = n0 + (wn * WN * 2 + j) * 16 + 4 * q16;
      float bias[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) bias[v] = (a.bias && nb + v < a.N) ? a.bias[nb + v] : 0.f;
      const bool full = vec && nb + 3 < a.N;
      for_tiles<0, 0, 2 * WM, 1>([&](auto I_, auto) {
        constexpr int i = decltype(I_)::value;
        const int m = m0 + (wm * WM * 2 + i) * 16 + r16;
        if (m >= a.M) return;
        const int64_t idx = (int64_t)m * a.ldo + nb;
        float val[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) val[v] = acc[i][j][v] * a.alpha + bias[v];
        if (full) {
          if (EPI == MTJ_EPI_RESID) {
            floatx4* o = reinterpret_cast<floatx4*>(reinterpret_cast<float*>(out) + idx);
            const floatx4 old = *o;
            *o = floatx4{old.x + val[0], old.y + val[1], old.z + val[2], old.w + val[3]};
          } else if (a.out_dtype == MTJ_F32) {
            *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(out) + idx) = floatx4{val[0], val[1], val[2], val[3]};
          } else {
            *reinterpret_cast<uint32x2*>(reinterpret_cast<uint16_t*>(out) + idx) =
                uint32x2{pack_16x2(val[0], val[1], a.out_dtype), pack_16x2(val[2], val[3], a.out_dtype)};
          }
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (nb + v < a.N) {
              if (EPI == MTJ_EPI_RESID) reinterpret_cast<float*>(out)[idx + v] += val[v];
              else store_as(out, idx + v, val[v], a.out_dtype);
            }
        }
      });
    });
  } else {
    for_tiles<0, 0, WM, WN>([&](auto I_, auto J_) {
      constexpr int i = decltype(I_)::value, j = decltype(J_)::value;
      const int n = n0 + (wn * WN + j) * 32 + fr;
      const bool n_ok = n < a.N;
      const float bias = (a.bias && n_ok) ? a.bias[n] : 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + (wm * WM + i) * 32 + 8 * (v / 4) + 4 * fg + (v % 4);
        if (m < a.M && n_ok) {
          const int64_t idx = (int64_t)m * a.ldo + n;
          const float val = acc[i][j][v] * a.alpha + bias;
          if (EPI == MTJ_EPI_RESID) reinterpret_cast<float*>(out)[idx] += val;
          else store_as(out, idx, val, a.out_dtype);
        }
      }
    });
  }
}

// Workgroup tile (WAVES_M*WM*32) x (WAVES_N*WN*32), K step BK elements, NS register stages, epilogue EPI.
//
// Pipeline: k-tile kt is multiplied out of LDS (two buffers) while the loads of k-tiles kt+1 .. kt+NS sit in
// registers or are still in flight; one k-tile in flight does not cover the load latency of a loaded GPU.
// Global reads are bounds-checked buffer loads (rows beyond M or N read as zero), whose addressing needs one
// VGPR per operand: the per-chunk and per-k-tile offsets are scalar.
template <typename T, int EPI, int WAVES_M, int WAVES_N, int WM, int WN, int BK, int NS>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_kernel(const gemm_args a) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
  constexpr int EPC = mma<T>::EPC;
  constexpr int ESZ = (int)sizeof(T);
  constexpr int CPR = BK / EPC;          // 16-byte chunks per tile row
  constexpr int LDS_ROW = BK + EPC;      // padded row, elements (row stride 144 B for both types)
  constexpr int A_CHUNKS = BM * CPR / NT, B_CHUNKS = BN * CPR / NT;
  constexpr int ROWS_PER_PASS = NT / CPR;   // tile rows covered by one chunk index
  static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0 && NT % CPR == 0, "tile does not divide over threads");
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

  // buffer resources over the rows of this tile: [m0, min(M, m0+BM)) of A and [n0, min(N, n0+BN)) of W
  const int rows_a = (a.M - m0 < BM) ? a.M - m0 : BM, rows_b = (a.N - n0 < BN) ? a.N - n0 : BN;
  const T* tile_a = reinterpret_cast<const T*>(a.A) + (int64_t)m0 * a.lda;
  const T* tile_b = reinterpret_cast<const T*>(a.W) + (int64_t)n0 * a.K;
  const __amdgpu_buffer_rsrc_t ra_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(tile_a), 0, (int)((((int64_t)rows_a - 1) * a.lda + a.K) * ESZ), 0x00020000);
  const __amdgpu_buffer_rsrc_t rb_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(tile_b), 0, (int)((((int64_t)rows_b - 1) * a.K + a.K) * ESZ), 0x00020000);
  const int row0 = tid / CPR, cc0 = tid % CPR;
  const int voff_a = (int)(((int64_t)row0 * a.lda + cc0 * EPC) * ESZ);
  const int voff_b = (int)(((int64_t)row0 * a.K + cc0 * EPC) * ESZ);
  const int pass_a = (int)((int64_t)ROWS_PER_PASS * a.lda * ESZ), pass_b = (int)((int64_t)ROWS_PER_PASS * a.K * ESZ);

  const int kt0 = (int)((int64_t)blockIdx.y * (a.K / BK) / a.splits);   // first k-tile of my K range
  const int KT = (int)((int64_t)(blockIdx.y + 1) * (a.K / BK) / a.splits) - kt0;
  // With few rows the weights are streamed once and every workgroup would ask for the same k offset of its rows at
  // the same time - addresses that differ by multiples of the row pitch, a power of two, which crowd into few memory
  // channels.  Each workgroup therefore starts its walk over k at a different k-tile and wraps around (M = 32,
  // N = 28672, K = 4096: 48.8 -> 41.5 us; which multiplier spreads the starts does not matter).  The start is a function
  // of the column tile alone: an output row is summed in the same order whatever else is in the batch.
  const int krot = BM <= 64 ? (int)(((unsigned)tn * 5u) % (unsigned)KT) : 0;
  uint32x4 ra[NS][A_CHUNKS], rb[NS][B_CHUNKS];
  auto load_global = [&](auto ST_, int kt) {
    constexpr int st = decltype(ST_)::value;
    const int kr = kt + krot;
    const int koff = (kt0 + (kr >= KT ? kr - KT : kr)) * BK * ESZ;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i)
      ra[st][i] = __builtin_amdgcn_raw_buffer_load_b128(ra_rsrc, voff_a, koff + i * pass_a, 0);
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i)
      rb[st][i] = __builtin_amdgcn_raw_buffer_load_b128(rb_rsrc, voff_b, koff + i * pass_b, BM <= 64 ? 2 : 0);  // nt: streamed once
  };
  auto store_lds = [&](auto ST_, int buf) {
    constexpr int st = decltype(ST_)::value;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i)
      *reinterpret_cast<uint32x4*>(As + (buf * BM + row0 + i * ROWS_PER_PASS) * LDS_ROW + cc0 * EPC) = ra[st][i];
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i)
      *reinterpret_cast<uint32x4*>(Bs + (buf * BN + row0 + i * ROWS_PER_PASS) * LDS_ROW + cc0 * EPC) = rb[st][i];
  };

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // k-tile t lives in register stage t % NS.  Prologue: request k-tiles 0 .. NS-1, park k-tile 0 in LDS,
  // reuse its stage for k-tile NS.
  for_stages<0, NS>([&](auto ST_) {
    if (decltype(ST_)::value < KT) load_global(ST_, decltype(ST_)::value);
  });
  store_lds(std::integral_constant<int, 0>{}, 0);
  if (NS < KT) load_global(std::integral_constant<int, 0>{}, NS);
  __syncthreads();

  // one k-tile; PARK = stage of k-tile kt+1 (a compile-time index: the k loop is unrolled by NS).  STEADY: k-tiles
  // kt+1 and kt+1+NS both exist, so the park and the request are unconditional.  That matters: the wait the
  // compiler puts before the park is the strictest over all paths that reach it, and with the request under a
  // condition that is "everything outstanding", the request of one iteration ago included.
  auto k_tile = [&](int kt, auto PARK_, auto STEADY_) {
    constexpr bool steady = decltype(STEADY_)::value;
    const int buf = kt & 1;
    const T* as = As + (buf * BM + wm * WM * 32 + fr) * LDS_ROW + fg * 8;
    const T* bs = Bs + (buf * BN + wn * WN * 32 + fr) * LDS_ROW + fg * 8;
    // fragments of k-step ks+1 are read from LDS while the MFMAs of k-step ks run
    typename mma<T>::frag fa[2][WM], fb[2][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i) fa[0][i] = mma<T>::load(as + i * 32 * LDS_ROW);
#pragma unroll
    for (int j = 0; j < WN; ++j) fb[0][j] = mma<T>::load(bs + j * 32 * LDS_ROW);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < BK / 16) {
#pragma unroll
        for (int i = 0; i < WM; ++i) fa[nxt][i] = mma<T>::load(as + i * 32 * LDS_ROW + (ks + 1) * 16);
#pragma unroll
        for (int j = 0; j < WN; ++j) fb[nxt][j] = mma<T>::load(bs + j * 32 * LDS_ROW + (ks + 1) * 16);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) mma<T>::run(acc[i][j], fa[cur][i], fb[cur][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (steady || kt + 1 < KT) store_lds(PARK_, buf ^ 1);
    if (steady || kt + 1 + NS < KT) load_global(PARK_, kt + 1 + NS);
    __syncthreads();
  };
  int kt = 0;
  for (; kt + 2 * NS < KT; kt += NS)          // the last k-tile of the round, kt+NS-1, still requests kt+2*NS
    for_stages<0, NS>([&](auto S_) {
      constexpr int s = decltype(S_)::value;
      k_tile(kt + s, std::integral_constant<int, (s + 1) % NS>{}, std::true_type{});
    });
  for (; kt < KT; kt += NS)
    for_stages<0, NS>([&](auto S_) {
      constexpr int s = decltype(S_)::value;
      if (kt + s < KT) k_tile(kt + s, std::integral_constant<int, (s + 1) % NS>{}, std::false_type{});
    });

  void* out = a.splits > 1 ? (void*)(reinterpret_cast<float*>(a.out) + blockIdx.y * a.split_stride) : a.out;
  epilogue<EPI, WAVES_M, WAVES_N, WM, WN>(a, out, acc, smem, m0, n0);
}

// 16-bit operands, 256x256 workgroup tile, 8 wavefronts of 128x64, K step 64, two LDS stages of 64 KiB,
// v_mfma_f32_16x16x32 (under the board's power limit it sustains a higher clock than the 32x32x16 form: 1820 against
// 1570 TFLOP/s in a register-only loop on random float16 data).
//
// The memory pipeline writes the operand tiles straight into LDS (buffer_load_dwordx4 ... lds: 64 lanes x
// 16 bytes land at consecutive LDS addresses), so there are no staging registers and no ds_write.  A tile row is
// 128 bytes = 8 chunks; LDS position (row, c) holds chunk c ^ ((row >> 1) & 7) of the row, which each lane arranges
// by choosing its global address, and which makes the 16-byte fragment reads of 16 consecutive rows hit 16 distinct
// bank groups without padding.  Rows beyond M or N are outside the buffer resource and read as zero.
//
// The two wavefronts of a SIMD (wave w and w + 4) never compete for the matrix pipe: a k-tile is eight clusters,
// memory clusters (fragment reads from LDS, two global->LDS loads, the wait for an older load) alternating with
// MFMA clusters (one quarter of the wavefront's tile: 64 rows x 32 columns x 64 k = 16 MFMAs), every cluster ends
// in a workgroup barrier, and wavefronts 4..7 run one cluster behind wavefronts 0..3, so that at any time four
// wavefronts multiply while the other four read.  Operands are loaded in four sets per k-tile (A rows / W rows
// of the first and second half of every wavefront's tile) in the order the clusters consume them, each set into
// the place of the same set two k-tiles earlier as soon as both groups have read that one; every load is issued
// nine to ten clusters before its first reader.
template <typename T, int EPI>
__global__ __launch_bounds__(512) void gemm_dma_kernel(const gemm_args a) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  constexpr int WAVES_M = 2, WAVES_N = 4, WM = 4, WN = 2, BM = 256, BN = 256, BK = 64;
  constexpr int ROWB = BK * 2, OPB = BM * ROWB, STAGEB = 2 * OPB;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int fr = lane & 15, fq = lane >> 4;

  // tile id: contiguous tile ranges per XCD; the 32 workgroups that an XCD runs at a time form 8 x 4 tiles (row-tiles x
  // column-tiles), or 4 x 8 when the problem has few column-tiles (the out projection: each row panel is then fetched
  // from memory twice instead of four times, the small weight matrix more often; 1.4 % faster there, 0.9 % slower on
  // the input projection)
  const int tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
  const int nblk = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int per = nblk / 8;
    if (pid < per * 8) pid = (pid % 8) * per + pid / 8;
  }
  const int GM = tiles_n <= 16 ? 4 : 8;
  const int group = pid / (GM * tiles_n);
  const int first_m = group * GM;
  const int gsz = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
  const int tm = first_m + (pid % (GM * tiles_n)) % gsz;
  const int tn = (pid % (GM * tiles_n)) / gsz;
  const int m0 = tm * BM, n0 = tn * BN;

  const int rows_a = (a.M - m0 < BM) ? a.M - m0 : BM, rows_b = (a.N - n0 < BN) ? a.N - n0 : BN;
  const T* tile_a = reinterpret_cast<const T*>(a.A) + (int64_t)m0 * a.lda;
  const T* tile_b = reinterpret_cast<const T*>(a.W) + (int64_t)n0 * a.K;
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(tile_a), 0, (int)((((int64_t)rows_a - 1) * a.lda + a.K) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T*>(tile_b), 0, (int)((((int64_t)rows_b - 1) * a.K + a.K) * 2), 0x00020000);

  // a wavefront load = 8 rows x 128 bytes at 1 KiB of consecutive LDS; lane l fetches, for LDS position l % 8 of
  // row l / 8, chunk (l % 8) ^ swizzle(row): every row base used below is a multiple of 8 whose bit 3 is wave & 1
  const int chunk = (lane & 7) ^ ((lane >> 4) & 3) ^ ((wave & 1) << 2);
  const int voff_a = (int)((int64_t)(lane >> 3) * a.lda * 2) + chunk * 16;
  const int voff_b = (int)((int64_t)(lane >> 3) * a.K * 2) + chunk * 16;
  // my two loads of a set: A rows wave*8 and 128 + wave*8 (+64 for the second-half set), W rows
  // (wave/4)*64 + (wave%4)*8 and 128 more (+32 for the second-half set)
  const int ra0 = wave * 8, rb0 = (wave >> 2) * 64 + (wave & 3) * 8;

  // my K range (split-K: blockIdx.y; the whole of K otherwise), in k-tiles
  const int kt0 = (int)((int64_t)blockIdx.y * (a.K / BK) / a.splits);
  const int KT = (int)((int64_t)(blockIdx.y + 1) * (a.K / BK) / a.splits) - kt0;
  // Every operand row of a k-tile lies at the same offset inside its row, and the rows are a power of two apart: when
  // the whole chip walks k in step it asks at any moment for addresses that fall into few memory channels.  With one
  // group of row tiles (a short prompt: every XCD then has its own range of column tiles, and all workgroups run at
  // once) the walk starts an eighth of the k range further on in every eighth of the column tiles and wraps around:
  // the workgroups of an XCD still walk together and share their activation panels through its L2, the XCDs do not.
  // The start depends on the column tile alone.
  const int krot = tiles_m <= 8 ? (int)((((int64_t)tn * 8) / tiles_n) * KT / 8) : 0;

  // set 0: A first half, 1: W first half, 2: W second half, 3: A second half
  auto issue = [&](int st, int kt, auto SET_) {
    constexpr int set = decltype(SET_)::value;
    const int kr = kt + krot;
    const int koff = (kt0 + (kr >= KT ? kr - KT : kr)) * ROWB;
    // a k-tile beyond the range is requested all the same (the wait counts stay the same in every k-tile) but with an
    // offset far outside the buffer: such a load fetches nothing and writes zeros into a stage that is not read again
    const int beyond = kt < KT ? 0 : 0x40000000;
    if constexpr (set == 0 || set == 3) {
      const int r = ra0 + (set == 3 ? 64 : 0);
      unsigned char* d = smem + st * STAGEB + r * ROWB;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr)d, 16, voff_a + beyond, koff + (int)((int64_t)r * a.lda * 2), 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr)(d + 128 * ROWB), 16, voff_a + beyond,
                                               koff + (int)((int64_t)(r + 128) * a.lda * 2), 0, 0);
    } else {
      const int r = rb0 + (set == 2 ? 32 : 0);
      unsigned char* d = smem + st * STAGEB + OPB + r * ROWB;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr)d, 16, voff_b + beyond, koff + (int)((int64_t)r * a.K * 2), 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr)(d + 128 * ROWB), 16, voff_b + beyond,
                                               koff + (int)((int64_t)(r + 128) * a.K * 2), 0, 0);
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

  floatx4 acc[2 * WM][2 * WN];
#pragma unroll
  for (int i = 0; i < 2 * WM; ++i)
#pragma unroll
    for (int j = 0; j < 2 * WN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  issue(0, 0, I0{}); issue(0, 0, I1{}); issue(0, 0, I2{}); issue(0, 0, I3{});
  issue(1, 1, I0{}); issue(1, 1, I1{});

  // fragments of a 16x16x32 MFMA: lane (fr, fq) supplies elements [8*fq, 8*fq + 8) of the 32-wide k-step of row fr
  int xo[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) xo[ks] = ((4 * ks + fq) ^ ((fr >> 1) & 7)) * 16;
  const int a_row = (wm * 128 + fr) * ROWB, b_row = OPB + (wn * 64 + fr) * ROWB;
  typename mma<T>::frag fa[2 * WM][2], fb[2 * WN][2];
  // read number n = 4*ks + i of A half h (row blocks 4h .. 4h+3), reads [n_lo, n_hi)
  auto read_a = [&](int st, int h, int n_lo, int n_hi) {
#pragma unroll
    for (int n = 0; n < 8; ++n)
      if (n >= n_lo && n < n_hi)
        fa[4 * h + (n & 3)][n >> 2] =
            mma<T>::load(reinterpret_cast<const T*>(smem + st * STAGEB + a_row + (4 * h + (n & 3)) * 16 * ROWB + xo[n >> 2]));
  };
  auto read_b = [&](int st, int h) {
#pragma unroll
    for (int n = 0; n < 4; ++n)
      fb[2 * h + (n & 1)][n >> 1] =
          mma<T>::load(reinterpret_cast<const T*>(smem + st * STAGEB + b_row + (2 * h + (n & 1)) * 16 * ROWB + xo[n >> 1]));
  };
  // 64 rows (A half ha) x 32 columns (W half hb) x 64: the two MFMAs of an accumulator are 8 instructions apart
  auto multiply = [&](auto HA_, auto HB_) {
    constexpr int ha = decltype(HA_)::value, hb = decltype(HB_)::value;
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) mma<T>::run16(acc[4 * ha + i][2 * hb + j], fb[2 * hb + j][ks], fa[4 * ha + i][ks]);
    __builtin_amdgcn_s_setprio(0);
  };
  // end of a memory cluster: the set that the next memory cluster reads was issued four sets ago
  auto landed = [&]() { __builtin_amdgcn_s_waitcnt(wait_vmcnt(8)); };
  auto cluster_end = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  landed();
  __builtin_amdgcn_s_barrier();
  if (wm) __builtin_amdgcn_s_barrier();        // wavefronts 4..7 start one cluster late
  __builtin_amdgcn_sched_barrier(0);
  read_a(0, 0, 0, 6);

  // k-tile kt in stage st; fragment reads per memory cluster: 6 + 6 + 4 + 8
  auto k_tile = [&](int kt, auto ST_) {
    constexpr int st = decltype(ST_)::value;
    read_a(st, 0, 6, 8);
    read_b(st, 0);
    issue(st ^ 1, kt + 1, I2{});
    landed();
    cluster_end();
    multiply(I0{}, I0{});
    cluster_end();
    read_b(st, 1);
    issue(st ^ 1, kt + 1, I3{});
    landed();
    cluster_end();
    multiply(I0{}, I1{});
    cluster_end();
    read_a(st, 1, 0, 8);
    issue(st, kt + 2, I0{});
    landed();
    cluster_end();
    multiply(I1{}, I0{});
    cluster_end();
    read_a(st ^ 1, 0, 0, 6);                   // of k-tile kt+1
    issue(st, kt + 2, I1{});
    landed();
    cluster_end();
    multiply(I1{}, I1{});
    cluster_end();
  };
  int kt = 0;
  for (; kt + 1 < KT; kt += 2) {
    k_tile(kt, I0{});
    k_tile(kt + 1, I1{});
  }
  if (kt < KT) k_tile(kt, I0{});
  __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));   // the surplus loads land before this workgroup's LDS is given away
  if (!wm) __builtin_amdgcn_s_barrier();
  __syncthreads();                             // every wavefront's loads have landed: the epilogue may reuse the stages

  void* out = a.splits > 1 ? (void*)(reinterpret_cast<float*>(a.out) + blockIdx.y * a.split_stride) : a.out;
  epilogue<EPI, WAVES_M, WAVES_N, WM, WN, true>(a, out, acc, smem, m0, n0);
}

template <typename T, int EPI>
int launch_dma(const gemm_args& a, hipStream_t s) {
  constexpr size_t lds = 2 * 2 * 256 * 64 * 2;
  static mtj_device_once once;
  if (int rc = mtj_allow_lds(once, "mtj_gemm", &gemm_dma_kernel<T, EPI>, lds)) return rc;
  const int tiles = ((a.M + 255) / 256) * ((a.N + 255) / 256);
  gemm_dma_kernel<T, EPI><<<dim3(tiles, a.splits), 512, lds, s>>>(a);
  return mtj_check_launch("mtj_gemm");
}

template <typename T, int EPI, int WAVES_M, int WAVES_N, int WM, int WN, int BK, int NS>
int launch(const gemm_args& a, hipStream_t s) {
  constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
  constexpr size_t lds = 2 * (size_t)(BM + BN) * (BK + mma<T>::EPC) * sizeof(T);
  static_assert(lds <= 160 * 1024, "tile does not fit LDS");
  static_assert(lds >= 2 * BM * sizeof(int) + WAVES_M * WAVES_N * 32 * 36 * sizeof(float), "epilogue scratch does not fit");
  static mtj_device_once once;
  if (int rc = mtj_allow_lds(once, "mtj_gemm", &gemm_kernel<T, EPI, WAVES_M, WAVES_N, WM, WN, BK, NS>, lds)) return rc;
  const int tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  gemm_kernel<T, EPI, WAVES_M, WAVES_N, WM, WN, BK, NS><<<dim3(tiles, a.splits), WAVES_M * WAVES_N * 64, lds, s>>>(a);
  return mtj_check_launch("mtj_gemm");
}

template <typename T, int EPI, int BK>
int dispatch_tile(const gemm_args& a, hipStream_t s) {
  if (a.M <= 32) return launch<T, EPI, 1, 4, 1, 1, BK, 2>(a, s);    // 32 x 128: batched decode, weights stream once
  if (a.M <= 64) return launch<T, EPI, 1, 4, 2, 1, BK, 2>(a, s);    // 64 x 128
  if constexpr (sizeof(T) == 2) {
    // e.g. M = 16384, N = 28672 or N = 4096 (a whole 6B layer at 8 x 2048 tokens): 7168 / 1024 tiles
    const int64_t big = (int64_t)((a.M + 255) / 256) * ((a.N + 255) / 256);
    if (big * a.splits >= 200) return launch_dma<T, EPI>(a, s);                         // 256 x 256, 8 wavefronts of 128 x 64
  }
  return launch<T, EPI, 2, 2, 2, 2, BK, 2>(a, s);                   // 128 x 128
}

template <typename T, int BK>
int dispatch(const gemm_args& a, int epi, hipStream_t s) {
  if (epi == MTJ_EPI_STORE) return dispatch_tile<T, MTJ_EPI_STORE, BK>(a, s);
  if (epi == MTJ_EPI_RESID) return dispatch_tile<T, MTJ_EPI_RESID, BK>(a, s);
  if (epi == MTJ_EPI_XENT) return dispatch_tile<T, MTJ_EPI_XENT, BK>(a, s);
  return dispatch_tile<T, MTJ_EPI_INPROJ, BK>(a, s);
}

// sums the per-split partial tiles in a fixed order and applies the epilogue (four columns per thread)
template <int EPI>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ work, int splits, int64_t split_stride,
                                                            int M, int N, const float* __restrict__ bias, void* out,
                                                            int64_t ldo, int out_dtype) {
  const int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;     // quad index over [M, N / 4]
  const int nq = N / 4;
  if (q >= (int64_t)M * nq) return;
  const int m = (int)(q / nq), n = (int)(q - (int64_t)m * nq) * 4;
  floatx4 acc = *reinterpret_cast<const floatx4*>(work + (int64_t)m * N + n);
  for (int sp = 1; sp < splits; ++sp) {
    const floatx4 p = *reinterpret_cast<const floatx4*>(work + sp * split_stride + (int64_t)m * N + n);
    acc.x += p.x; acc.y += p.y; acc.z += p.z; acc.w += p.w;
  }
  if (bias) {
    const floatx4 b = *reinterpret_cast<const floatx4*>(bias + n);
    acc.x += b.x; acc.y += b.y; acc.z += b.z; acc.w += b.w;
  }
  const int64_t idx = (int64_t)m * ldo + n;
  if (EPI == MTJ_EPI_RESID) {
    float* o = reinterpret_cast<float*>(out) + idx;
    o[0] += acc.x; o[1] += acc.y; o[2] += acc.z; o[3] += acc.w;
  } else if (out_dtype == MTJ_F32) {
    float* o = reinterpret_cast<float*>(out) + idx;
    o[0] = acc.x; o[1] = acc.y; o[2] = acc.z; o[3] = acc.w;
  } else {
    uint32x2 pk;
    pk.x = pack_16x2(acc.x, acc.y, out_dtype);
    pk.y = pack_16x2(acc.z, acc.w, out_dtype);
    *reinterpret_cast<uint32x2*>(reinterpret_cast<uint16_t*>(out) + idx) = pk;
  }
}

// The RESID reduce of one whole row per workgroup, followed by the LayerNorm of the row it has just completed
// (ReplicatedLayerNorm, layers.py:17-36, of the NEXT layer or of the projection): x += sum of partials + bias, then
// h = scale * (x - mean) * rsqrt(var + 1e-5) + offset in h_dtype.  Saves the LayerNorm launch and its round trip
// through memory between two decode layers.  N <= 4 * RLN_Q * 1024.
constexpr int RLN_Q = 4;
__global__ __launch_bounds__(1024) void splitk_reduce_ln_kernel(const float* __restrict__ work, int splits,
                                                                int64_t split_stride, int N, const float* __restrict__ bias,
                                                                float* __restrict__ x, int64_t ldx,
                                                                const float* __restrict__ ln_scale,
                                                                const float* __restrict__ ln_offset, void* __restrict__ h,
                                                                int64_t ldh, int h_dtype) {
  __shared__ float red[2][16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = blockIdx.x, nq = N / 4;
  floatx4 v[RLN_Q];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < RLN_Q; ++i) {
    const int q = i * 1024 + tid;
    if (q < nq) {
      const int n = q * 4;
      floatx4 acc = *reinterpret_cast<const floatx4*>(work + (int64_t)m * N + n);
      for (int sp = 1; sp < splits; ++sp) {
        const floatx4 p = *reinterpret_cast<const floatx4*>(work + sp * split_stride + (int64_t)m * N + n);
        acc.x += p.x; acc.y += p.y; acc.z += p.z; acc.w += p.w;
      }
      if (bias) {
        const floatx4 b = *reinterpret_cast<const floatx4*>(bias + n);
        acc.x += b.x; acc.y += b.y; acc.z += b.z; acc.w += b.w;
      }
      float* o = x + (int64_t)m * ldx + n;
      const floatx4 old = *reinterpret_cast<const floatx4*>(o);
      // the same two roundings per element as "o[j] += acc.j" of the plain reduce
      acc.x = old.x + acc.x; acc.y = old.y + acc.y; acc.z = old.z + acc.z; acc.w = old.w + acc.w;
      *reinterpret_cast<floatx4*>(o) = acc;
      v[i] = acc;
      sum += (acc.x + acc.y) + (acc.z + acc.w);
    }
  }
  sum = wave_sum(sum);
  if (lane == 0) red[0][wave] = sum;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) tot += red[0][i];
  const float mean = tot / (float)N;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < RLN_Q; ++i) {
    if (i * 1024 + tid < nq) {
      const floatx4 t = v[i] - mean;
      sq += (t.x * t.x + t.y * t.y) + (t.z * t.z + t.w * t.w);
    }
  }
  sq = wave_sum(sq);
  if (lane == 0) red[1][wave] = sq;
  __syncthreads();
  float var = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) var += red[1][i];
  const float inv = rsqrtf(var / (float)N + 1e-5f);
#pragma unroll
  for (int i = 0; i < RLN_Q; ++i) {
    const int q = i * 1024 + tid;
    if (q < nq) {
      const int n = q * 4;
      const floatx4 sc = *reinterpret_cast<const floatx4*>(ln_scale + n);
      const floatx4 of = *reinterpret_cast<const floatx4*>(ln_offset + n);
      const floatx4 y = (sc * inv) * (v[i] - mean) + of;
      if (h_dtype == MTJ_F32) {
        *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(h) + (int64_t)m * ldh + n) = y;
      } else {
        uint32x2 pk;
        pk.x = pack_16x2(y.x, y.y, h_dtype);
        pk.y = pack_16x2(y.z, y.w, h_dtype);
        *reinterpret_cast<uint32x2*>(reinterpret_cast<uint16_t*>(h) + (int64_t)m * ldh + n) = pk;
      }
    }
  }
}

// Second half of the fused logits + cross entropy: merges the per-column-tile statistics of a row.
// loss = log(sum exp(l - max)) - (l[target] - max), correct = (l[target] == max); a target outside [0, N) selects
// nothing (pred = 0), as in xent_kernel.
__global__ __launch_bounds__(256) void xent_merge_kernel(const float* __restrict__ pmax, const float* __restrict__ psum,
                                                         const float* __restrict__ tlogit, const int32_t* __restrict__ target,
                                                         int M, int N, int tiles_n, float* __restrict__ loss,
                                                         uint8_t* __restrict__ correct) {
  const int m = blockIdx.x * blockDim.x + threadIdx.x;
  if (m >= M) return;
  float mx = -INFINITY;
  for (int t = 0; t < tiles_n; ++t) mx = fmaxf(mx, pmax[(int64_t)t * M + m]);
  float sm = 0.f;
  for (int t = 0; t < tiles_n; ++t) sm += __expf(pmax[(int64_t)t * M + m] - mx) * psum[(int64_t)t * M + m];
  const int tg = target[m];
  const float pred = ((uint32_t)tg < (uint32_t)N) ? tlogit[m] - mx : 0.f;
  loss[m] = logf(sm) - pred;
  if (correct) correct[m] = (pred == 0.f) ? 1 : 0;
}

// column-tile width that dispatch_tile will use for this problem
int xent_tile_n(int64_t M, int64_t N, int dtype) {
  if (M > 64 && dtype != MTJ_F32 && ((M + 255) / 256) * ((N + 255) / 256) >= 200) return 256;
  return 128;
}

// how many K ranges a skinny problem is cut into so that its few output tiles still fill the chip
int pick_splits(int64_t M, int64_t N, int64_t K, int dtype) {
  if (N % 4) return 1;
  const int bk = dtype == MTJ_F32 ? 32 : 64;
  const int64_t kt = K / bk;
  int splits = 1;
  if (M <= 64) {          // one row of 32 x 128 or 64 x 128 tiles: up to 16 ranges
    const int64_t tiles = (N + 127) / 128;
    while (splits < 16 && tiles * splits * 2 <= 256 && kt % (splits * 2) == 0 && kt / (splits * 2) >= 4) splits *= 2;
  } else {
    if (dtype != MTJ_F32) {   // 256 x 256 tiles of the direct-to-LDS kernel, one workgroup per CU (a short prompt's out projection)
      const int64_t big = ((M + 255) / 256) * ((N + 255) / 256);
      while (splits < 16 && big * splits * 2 <= 256 && kt % (splits * 2) == 0 && kt / (splits * 2) >= 16) splits *= 2;
      if (big * splits >= 200) return splits;
      splits = 1;
    }
    // 128 x 128 tiles, two workgroups per CU: up to 4 ranges
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    while (splits < 4 && tiles * splits * 2 <= 512 && kt % (splits * 2) == 0 && kt / (splits * 2) >= 16) splits *= 2;
  }
  return splits;
}

int check_common(const void* A, int64_t lda, const void* W, int64_t M, int64_t N, int64_t K, int dtype, const char* who) {
  MTJ_REQUIRE(A && W, MTJ_EINVAL, "%s: null pointer", who);
  MTJ_REQUIRE(mtj_is_dtype(dtype), MTJ_EDTYPE, "%s: dtype %d", who, dtype);
  const int bk = dtype == MTJ_F32 ? 32 : 64;
  const int esz = mtj_elem_size(dtype);
  MTJ_REQUIRE(M > 0 && N > 0 && K > 0 && K % bk == 0 && lda >= K, MTJ_EINVAL,
              "%s: bad shape M=%lld N=%lld K=%lld lda=%lld (K must be a multiple of %d)", who, (long long)M,
              (long long)N, (long long)K, (long long)lda, bk);
  MTJ_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), MTJ_ELIMIT, "%s: dimension too large", who);
  MTJ_REQUIRE(mtj_aligned16(A) && mtj_aligned16(W) && (lda * esz) % 16 == 0, MTJ_EALIGN,
              "%s: A, W and the row stride of A must be 16-byte aligned", who);
  MTJ_REQUIRE(256 * lda * esz < (1ll << 30) && 256 * K * esz < (1ll << 30), MTJ_ELIMIT,
              "%s: a 256-row tile of A or W must span less than 1 GiB", who);
  return MTJ_OK;
}

}  // namespace

namespace {
int dispatch_dtype(const gemm_args& a, int dtype, int epi, hipStream_t s) {
  if (dtype == MTJ_BF16) return dispatch<bf16_t, 64>(a, epi, s);
  if (dtype == MTJ_F16) return dispatch<f16_t, 64>(a, epi, s);
  return dispatch<float, 32>(a, epi, s);
}
}  // namespace

extern "C" int mtj_gemm(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N, int64_t K,
                        int dtype, int epi, void* out, int64_t ldo, int out_dtype, const mtj_inproj* ip, float alpha,
                        void* stream) {
  if (int rc = check_common(A, lda, W, M, N, K, dtype, "mtj_gemm")) return rc;
  gemm_args a{};
  a.A = A; a.lda = lda; a.W = W; a.bias = bias; a.M = (int)M; a.N = (int)N; a.K = (int)K;
  a.out = out; a.ldo = ldo; a.out_dtype = out_dtype; a.alpha = alpha; a.splits = 1;
  if (epi == MTJ_EPI_INPROJ) {
    MTJ_REQUIRE(ip && bias, MTJ_EINVAL, "mtj_gemm: INPROJ needs ip and the fc_in bias");
    a.ip = *ip;
    const int64_t d = (int64_t)ip->n_heads * ip->d_head;
    MTJ_REQUIRE(ip->Tp > 0 && M % ip->Tp == 0 && N > 3 * d && N % 32 == 0 && d % 32 == 0 && ip->d_head % 32 == 0 &&
                    ip->rotary_dims % 16 == 0 && ip->ld_act % 16 == 0 &&
                    ip->rotary_dims <= ip->d_head && ip->Tcap > 0 && ip->max_pos > 0 && ip->pos0 && ip->sin_tab &&
                    ip->cos_tab && ip->q && ip->k_cache && ip->v_cache && ip->act && ip->ld_act >= N - 2 * d &&
                    mtj_is_dtype(ip->act_dtype) && mtj_is_dtype(ip->q_dtype) && mtj_is_dtype(ip->kv_dtype) &&
                    (!ip->v_t || ip->ldvt >= ip->Tp),
                MTJ_EINVAL, "mtj_gemm: inconsistent INPROJ geometry");
    MTJ_REQUIRE(mtj_aligned16(bias) && mtj_aligned16(ip->sin_tab) && mtj_aligned16(ip->cos_tab), MTJ_EALIGN,
                "mtj_gemm: the fc_in bias and the rotary tables must be 16-byte aligned");
  } else if (epi == MTJ_EPI_STORE) {
    MTJ_REQUIRE(out && ldo >= N && mtj_is_dtype(out_dtype), MTJ_EINVAL, "mtj_gemm: STORE needs out with ldo >= N");
  } else if (epi == MTJ_EPI_RESID) {
    MTJ_REQUIRE(out && ldo >= N, MTJ_EINVAL, "mtj_gemm: RESID needs out with ldo >= N");
  } else {
    return mtj_fail(MTJ_EINVAL, "mtj_gemm: epilogue %d", epi);
  }
  return dispatch_dtype(a, dtype, epi, (hipStream_t)stream);
}

extern "C" int64_t mtj_gemm_splitk_work_bytes(int64_t M, int64_t N, int64_t K, int dtype) {
  if (M <= 0 || N <= 0 || K <= 0 || !mtj_is_dtype(dtype)) return 0;
  const int splits = pick_splits(M, N, K, dtype);
  return splits > 1 ? (int64_t)splits * M * N * (int64_t)sizeof(float) : 0;
}

extern "C" int mtj_gemm_splitk(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N,
                               int64_t K, int dtype, int epi, void* out, int64_t ldo, int out_dtype, void* work,
                               int64_t work_bytes, float alpha, void* stream) {
  MTJ_REQUIRE(epi == MTJ_EPI_STORE || epi == MTJ_EPI_RESID, MTJ_EINVAL, "mtj_gemm_splitk: epilogue %d", epi);
  if (int rc = check_common(A, lda, W, M, N, K, dtype, "mtj_gemm_splitk")) return rc;
  const int splits = pick_splits(M, N, K, dtype);
  if (splits == 1) return mtj_gemm(A, lda, W, bias, M, N, K, dtype, epi, out, ldo, out_dtype, nullptr, alpha, stream);
  MTJ_REQUIRE(out && ldo >= N && ldo % 4 == 0 && mtj_aligned16(out) && (!bias || mtj_aligned16(bias)), MTJ_EINVAL,
              "mtj_gemm_splitk: out needs ldo >= N, a multiple of 4, and 16-byte alignment (bias too)");
  MTJ_REQUIRE(epi == MTJ_EPI_RESID || mtj_is_dtype(out_dtype), MTJ_EDTYPE, "mtj_gemm_splitk: out_dtype %d", out_dtype);
  MTJ_REQUIRE(work && mtj_aligned16(work) && work_bytes >= (int64_t)splits * M * N * (int64_t)sizeof(float), MTJ_EINVAL,
              "mtj_gemm_splitk: work must hold mtj_gemm_splitk_work_bytes() bytes");
  gemm_args a{};
  a.A = A; a.lda = lda; a.W = W; a.bias = nullptr; a.M = (int)M; a.N = (int)N; a.K = (int)K;
  a.out = work; a.ldo = N; a.out_dtype = MTJ_F32; a.alpha = alpha;
  a.splits = splits; a.split_stride = M * N;
  hipStream_t s = (hipStream_t)stream;
  if (int rc = dispatch_dtype(a, dtype, MTJ_EPI_STORE, s)) return rc;
  const int64_t quads = M * (N / 4);
  const unsigned grid = (unsigned)((quads + 255) / 256);
  if (epi == MTJ_EPI_RESID)
    splitk_reduce_kernel<MTJ_EPI_RESID><<<grid, 256, 0, s>>>((const float*)work, splits, M * N, (int)M, (int)N, bias, out, ldo, MTJ_F32);
  else
    splitk_reduce_kernel<MTJ_EPI_STORE><<<grid, 256, 0, s>>>((const float*)work, splits, M * N, (int)M, (int)N, bias, out, ldo, out_dtype);
  return mtj_check_launch("mtj_gemm_splitk");
}

extern "C" int mtj_gemm_splitk_ln(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N,
                                  int64_t K, int dtype, float* x, int64_t ldx, void* work, int64_t work_bytes,
                                  const float* ln_scale, const float* ln_offset, void* h, int64_t ldh, int h_dtype,
                                  float alpha, void* stream) {
  MTJ_REQUIRE(ln_scale && ln_offset && h && x, MTJ_EINVAL, "mtj_gemm_splitk_ln: null pointer");
  MTJ_REQUIRE(mtj_is_dtype(h_dtype), MTJ_EDTYPE, "mtj_gemm_splitk_ln: h_dtype %d", h_dtype);
  MTJ_REQUIRE(N % 4 == 0 && N <= 4 * RLN_Q * 1024 && ldh >= N && ldh % 4 == 0 && ldx >= N && ldx % 4 == 0 &&
                  mtj_aligned16(x) && mtj_aligned16(h) && mtj_aligned16(ln_scale) && mtj_aligned16(ln_offset) &&
                  (!bias || mtj_aligned16(bias)),
              MTJ_EINVAL, "mtj_gemm_splitk_ln: N a multiple of 4 and <= %d, rows of x and h 16-byte aligned", 4 * RLN_Q * 1024);
  if (int rc = check_common(A, lda, W, M, N, K, dtype, "mtj_gemm_splitk_ln")) return rc;
  const int splits = pick_splits(M, N, K, dtype);
  hipStream_t s = (hipStream_t)stream;
  if (splits == 1) {      // no partials to reduce: the product with its own residual epilogue, then the plain LayerNorm
    MTJ_REQUIRE(ldx == N && ldh == N, MTJ_EINVAL, "mtj_gemm_splitk_ln: without a split, x and h must be dense");
    if (int rc = mtj_gemm(A, lda, W, bias, M, N, K, dtype, MTJ_EPI_RESID, x, ldx, MTJ_F32, nullptr, alpha, stream)) return rc;
    return mtj_layernorm(x, ln_scale, ln_offset, M, N, h, h_dtype, stream);
  }
  MTJ_REQUIRE(work && mtj_aligned16(work) && work_bytes >= (int64_t)splits * M * N * (int64_t)sizeof(float), MTJ_EINVAL,
              "mtj_gemm_splitk_ln: work must hold mtj_gemm_splitk_work_bytes() bytes");
  gemm_args a{};
  a.A = A; a.lda = lda; a.W = W; a.bias = nullptr; a.M = (int)M; a.N = (int)N; a.K = (int)K;
  a.out = work; a.ldo = N; a.out_dtype = MTJ_F32; a.alpha = alpha;
  a.splits = splits; a.split_stride = M * N;
  if (int rc = dispatch_dtype(a, dtype, MTJ_EPI_STORE, s)) return rc;
  splitk_reduce_ln_kernel<<<(unsigned)M, 1024, 0, s>>>((const float*)work, splits, M * N, (int)N, bias, x, ldx, ln_scale,
                                                       ln_offset, h, ldh, h_dtype);
  return mtj_check_launch("mtj_gemm_splitk_ln");
}

extern "C" int64_t mtj_gemm_xent_work_bytes(int64_t M, int64_t N, int dtype) {
  if (M <= 0 || N <= 0 || !mtj_is_dtype(dtype)) return 0;
  const int64_t tiles_n = (N + xent_tile_n(M, N, dtype) - 1) / xent_tile_n(M, N, dtype);
  return (2 * tiles_n + 1) * M * (int64_t)sizeof(float);
}

extern "C" int mtj_gemm_xent(const void* A, int64_t lda, const void* W, const float* bias, int64_t M, int64_t N, int64_t K,
                             int dtype, float alpha, const int32_t* target, float* loss, uint8_t* correct, void* work,
                             int64_t work_bytes, void* stream) {
  if (int rc = check_common(A, lda, W, M, N, K, dtype, "mtj_gemm_xent")) return rc;
  MTJ_REQUIRE(target && loss && work, MTJ_EINVAL, "mtj_gemm_xent: null pointer");
  MTJ_REQUIRE(mtj_aligned16(work) && work_bytes >= mtj_gemm_xent_work_bytes(M, N, dtype), MTJ_EINVAL,
              "mtj_gemm_xent: work must hold mtj_gemm_xent_work_bytes() bytes");
  const int bn = xent_tile_n(M, N, dtype);
  const int64_t tiles_n = (N + bn - 1) / bn;
  gemm_args a{};
  a.A = A; a.lda = lda; a.W = W; a.bias = bias; a.M = (int)M; a.N = (int)N; a.K = (int)K;
  a.alpha = alpha; a.splits = 1;
  a.target = target;
  a.pmax = reinterpret_cast<float*>(work);
  a.psum = a.pmax + tiles_n * M;
  a.tlogit = a.psum + tiles_n * M;
  hipStream_t s = (hipStream_t)stream;
  if (int rc = dispatch_dtype(a, dtype, MTJ_EPI_XENT, s)) return rc;
  xent_merge_kernel<<<(unsigned)((M + 255) / 256), 256, 0, s>>>(a.pmax, a.psum, a.tlogit, target, (int)M, (int)N, (int)tiles_n,
                                                              loss, correct);
  return mtj_check_launch("mtj_gemm_xent");
}

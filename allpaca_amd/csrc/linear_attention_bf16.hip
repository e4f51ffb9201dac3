// Linear attention with a decay (see plain_recurrent.hip for the formulas) for bfloat16 rows on MFMA, a segment's rows
// in chunks of 64.  With S0 the state in front of a chunk, lam the head's decay, rows t, s = 0 .. n-1 of the chunk:
//   A[t][s] = (q_t . k_s) lam^(t-s) for s <= t                      (scores and decay in float32)
//   o_t     = lam^(t+1) S0^T q_t + sum_s A[t][s] v_s
//   S       = lam^n S0 + sum_s (lam^(n-1-s) k_s) v_s^T
// A block takes one segment x one head x 64 value columns and walks the chunks in order; the state's tile stays in
// the accumulators of the last product (float32) from chunk to chunk.  q, k and v are bfloat16 (through silu if asked,
// rounded once); everything that is float32 in the formulas and has to be an MFMA operand (S0, the decayed keys, A)
// goes in as two bfloat16 pieces, value = hi + lo, so that a product keeps 16 bits of it and not 8.
// All products are transposed (keys or value columns as the rows of a tile) so that a lane holds 4 consecutive
// elements of what it stores.
#include "mfma.h"
#include <math.h>

namespace {

constexpr int C = 64;      // rows of a chunk
constexpr int VT = 64;     // value columns of a block
constexpr int PAD = 8;
constexpr int SR = C + PAD;

__device__ __forceinline__ void unpack8f(const Frag& f, float* v) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    v[2 * w] = __uint_as_float(f.w[w] << 16);
    v[2 * w + 1] = __uint_as_float(f.w[w] & 0xffff0000u);
  }
}
__device__ __forceinline__ float round_bf16(float v) { return bf16_to_float(float_to_bf16(v)); }

// four consecutive float32 as two bfloat16 pieces each: hi to `ph`, lo to `pl`
__device__ __forceinline__ void store_split4(bf16_t* ph, bf16_t* pl, float a, float b, float c, float d) {
  uint2 hi, lo;
  hi.x = pack_bf16x2(a, b);
  hi.y = pack_bf16x2(c, d);
  const float ha = __uint_as_float(hi.x << 16), hb = __uint_as_float(hi.x & 0xffff0000u);
  const float hc = __uint_as_float(hi.y << 16), hd = __uint_as_float(hi.y & 0xffff0000u);
  lo.x = pack_bf16x2(a - ha, b - hb);
  lo.y = pack_bf16x2(c - hc, d - hd);
  *reinterpret_cast<uint2*>(ph) = hi;
  *reinterpret_cast<uint2*>(pl) = lo;
}

template <int DKP>  // key size rounded up to a multiple of 64
__global__ __launch_bounds__(256) void linear_attention_chunk_kernel(
    const bf16_t* __restrict__ proj, int ld, int q_off, int k_off, int v_off, int H, int dk, int dv, int act,
    const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ seg_row0,
    const int* __restrict__ seg_rows, const int* __restrict__ slots, float* __restrict__ out, int ldo) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  constexpr int QR = DKP + PAD;
  constexpr int IT = DKP / 64;               // tiles of 16 state rows a wave owns
  bf16_t* Qs = reinterpret_cast<bf16_t*>(lds);   // [C][QR]   q of the chunk's rows
  bf16_t* Ks = Qs + C * QR;                      // [C][QR]   k
  bf16_t* Vt = Ks + C * QR;                      // [VT][SR]  v, a column's rows side by side
  bf16_t* KtH = Vt + VT * SR;                    // [DKP][SR] decayed k, a key element's rows side by side (hi, lo)
  bf16_t* KtL = KtH + DKP * SR;
  bf16_t* AsH = KtL + DKP * SR;                  // [C][SR]   A[t][s] (hi, lo)
  bf16_t* AsL = AsH + C * SR;
  bf16_t* StH = AsL + C * SR;                    // [VT][QR]  the state in front of the chunk, S0[i][j] at [j][i]
  bf16_t* StL = StH + VT * QR;
  float* pw = reinterpret_cast<float*>(StL + VT * QR);   // [C + 1] powers of the decay

  const int seg = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * VT;
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int li = lane % 16, lc = lane / 16;
  const int r0 = seg_row0[seg], n = seg_rows[seg];
  float* S = state + (((size_t)slots[seg] * H + h) * dk) * dv;
  const double lam = (double)decay[h];

  {
    uint32_t* z = reinterpret_cast<uint32_t*>(lds);
    const int words = (int)((reinterpret_cast<unsigned char*>(pw) - lds) / 4);
    for (int i = tid; i < words; i += 256) z[i] = 0u;
  }
  if (tid <= C) pw[tid] = (float)pow(lam, (double)tid);

  floatx4 sreg[IT][4];   // element r: S[i0 + lc * 4 + r][j0 + jt * 16 + li]
#pragma unroll
  for (int it = 0; it < IT; ++it)
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = (wave * IT + it) * 16 + lc * 4 + r, j = j0 + jt * 16 + li;
        sreg[it][jt][r] = (i < dk && j < dv) ? S[(size_t)i * dv + j] : 0.f;
      }
  __syncthreads();

  for (int c0 = 0; c0 < n; c0 += C) {
    const int nc = min(C, n - c0);
    // ---- the state in front of the chunk, as an operand
#pragma unroll
    for (int it = 0; it < IT; ++it)
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) {
        const int at = (jt * 16 + li) * QR + (wave * IT + it) * 16 + lc * 4;
        store_split4(StH + at, StL + at, sreg[it][jt][0], sreg[it][jt][1], sreg[it][jt][2], sreg[it][jt][3]);
      }
    // ---- the chunk's q, k, v
    for (int idx = tid; idx < C * (DKP / 8); idx += 256) {
      const int s = idx % C, e = (idx / C) * 8;
      float qv[8], kv[8];
#pragma unroll
      for (int x = 0; x < 8; ++x) qv[x] = kv[x] = 0.f;
      if (s < nc && e < dk) {
        const bf16_t* row = proj + (size_t)(r0 + c0 + s) * ld + (size_t)h * dk + e;
        unpack8f(load_frag(row + q_off), qv);
        unpack8f(load_frag(row + k_off), kv);
        if (act) {
#pragma unroll
          for (int x = 0; x < 8; ++x) { qv[x] = silu_f(qv[x]); kv[x] = silu_f(kv[x]); }
        }
      }
      Frag fq, fk;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        fq.w[w] = pack_bf16x2(qv[2 * w], qv[2 * w + 1]);
        fk.w[w] = pack_bf16x2(kv[2 * w], kv[2 * w + 1]);
      }
      *reinterpret_cast<Frag*>(Qs + s * QR + e) = fq;
      *reinterpret_cast<Frag*>(Ks + s * QR + e) = fk;
      const float d = s < nc ? pw[nc - 1 - s] : 0.f;
      float kr[8];
      unpack8f(fk, kr);                       // the rounded keys, as the scores see them
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const float kd = kr[x] * d;
        const bf16_t hi = float_to_bf16(kd);
        KtH[(e + x) * SR + s] = hi;
        KtL[(e + x) * SR + s] = float_to_bf16(kd - bf16_to_float(hi));
      }
    }
    for (int idx = tid; idx < C * (VT / 8); idx += 256) {
      const int s = idx % C, e = (idx / C) * 8;
      float vv[8];
#pragma unroll
      for (int x = 0; x < 8; ++x) vv[x] = 0.f;
      if (s < nc && j0 + e < dv) {
        unpack8f(load_frag(proj + (size_t)(r0 + c0 + s) * ld + v_off + (size_t)h * dv + j0 + e), vv);
        if (act) {
#pragma unroll
          for (int x = 0; x < 8; ++x) vv[x] = silu_f(vv[x]);
        }
      }
#pragma unroll
      for (int x = 0; x < 8; ++x) Vt[(e + x) * SR + s] = float_to_bf16(vv[x]);
    }
    __syncthreads();

    // ---- scores of the wave's 16 rows t with all 64 rows s, transposed: tile rows s, columns t
    const int t = wave * 16 + li;              // the lane's row of the chunk as a column of the tiles
    Frag qf[DKP / 32];
#pragma unroll
    for (int ks = 0; ks < DKP / 32; ++ks) qf[ks] = *reinterpret_cast<const Frag*>(Qs + t * QR + ks * 32 + lc * 8);
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
      if (st <= wave) {                        // (tiles of later rows s hold nothing the rows t see)
#pragma unroll
        for (int ks = 0; ks < DKP / 32; ++ks) {
          const Frag kf = *reinterpret_cast<const Frag*>(Ks + (st * 16 + li) * QR + ks * 32 + lc * 8);
          acc = mfma16(kf, qf[ks], acc);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int s = st * 16 + lc * 4 + r;
          acc[r] = s <= t ? acc[r] * pw[t - s] : 0.f;
        }
      }
      const int at = t * SR + st * 16 + lc * 4;
      store_split4(AsH + at, AsL + at, acc[0], acc[1], acc[2], acc[3]);
    }
    wave_lds_order();

    // ---- outputs of the wave's rows, transposed: tile rows value columns j, columns t
    const float from_state = pw[min(t, C - 1) + 1];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) {
      floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DKP / 32; ++ks) {
        const int at = (jt * 16 + li) * QR + ks * 32 + lc * 8;
        acc = mfma16(*reinterpret_cast<const Frag*>(StH + at), qf[ks], acc);
        acc = mfma16(*reinterpret_cast<const Frag*>(StL + at), qf[ks], acc);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] *= from_state;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        if (kk * 32 > wave * 16 + 15) continue;
        const Frag vf = *reinterpret_cast<const Frag*>(Vt + (jt * 16 + li) * SR + kk * 32 + lc * 8);
        const int at = t * SR + kk * 32 + lc * 8;
        acc = mfma16(vf, *reinterpret_cast<const Frag*>(AsH + at), acc);
        acc = mfma16(vf, *reinterpret_cast<const Frag*>(AsL + at), acc);
      }
      const int j = j0 + jt * 16 + lc * 4;
      if (t < nc && j < dv)
        *reinterpret_cast<float4*>(out + (size_t)(r0 + c0 + t) * ldo + (size_t)h * dv + j) =
            float4{acc[0], acc[1], acc[2], acc[3]};
    }

    // ---- the state behind the chunk: tile rows key elements i (the wave's own), columns j
    const float keep = pw[nc];
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int i = (wave * IT + it) * 16 + li;
      Frag kh[2], kl[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        kh[kk] = *reinterpret_cast<const Frag*>(KtH + i * SR + kk * 32 + lc * 8);
        kl[kk] = *reinterpret_cast<const Frag*>(KtL + i * SR + kk * 32 + lc * 8);
      }
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) {
#pragma unroll
        for (int r = 0; r < 4; ++r) sreg[it][jt][r] *= keep;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const Frag vf = *reinterpret_cast<const Frag*>(Vt + (jt * 16 + li) * SR + kk * 32 + lc * 8);
          sreg[it][jt] = mfma16(kh[kk], vf, sreg[it][jt]);
          sreg[it][jt] = mfma16(kl[kk], vf, sreg[it][jt]);
        }
      }
    }
    __syncthreads();     // every wave has read this chunk's operands before the next chunk's are written
  }

#pragma unroll
  for (int it = 0; it < IT; ++it)
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = (wave * IT + it) * 16 + lc * 4 + r, j = j0 + jt * 16 + li;
        if (i < dk && j < dv) S[(size_t)i * dv + j] = sreg[it][jt][r];
      }
}

template <int DKP>
constexpr size_t lds_bytes() {
  return (size_t)(2 * C * (DKP + PAD) + VT * SR + 2 * DKP * SR + 2 * C * SR + 2 * VT * (DKP + PAD)) * 2 + (C + 1) * 4;
}

}  // namespace

// 1 if the kernel takes these sizes, else 0 (the caller then runs the plain kernel)
APC_EXPORT int apc_linear_attention_bf16_takes(int ld, int q_off, int k_off, int v_off, int H, int dk, int dv) {
  if (H <= 0 || dk <= 0 || dv <= 0 || dk > 128 || dk % 8 || dv % 8 || ld % 8 || q_off % 8 || k_off % 8 || v_off % 8) return 0;
  return 1;
}

APC_EXPORT int apc_linear_attention_bf16(const void* proj, int ld, int q_off, int k_off, int v_off, int H, int dk,
                                         int dv, int act, const float* decay, float* state, int n_segs,
                                         const int* seg_row0, const int* seg_rows, const int* slots, float* out,
                                         int ldo, hipStream_t stream) {
  if (n_segs <= 0) return 0;
  if (!apc_linear_attention_bf16_takes(ld, q_off, k_off, v_off, H, dk, dv)) return APC_ERR_UNSUPPORTED;
  if (!decay || !state || !slots || ldo < H * dv || ldo % 4 || ((uintptr_t)proj & 15u) || ((uintptr_t)out & 15u))
    return APC_ERR_BAD_ARG;
  dim3 grid(n_segs, H, ceil_div(dv, VT));
  if (H > 65535 || grid.z > 65535) return APC_ERR_UNSUPPORTED;
#define LAC_LAUNCH(DKP_)                                                                                            \
  do {                                                                                                              \
    static bool set_##DKP_ = false;                                                                                 \
    if (!set_##DKP_) {                                                                                              \
      hipError_t e_ = hipFuncSetAttribute(reinterpret_cast<const void*>(&linear_attention_chunk_kernel<DKP_>),      \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes<DKP_>());      \
      if (e_ != hipSuccess) return (int)e_;                                                                         \
      set_##DKP_ = true;                                                                                            \
    }                                                                                                               \
    hipLaunchKernelGGL(linear_attention_chunk_kernel<DKP_>, grid, dim3(256), lds_bytes<DKP_>(), stream,             \
                       (const bf16_t*)proj, ld, q_off, k_off, v_off, H, dk, dv, act, decay, state, seg_row0,        \
                       seg_rows, slots, out, ldo);                                                                  \
  } while (0)
  if (dk <= 64) LAC_LAUNCH(64);
  else LAC_LAUNCH(128);
#undef LAC_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

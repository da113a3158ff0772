// Decode-step kernels around the quantized linears (HBM-bound, one launch each per layer):
//   e2h_decode_attention   single-query attention over the bf16 KV cache, reading only the live positions
//   e2h_rmsnorm            RMSNorm with the reference's rounding points
//   e2h_rope_kv_write      rotary embedding of q and k + write of k, v into the cache at input_pos
//   e2h_silu_mul           silu(a) * b
// They restate, for one new token per sequence, what the reference's model code does with stock ops
// (models/model.py: KVCache.update :121-129, Attention.forward :310-349, RMSNorm :363-377, apply_rotary_emb
// :400-412, FeedForward.forward :359-360; decode loop inference_generate.py:110-157).
#include "e2h_common.h"
#include "e2h_staged.h"

namespace e2h {
namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

// ------------------------------------------------------------------------------------------------
// decode attention: q [B, H, D], caches [Bmax, Hkv, S, D] bf16, out [B, H, D] bf16.
// One workgroup (NW = 4 or 8 waves) per (b, kv head); the waves split the live positions, every wave keeps REP query heads
// (the heads that share the kv head) so that each K / V row is loaded once.  Lane layout: LPP = D/8 lanes cover
// one position (16 bytes each), a wave-wide load covers 64/LPP positions.  Online softmax in float32.
// Visible positions: t <= pos, and if left_pad is given additionally (t >= left_pad[b] or t == pos)
// (reference models/model.py:221-228).
// ------------------------------------------------------------------------------------------------
template <int D, int REP, int NW>
__global__ __launch_bounds__(64 * NW) void decode_attention_kernel(const uint16_t *__restrict__ q, const uint16_t *__restrict__ kc,
                                                               const uint16_t *__restrict__ vc, uint16_t *__restrict__ out,
                                                               const int64_t *__restrict__ input_pos, const int64_t *__restrict__ left_pad,
                                                               int H, int Hkv, int S, float scale, StagedOut staged) {
  constexpr int LPP = D / 8;        // lanes per position
  constexpr int PPL = 64 / LPP;     // positions per wave-wide load
  constexpr int UNR = 4;            // loads in flight per wave
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int dg = lane % LPP;        // which 8 values of the head dimension
  const int pg = lane / LPP;        // which position within a load
  const int b = blockIdx.x / Hkv, hk = blockIdx.x % Hkv;
  const int pos = static_cast<int>(input_pos[0]);
  const int first = left_pad ? static_cast<int>(left_pad[b]) : 0;
  const int n_live = pos + 1 < S ? pos + 1 : S;  // never past the cache, whatever the position tensor holds

  float qf[REP][8];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(q + (static_cast<size_t>(b) * H + hk * REP + r) * D + dg * 8);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      qf[r][2 * i] = __builtin_bit_cast(float, raw[i] << 16) * scale;
      qf[r][2 * i + 1] = __builtin_bit_cast(float, raw[i] & 0xFFFF0000u) * scale;
    }
  }
  const size_t head_base = (static_cast<size_t>(b) * Hkv + hk) * S * D;
  const uint16_t *kbase = kc + head_base + dg * 8;
  const uint16_t *vbase = vc + head_base + dg * 8;

  float m_run[REP], l_run[REP], acc[REP][8];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    m_run[r] = -1e30f;
    l_run[r] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[r][i] = 0.f;
  }

  // waves take interleaved tiles of UNR * PPL positions; the rows of a wave's next tile are requested before the
  // current tile is worked on, so a wave has two tiles in flight instead of one HBM round trip per tile
  auto fetch = [&](int t0, u32x4_t (&kr)[UNR], u32x4_t (&vr)[UNR]) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int tp = t0 + u * PPL + pg;
      const int tc = tp < n_live ? tp : n_live - 1;
      // streaming loads: a cache row is read once per step, and with the default policy the same kernel runs 10 % slower
      kr[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(kbase + static_cast<size_t>(tc) * D));
      vr[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(vbase + static_cast<size_t>(tc) * D));
    }
  };
  u32x4_t kr[UNR], vr[UNR], kn[UNR], vn[UNR];
  if (wave * (UNR * PPL) < n_live) fetch(wave * (UNR * PPL), kr, vr);
  for (int t0 = wave * (UNR * PPL); t0 < n_live; t0 += NW * UNR * PPL) {
    const bool more = t0 + NW * UNR * PPL < n_live;
    if (more) fetch(t0 + NW * UNR * PPL, kn, vn);
    int tpos[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) tpos[u] = t0 + u * PPL + pg;
    float s[REP][UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      float kf[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        kf[2 * i] = __builtin_bit_cast(float, kr[u][i] << 16);
        kf[2 * i + 1] = __builtin_bit_cast(float, kr[u][i] & 0xFFFF0000u);
      }
      const bool visible = tpos[u] < n_live && (tpos[u] >= first || tpos[u] == pos);
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        float d = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) d = __builtin_fmaf(qf[r][i], kf[i], d);
#pragma unroll
        for (int off = 1; off < LPP; off <<= 1) d += __shfl_xor(d, off);
        s[r][u] = visible ? d : -1e30f;
      }
    }
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      float mx = s[r][0];
#pragma unroll
      for (int u = 1; u < UNR; ++u) mx = fmaxf(mx, s[r][u]);
#pragma unroll
      for (int off = LPP; off < 64; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
      const float m_new = fmaxf(m_run[r], mx);
      const float corr = __expf(m_run[r] - m_new);
      m_run[r] = m_new;
      l_run[r] *= corr;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[r][i] *= corr;
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const float p = s[r][u] > -1e29f ? __expf(s[r][u] - m_new) : 0.f;
        l_run[r] += p;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[r][2 * i] = __builtin_fmaf(p, __builtin_bit_cast(float, vr[u][i] << 16), acc[r][2 * i]);
          acc[r][2 * i + 1] = __builtin_fmaf(p, __builtin_bit_cast(float, vr[u][i] & 0xFFFF0000u), acc[r][2 * i + 1]);
        }
      }
    }
    if (more) {
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        kr[u] = kn[u];
        vr[u] = vn[u];
      }
    }
  }

  // combine the position groups of a wave, then the waves
  __shared__ float sh_m[NW][REP], sh_l[NW][REP], sh_acc[NW][REP][D];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    // l_run counts each position once per lane of its group (every lane of the group holds the same p): sum over groups
    float l = l_run[r];
#pragma unroll
    for (int off = LPP; off < 64; off <<= 1) l += __shfl_xor(l, off);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float a = acc[r][i];
#pragma unroll
      for (int off = LPP; off < 64; off <<= 1) a += __shfl_xor(a, off);
      acc[r][i] = a;
    }
    if (pg == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) sh_acc[wave][r][dg * 8 + i] = acc[r][i];
      if (dg == 0) {
        sh_m[wave][r] = m_run[r];
        sh_l[wave][r] = l;
      }
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < REP * D; e += 64 * NW) {
    const int r = e / D, d = e % D;
    float m = sh_m[0][r];
#pragma unroll
    for (int w = 1; w < NW; ++w) m = fmaxf(m, sh_m[w][r]);
    float l = 0.f, a = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float c = __expf(sh_m[w][r] - m);
      l += sh_l[w][r] * c;
      a += sh_acc[w][r][d] * c;
    }
    const uint16_t o = f32_to_bf16_rne(a / l);
    if (out) out[(static_cast<size_t>(b) * H + hk * REP + r) * D + d] = o;
    if (staged.frag) staged_store_run16(staged, b, (hk * REP + r) * D + d, o);  // whole aligned 16-lane groups get here together
  }
}

// ------------------------------------------------------------------------------------------------
// decode attention for grouped queries (REP = 4 .. 16 query heads per kv head, head_dim 128) on the matrix cores.
// With several query heads per K / V row the float32 dot products of the kernel above become the bound (8 heads:
// 3.5 x slower than the memory traffic allows), so both products go through v_mfma_f32_16x16x32_bf16:
//   S [heads x positions] = Q K^T:  A = Q (rows = heads, padded to 16; 4 steps of 32 over head_dim), B = K^T -- lane
//     (b, c) of a B operand is 16 contiguous bytes of K row `position c`, read straight from the cache;
//   O [heads x head_dim] += P V:    A = P (bfloat16, through a 1 KB wave-private LDS tile that turns the accumulator
//     layout of S into operand layout), B = V -- contracted over positions, so its operand needs 8 consecutive
//     positions of one column: the wave's V tile (32 positions) goes through LDS and is gathered from there.
// One workgroup per (sequence, kv head), waves take tiles of 32 positions round robin, online softmax in float32 on
// the accumulator layout (lane (c, b) holds positions c / heads 4b .. 4b+3 of S, head_dim column c / the same heads of
// O); the softmax scale is applied to S in float32, Q stays exact.  Visibility as above.
// ------------------------------------------------------------------------------------------------
constexpr int kGqaVRow = 264;  // bytes per V row in LDS (256 + 8: rows 8 apart land 16 banks apart)

template <int NW>
__global__ __launch_bounds__(64 * NW) void decode_attention_gqa_kernel(const uint16_t *__restrict__ q, const uint16_t *__restrict__ kc,
                                                                       const uint16_t *__restrict__ vc, uint16_t *__restrict__ out,
                                                                       const int64_t *__restrict__ input_pos,
                                                                       const int64_t *__restrict__ left_pad, int H, int Hkv, int S, int rep,
                                                                       float scale, StagedOut staged) {
  constexpr int D = 128;
  constexpr int kWaveLds = 1024 + 32 * kGqaVRow;                  // P tile + V tile
  constexpr int kLoopLds = NW * kWaveLds;
  constexpr int kEndLds = NW * (16 * D + 32) * 4;                 // per wave: O [16][D], m [16], l [16] as float32
  __shared__ __attribute__((aligned(16))) uint8_t lds[kLoopLds > kEndLds ? kLoopLds : kEndLds];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, b = lane >> 4;
  const int bi = blockIdx.x / Hkv, hk = blockIdx.x % Hkv;
  const int pos = static_cast<int>(input_pos[0]);
  const int first = left_pad ? static_cast<int>(left_pad[bi]) : 0;
  const int n_live = pos + 1 < S ? pos + 1 : S;

  // Q as A operands: lane (b, r) holds Q[head r][32 s + 8 b .. + 7]; rows beyond rep are zero
  bf16x8_t qa[4];
#pragma unroll
  for (int s4 = 0; s4 < 4; ++s4) {
    u32x4_t raw = {0u, 0u, 0u, 0u};
    if (c < rep) raw = *reinterpret_cast<const u32x4_t *>(q + (static_cast<size_t>(bi) * H + hk * rep + c) * D + 32 * s4 + 8 * b);
    qa[s4] = __builtin_bit_cast(bf16x8_t, raw);
  }
  const size_t head_base = (static_cast<size_t>(bi) * Hkv + hk) * S * D;
  const uint16_t *kbase = kc + head_base + 8 * b;  // + position * D + 32 s
  const uint16_t *vbase = vc + head_base;
  uint8_t *const p_lds = lds + wave * kWaveLds;
  uint8_t *const v_lds = p_lds + 1024;

  float m_run[4], l_part[4];
  f32x4_t oacc[8];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m_run[r] = -1e30f;
    l_part[r] = 0.f;
  }
#pragma unroll
  for (int nt = 0; nt < 8; ++nt) oacc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  for (int t0 = wave * 32; t0 < n_live; t0 += NW * 32) {
    // K operands of the two 16-position halves and this lane's share of the V tile (eight 16-byte pieces: piece
    // lane % 16 of rows lane / 16 + 4 i), all requested before anything is waited for.  The V loads cover whole rows per
    // instruction and stream (8 % less time than with the default policy); a K row is covered by four instructions in
    // operand order, and streamed that way the pieces of a line are fetched again and again (1.7 x the time), so the K
    // loads keep the default policy.
    u32x4_t kf[2][4], vr[8];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int tp = t0 + 16 * j + c;
      const int tc = tp < n_live ? tp : n_live - 1;
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) kf[j][s4] = *reinterpret_cast<const u32x4_t *>(kbase + static_cast<size_t>(tc) * D + 32 * s4);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {  // instruction i: rows 4 i .. 4 i + 3 of the tile, sixteen lanes per 256-byte row
      const int tp = t0 + 4 * i + (lane >> 4);
      const int tc = tp < n_live ? tp : n_live - 1;
      vr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(vbase + static_cast<size_t>(tc) * D + 8 * (lane & 15)));
    }
    // S = Q K^T for 32 positions
    f32x4_t sacc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      sacc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4)
        sacc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[s4], __builtin_bit_cast(bf16x8_t, kf[j][s4]), sacc[j], 0, 0, 0);
    }
    // the V tile goes to LDS while the softmax is worked out
    {
      uint8_t *dst = v_lds + (lane >> 4) * kGqaVRow + 16 * (lane & 15);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        *reinterpret_cast<u32x2_t *>(dst + 4 * i * kGqaVRow) = u32x2_t{vr[i][0], vr[i][1]};
        *reinterpret_cast<u32x2_t *>(dst + 4 * i * kGqaVRow + 8) = u32x2_t{vr[i][2], vr[i][3]};
      }
    }
    float pv[2][4], corr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float sv[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int tp = t0 + 16 * j + c;
        const bool visible = tp < n_live && (tp >= first || tp == pos);
        sv[j] = visible ? sacc[j][r] * scale : -1e30f;
      }
      float mx = fmaxf(sv[0], sv[1]);
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off));  // over the 16 positions of this head's lanes
      const float m_new = fmaxf(m_run[r], mx);
      corr[r] = __expf(m_run[r] - m_new);
      m_run[r] = m_new;
#pragma unroll
      for (int j = 0; j < 2; ++j) pv[j][r] = sv[j] > -1e29f ? __expf(sv[j] - m_new) : 0.f;
      l_part[r] = l_part[r] * corr[r] + pv[0][r] + pv[1][r];
    }
    // P (bfloat16) -> LDS [head][position], then back as the A operand: lane (b, r) = head r, positions 8b .. 8b+7
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) *reinterpret_cast<uint16_t *>(p_lds + (4 * b + r) * 64 + (16 * j + c) * 2) = f32_to_bf16_rne(pv[j][r]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // wave-private tiles: the wave's own writes have landed
    const bf16x8_t pa = *reinterpret_cast<const bf16x8_t *>(p_lds + c * 64 + b * 16);
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) {
      // V operand of column tile nt: lane (b, c) = positions 8b .. 8b+7 of column 16 nt + c
      uint32_t vw[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lo = *reinterpret_cast<const uint16_t *>(v_lds + (8 * b + 2 * i) * kGqaVRow + (16 * nt + c) * 2);
        const uint32_t hi = *reinterpret_cast<const uint16_t *>(v_lds + (8 * b + 2 * i + 1) * kGqaVRow + (16 * nt + c) * 2);
        vw[i] = lo | (hi << 16);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) oacc[nt][r] *= corr[r];
      oacc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, __builtin_bit_cast(bf16x8_t, u32x4_t{vw[0], vw[1], vw[2], vw[3]}), oacc[nt], 0, 0, 0);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // reads done before the next tile overwrites the wave's LDS
  }

  // combine: sum l over the 16 position lanes of each head, then the waves through LDS
  __syncthreads();  // every wave is done with its loop tiles: the LDS is reused
  float *const sh_o = reinterpret_cast<float *>(lds);                 // [NW][16][D]
  float *const sh_m = sh_o + NW * 16 * D;                             // [NW][16]
  float *const sh_l = sh_m + NW * 16;                                 // [NW][16]
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float l = l_part[r];
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) l += __shfl_xor(l, off);
    const int head = 4 * b + r;
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) sh_o[(wave * 16 + head) * D + 16 * nt + c] = oacc[nt][r];
    if (c == 0) {
      sh_m[wave * 16 + head] = m_run[r];
      sh_l[wave * 16 + head] = l;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < rep * D; e += 64 * NW) {
    const int r = e / D, d = e % D;
    float m = sh_m[r];
#pragma unroll
    for (int w = 1; w < NW; ++w) m = fmaxf(m, sh_m[w * 16 + r]);
    float l = 0.f, a = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float cw = __expf(sh_m[w * 16 + r] - m);
      l += sh_l[w * 16 + r] * cw;
      a += sh_o[(w * 16 + r) * D + d] * cw;
    }
    const uint16_t o = f32_to_bf16_rne(a / l);
    if (out) out[(static_cast<size_t>(bi) * H + hk * rep + r) * D + d] = o;
    if (staged.frag) staged_store_run16(staged, bi, (hk * rep + r) * D + d, o);  // whole aligned 16-lane groups get here together
  }
}

// ------------------------------------------------------------------------------------------------
// RMSNorm (reference :363-377): bf16(bf16(x * rsqrt(mean(x^2) + eps)) * w), float32 statistics.
// ------------------------------------------------------------------------------------------------
// One workgroup of BLOCK threads per row.  With `delta` the kernel first forms h = bf16(x + delta) (the residual add
// of TransformerBlock.forward, reference :279-282), stores it to h_out and normalises h.  The first kPieces pieces of
// 8 values per thread stay in registers and all their loads are issued before anything is waited for (one memory
// round trip for the whole row up to BLOCK * 8 * kPieces values); longer rows re-read the rest.
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void rmsnorm_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ delta,
                                                        const float *__restrict__ psum, int slices,
                                                        const uint16_t *__restrict__ col_scales,
                                                        const uint16_t *__restrict__ w, uint16_t *__restrict__ h_out,
                                                        uint16_t *__restrict__ y, StagedOut staged, int dim, float eps) {
  constexpr int kPieces = 2, kStride = BLOCK * 8, kWaves = BLOCK / 64;
  constexpr int kMaxSlices = 4;  // slices whose loads are all issued before the first addition
  const size_t row = blockIdx.x;
  const uint16_t *xr = x + row * dim;
  const uint16_t *dr_row = delta ? delta + row * dim : nullptr;
  // psum: the term to add arrives as float32 partial sums [slices][rows][dim] of a matmul split along K; the term is
  // bf16(p[0] + p[1] + .. in slice order), the value the matmul's own combine step would have stored -- with
  // col_scales (int8 weights) bf16(that * scale[column]), the two roundings of the int8 linear
  const size_t slice_floats = static_cast<size_t>(gridDim.x) * dim;
  const float *pr = psum ? psum + row * dim : nullptr;
  auto sum_slices = [&](int i) {
    f32x4_t lo[kMaxSlices], hi[kMaxSlices];
#pragma unroll
    for (int u = 0; u < kMaxSlices; ++u) {
      const int s2 = u < slices ? u : slices - 1;
      lo[u] = *reinterpret_cast<const f32x4_t *>(pr + s2 * slice_floats + i);
      hi[u] = *reinterpret_cast<const f32x4_t *>(pr + s2 * slice_floats + i + 4);
    }
    f32x4_t a = lo[0], b = hi[0];
#pragma unroll
    for (int u = 1; u < kMaxSlices; ++u)
      if (u < slices) {
        a += lo[u];
        b += hi[u];
      }
    for (int s2 = kMaxSlices; s2 < slices; ++s2) {
      a += *reinterpret_cast<const f32x4_t *>(pr + s2 * slice_floats + i);
      b += *reinterpret_cast<const f32x4_t *>(pr + s2 * slice_floats + i + 4);
    }
    if (col_scales) {
      const u32x4_t cs = *reinterpret_cast<const u32x4_t *>(col_scales + i);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        a[2 * j] = bf16_round(a[2 * j]) * __builtin_bit_cast(float, cs[j] << 16);
        a[2 * j + 1] = bf16_round(a[2 * j + 1]) * __builtin_bit_cast(float, cs[j] & 0xFFFF0000u);
        b[2 * j] = bf16_round(b[2 * j]) * __builtin_bit_cast(float, cs[2 + j] << 16);
        b[2 * j + 1] = bf16_round(b[2 * j + 1]) * __builtin_bit_cast(float, cs[2 + j] & 0xFFFF0000u);
      }
    }
    u32x4_t d;
    d[0] = static_cast<uint32_t>(f32_to_bf16_rne(a[0])) | (static_cast<uint32_t>(f32_to_bf16_rne(a[1])) << 16);
    d[1] = static_cast<uint32_t>(f32_to_bf16_rne(a[2])) | (static_cast<uint32_t>(f32_to_bf16_rne(a[3])) << 16);
    d[2] = static_cast<uint32_t>(f32_to_bf16_rne(b[0])) | (static_cast<uint32_t>(f32_to_bf16_rne(b[1])) << 16);
    d[3] = static_cast<uint32_t>(f32_to_bf16_rne(b[2])) | (static_cast<uint32_t>(f32_to_bf16_rne(b[3])) << 16);
    return d;
  };
  const bool adds = delta || psum;
  auto add_round = [](u32x4_t a, u32x4_t d) {  // bf16(x + delta), value by value
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float lo = __builtin_bit_cast(float, a[j] << 16) + __builtin_bit_cast(float, d[j] << 16);
      const float hi = __builtin_bit_cast(float, a[j] & 0xFFFF0000u) + __builtin_bit_cast(float, d[j] & 0xFFFF0000u);
      a[j] = static_cast<uint32_t>(f32_to_bf16_rne(lo)) | (static_cast<uint32_t>(f32_to_bf16_rne(hi)) << 16);
    }
    return a;
  };
  auto sum_sq = [](u32x4_t a, float ss) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float lo = __builtin_bit_cast(float, a[j] << 16), hi = __builtin_bit_cast(float, a[j] & 0xFFFF0000u);
      ss = __builtin_fmaf(lo, lo, ss);
      ss = __builtin_fmaf(hi, hi, ss);
    }
    return ss;
  };
  // y (row-major, may be null) and / or the staged form the decode-batch int4 kernels read (dim % 16 == 0 then, so the
  // two threads that hold a run of 16 values are neighbouring lanes and take this path together)
  auto scale_store = [&](u32x4_t raw, u32x4_t wr, float inv, int i) {
    u32x4_t o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float lo = bf16_round(__builtin_bit_cast(float, raw[j] << 16) * inv) * __builtin_bit_cast(float, wr[j] << 16);
      const float hi = bf16_round(__builtin_bit_cast(float, raw[j] & 0xFFFF0000u) * inv) * __builtin_bit_cast(float, wr[j] & 0xFFFF0000u);
      o[j] = static_cast<uint32_t>(f32_to_bf16_rne(lo)) | (static_cast<uint32_t>(f32_to_bf16_rne(hi)) << 16);
    }
    if (y) *reinterpret_cast<u32x4_t *>(y + row * dim + i) = o;
    if (staged.frag) staged_store_piece(staged, static_cast<int>(row), i >> 3, o);
  };

  u32x4_t keep[kPieces], keepd[kPieces], keepw[kPieces];
#pragma unroll
  for (int p = 0; p < kPieces; ++p) {
    const int i = threadIdx.x * 8 + p * kStride;
    if (i < dim) {
      keep[p] = *reinterpret_cast<const u32x4_t *>(xr + i);
      if (delta) keepd[p] = *reinterpret_cast<const u32x4_t *>(dr_row + i);
      else if (psum) keepd[p] = sum_slices(i);
      keepw[p] = *reinterpret_cast<const u32x4_t *>(w + i);  // needed only after the reduction
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int p = 0; p < kPieces; ++p) {
    const int i = threadIdx.x * 8 + p * kStride;
    if (i < dim) {
      if (adds) {
        keep[p] = add_round(keep[p], keepd[p]);
        *reinterpret_cast<u32x4_t *>(h_out + row * dim + i) = keep[p];
      }
      ss = sum_sq(keep[p], ss);
    }
  }
  for (int i = threadIdx.x * 8 + kPieces * kStride; i < dim; i += kStride) {
    u32x4_t raw = *reinterpret_cast<const u32x4_t *>(xr + i);
    if (adds) {
      raw = add_round(raw, delta ? *reinterpret_cast<const u32x4_t *>(dr_row + i) : sum_slices(i));
      *reinterpret_cast<u32x4_t *>(h_out + row * dim + i) = raw;
    }
    ss = sum_sq(raw, ss);
  }
  ss = wave_sum(ss);
  __shared__ float part[kWaves];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();  // also makes this thread's own h_out stores visible to its re-reads below
  ss = 0.f;
#pragma unroll
  for (int wv = 0; wv < kWaves; ++wv) ss += part[wv];
  const float inv = rsqrtf(ss / static_cast<float>(dim) + eps);
  const uint16_t *src = adds ? h_out + row * dim : xr;
#pragma unroll
  for (int p = 0; p < kPieces; ++p) {
    const int i = threadIdx.x * 8 + p * kStride;
    if (i < dim) scale_store(keep[p], keepw[p], inv, i);
  }
  for (int i = threadIdx.x * 8 + kPieces * kStride; i < dim; i += kStride)
    scale_store(*reinterpret_cast<const u32x4_t *>(src + i), *reinterpret_cast<const u32x4_t *>(w + i), inv, i);
}

// ------------------------------------------------------------------------------------------------
// RoPE + KV write.  qkv [B * T, (H + 2 Hkv) * D] bf16 (row b * T + t, columns ordered q | k | v), T new tokens per
// sequence at positions input_pos[0 .. T-1]; freqs [>= S, D/2, 2] bf16 (cos, sin).  Writes q_out [B, H, T, D]
// (rotated, head-major as attention wants it) and k (rotated) / v into [B, Hkv, S, D] at the positions.
// Rotation of interleaved pairs in float32, rounded to bf16 (reference :400-412); positions outside [0, S) write
// nothing to the caches.  rows_by_token: k / v row = token index t instead of its position (a pass without KV
// cache, where k and v are fresh tensors of exactly T rows).
// ------------------------------------------------------------------------------------------------
// PAIRS = interleaved pairs per thread: 4 (one 16-byte access per tensor, head_dim % 8 == 0) or 1.
template <int PAIRS>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ freqs,
                                                            uint16_t *__restrict__ q_out, uint16_t *__restrict__ kc, uint16_t *__restrict__ vc,
                                                            const int64_t *__restrict__ input_pos, int B, int T, int H, int Hkv, int S, int D,
                                                            int rows_by_token) {
  typedef uint32_t vec_t __attribute__((ext_vector_type(PAIRS)));
  const int units_per_row = (H + 2 * Hkv) * D / (2 * PAIRS);
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= static_cast<int64_t>(B) * T * units_per_row) return;
  const int row = static_cast<int>(idx / units_per_row), p = static_cast<int>(idx % units_per_row) * PAIRS;  // first pair
  const int b = row / T, t = row % T;
  const int head = (2 * p) / D, dpair = p % (D / 2);
  const int pos = static_cast<int>(input_pos[t]);   // rotation angle
  const int slot = rows_by_token ? t : pos;         // row of the k / v tensors that receives this token
  const bool pos_ok = pos >= 0 && slot >= 0 && slot < S;
  const vec_t raw = reinterpret_cast<const vec_t *>(qkv)[idx];
  if (head < H + Hkv) {
    if (!pos_ok) return;  // no angle for such a position
    const vec_t f = *reinterpret_cast<const vec_t *>(reinterpret_cast<const uint32_t *>(freqs) + static_cast<size_t>(pos) * (D / 2) + dpair);
    vec_t o;
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
      const uint32_t ri = raw[i], fi = f[i];
      const float x0 = __builtin_bit_cast(float, ri << 16), x1 = __builtin_bit_cast(float, ri & 0xFFFF0000u);
      const float cs = __builtin_bit_cast(float, fi << 16), sn = __builtin_bit_cast(float, fi & 0xFFFF0000u);
      // two separately rounded products and their difference / sum, as torch evaluates the expression in float32
      const float r0 = x0 * cs - x1 * sn;
      const float r1 = x1 * cs + x0 * sn;
      const uint32_t oi = static_cast<uint32_t>(f32_to_bf16_rne(r0)) | (static_cast<uint32_t>(f32_to_bf16_rne(r1)) << 16);
      o[i] = oi;
    }
    if (head < H) {
      *reinterpret_cast<vec_t *>(reinterpret_cast<uint32_t *>(q_out) + ((static_cast<size_t>(b) * H + head) * T + t) * (D / 2) + dpair) = o;
    } else {
      const int hk = head - H;
      *reinterpret_cast<vec_t *>(reinterpret_cast<uint32_t *>(kc) + ((static_cast<size_t>(b) * Hkv + hk) * S + slot) * (D / 2) + dpair) = o;
    }
  } else if (pos_ok) {
    const int hk = head - H - Hkv;
    *reinterpret_cast<vec_t *>(reinterpret_cast<uint32_t *>(vc) + ((static_cast<size_t>(b) * Hkv + hk) * S + slot) * (D / 2) + dpair) = raw;
  }
}

// silu(a) * b with torch's rounding points: bf16(bf16(silu(a)) * b)
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t *__restrict__ a, const uint16_t *__restrict__ bq,
                                                       uint16_t *__restrict__ y, int64_t n8) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n8) return;
  const u32x4_t ra = reinterpret_cast<const u32x4_t *>(a)[idx];
  const u32x4_t rb = reinterpret_cast<const u32x4_t *>(bq)[idx];
  u32x4_t o;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float a0 = __builtin_bit_cast(float, ra[j] << 16), a1 = __builtin_bit_cast(float, ra[j] & 0xFFFF0000u);
    const float s0 = bf16_round(a0 / (1.0f + expf(-a0))), s1 = bf16_round(a1 / (1.0f + expf(-a1)));
    const float y0 = s0 * __builtin_bit_cast(float, rb[j] << 16), y1 = s1 * __builtin_bit_cast(float, rb[j] & 0xFFFF0000u);
    o[j] = static_cast<uint32_t>(f32_to_bf16_rne(y0)) | (static_cast<uint32_t>(f32_to_bf16_rne(y1)) << 16);
  }
  reinterpret_cast<u32x4_t *>(y)[idx] = o;
}

// few rows (decode): 512 threads so that a 4096-wide row is one piece per thread; many rows: 256-thread workgroups
void launch_rmsnorm(const uint16_t *x, const uint16_t *delta, const float *psum, int slices, const uint16_t *col_scales, const uint16_t *w,
                    uint16_t *h_out, uint16_t *y, StagedOut staged, int64_t rows, int64_t dim, float eps, hipStream_t stream) {
  if (rows <= 512 && dim >= 4096)
    hipLaunchKernelGGL(rmsnorm_kernel<512>, dim3(static_cast<unsigned>(rows)), dim3(512), 0, stream, x, delta, psum, slices, col_scales, w, h_out,
                       y, staged, static_cast<int>(dim), eps);
  else
    hipLaunchKernelGGL(rmsnorm_kernel<256>, dim3(static_cast<unsigned>(rows)), dim3(256), 0, stream, x, delta, psum, slices, col_scales, w, h_out,
                       y, staged, static_cast<int>(dim), eps);
}

template <int D, int NW>
int launch_attention_nw(int rep, dim3 grid, hipStream_t s, const uint16_t *q, const uint16_t *kc, const uint16_t *vc, uint16_t *out,
                        const int64_t *input_pos, const int64_t *left_pad, int H, int Hkv, int S, float scale, StagedOut staged) {
  switch (rep) {
    case 1: hipLaunchKernelGGL((decode_attention_kernel<D, 1, NW>), grid, dim3(64 * NW), 0, s, q, kc, vc, out, input_pos, left_pad, H, Hkv, S, scale, staged); break;
    case 2: hipLaunchKernelGGL((decode_attention_kernel<D, 2, NW>), grid, dim3(64 * NW), 0, s, q, kc, vc, out, input_pos, left_pad, H, Hkv, S, scale, staged); break;
    case 4: hipLaunchKernelGGL((decode_attention_kernel<D, 4, NW>), grid, dim3(64 * NW), 0, s, q, kc, vc, out, input_pos, left_pad, H, Hkv, S, scale, staged); break;
    case 8: hipLaunchKernelGGL((decode_attention_kernel<D, 8, NW>), grid, dim3(64 * NW), 0, s, q, kc, vc, out, input_pos, left_pad, H, Hkv, S, scale, staged); break;
    default: return E2H_ERR_BAD_SHAPE;
  }
  return launch_status();
}

// The live length is a device value (graph replays move it), so the waves per workgroup follow the cache length:
// eight waves for caches beyond 256 positions halve the tiles a wave walks through one after the other.
template <int D>
int launch_attention(int rep, dim3 grid, hipStream_t s, const uint16_t *q, const uint16_t *kc, const uint16_t *vc, uint16_t *out,
                     const int64_t *input_pos, const int64_t *left_pad, int H, int Hkv, int S, float scale, StagedOut staged) {
  const int nw = options().attention_waves ? options().attention_waves : (S > 256 ? 8 : 4);
  if (D == 128 && rep >= 4 && rep <= 16 && !options().attention_no_mfma) {
    // several query heads per K / V row: both products on the matrix cores; four waves measured faster than eight
    // (three workgroups fit a CU instead of one)
    if (options().attention_waves == 8)
      hipLaunchKernelGGL(decode_attention_gqa_kernel<8>, grid, dim3(512), 0, s, q, kc, vc, out, input_pos, left_pad, H, Hkv, S, rep, scale, staged);
    else
      hipLaunchKernelGGL(decode_attention_gqa_kernel<4>, grid, dim3(256), 0, s, q, kc, vc, out, input_pos, left_pad, H, Hkv, S, rep, scale, staged);
    return launch_status();
  }
  if (nw == 8) return launch_attention_nw<D, 8>(rep, grid, s, q, kc, vc, out, input_pos, left_pad, H, Hkv, S, scale, staged);
  return launch_attention_nw<D, 4>(rep, grid, s, q, kc, vc, out, input_pos, left_pad, H, Hkv, S, scale, staged);
}

}  // namespace
}  // namespace e2h

using namespace e2h;

namespace {
int decode_attention_impl(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *out, void *staged,
                          const int64_t *input_pos, const int64_t *left_pad_mask_pos, int64_t batch, int64_t n_head, int64_t n_kv_head,
                          int64_t cache_len, int64_t head_dim, float scale, void *stream) {
  if (!q || !k_cache || !v_cache || (!out && !staged) || !input_pos) return E2H_ERR_NULL_POINTER;
  if (batch < 1 || n_head < 1 || n_kv_head < 1 || n_head % n_kv_head != 0 || cache_len < 1 || batch * n_kv_head > INT32_MAX)
    return E2H_ERR_BAD_SHAPE;
  if (staged && (batch > 64 || (n_head * head_dim) % 128 != 0)) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(staged)) return E2H_ERR_MISALIGNED;
  const int rep = static_cast<int>(n_head / n_kv_head);
  dim3 grid(static_cast<unsigned>(batch * n_kv_head));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const StagedOut so = staged_out(staged, batch, n_head * head_dim);
  if (head_dim == 128)
    return launch_attention<128>(rep, grid, s, q, k_cache, v_cache, out, input_pos, left_pad_mask_pos, (int)n_head, (int)n_kv_head, (int)cache_len, scale, so);
  if (head_dim == 64)
    return launch_attention<64>(rep, grid, s, q, k_cache, v_cache, out, input_pos, left_pad_mask_pos, (int)n_head, (int)n_kv_head, (int)cache_len, scale, so);
  return E2H_ERR_BAD_SHAPE;
}
}  // namespace

extern "C" int e2h_decode_attention(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *out,
                                    const int64_t *input_pos, const int64_t *left_pad_mask_pos, int64_t batch, int64_t n_head,
                                    int64_t n_kv_head, int64_t cache_len, int64_t head_dim, float scale, void *stream) {
  if (!out) return E2H_ERR_NULL_POINTER;
  return decode_attention_impl(q, k_cache, v_cache, out, nullptr, input_pos, left_pad_mask_pos, batch, n_head, n_kv_head, cache_len, head_dim, scale, stream);
}

extern "C" int e2h_decode_attention_staged(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *out, void *staged,
                                           const int64_t *input_pos, const int64_t *left_pad_mask_pos, int64_t batch, int64_t n_head,
                                           int64_t n_kv_head, int64_t cache_len, int64_t head_dim, float scale, void *stream) {
  return decode_attention_impl(q, k_cache, v_cache, out, staged, input_pos, left_pad_mask_pos, batch, n_head, n_kv_head, cache_len, head_dim, scale, stream);
}

extern "C" int e2h_rmsnorm(const uint16_t *x, const uint16_t *weight, uint16_t *y, int64_t rows, int64_t dim, float eps, void *stream) {
  if (!x || !weight || !y) return E2H_ERR_NULL_POINTER;
  if (rows < 1 || dim < 8 || dim % 8 != 0 || rows > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(weight) || !aligned16(y)) return E2H_ERR_MISALIGNED;
  launch_rmsnorm(x, nullptr, nullptr, 0, nullptr, weight, nullptr, y, StagedOut{}, rows, dim, eps, static_cast<hipStream_t>(stream));
  return launch_status();
}

extern "C" int e2h_add_rmsnorm(const uint16_t *x, const uint16_t *delta, const uint16_t *weight, uint16_t *h_out, uint16_t *y,
                               int64_t rows, int64_t dim, float eps, void *stream) {
  if (!x || !delta || !weight || !h_out || !y) return E2H_ERR_NULL_POINTER;
  if (rows < 1 || dim < 8 || dim % 8 != 0 || rows > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(delta) || !aligned16(weight) || !aligned16(h_out) || !aligned16(y)) return E2H_ERR_MISALIGNED;
  launch_rmsnorm(x, delta, nullptr, 0, nullptr, weight, h_out, y, StagedOut{}, rows, dim, eps, static_cast<hipStream_t>(stream));
  return launch_status();
}

extern "C" int e2h_add_rmsnorm_partials(const uint16_t *x, const float *partials, int slices, const uint16_t *col_scales,
                                        const uint16_t *weight, uint16_t *h_out, uint16_t *y, int64_t rows, int64_t dim, float eps,
                                        void *stream) {
  if (!x || !partials || !weight || !h_out || !y) return E2H_ERR_NULL_POINTER;
  if (rows < 1 || dim < 8 || dim % 8 != 0 || rows > INT32_MAX || slices < 1 || slices > 64) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(partials) || !aligned16(weight) || !aligned16(h_out) || !aligned16(y) || (col_scales && !aligned16(col_scales)))
    return E2H_ERR_MISALIGNED;
  launch_rmsnorm(x, nullptr, partials, slices, col_scales, weight, h_out, y, StagedOut{}, rows, dim, eps, static_cast<hipStream_t>(stream));
  return launch_status();
}

extern "C" int e2h_add_rmsnorm_staged(const uint16_t *x, const uint16_t *delta, const float *partials, int slices, const uint16_t *col_scales,
                                      const uint16_t *weight, uint16_t *h_out, uint16_t *y, void *staged, int64_t rows, int64_t dim, float eps,
                                      void *stream) {
  if (!x || !weight || (!y && !staged)) return E2H_ERR_NULL_POINTER;
  if (delta && partials) return E2H_ERR_BAD_SHAPE;
  if ((delta || partials) && !h_out) return E2H_ERR_NULL_POINTER;
  if (rows < 1 || dim < 8 || dim % 8 != 0 || rows > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if (partials && (slices < 1 || slices > 64)) return E2H_ERR_BAD_SHAPE;
  if (staged && (rows > 64 || dim % 128 != 0)) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(x) || !aligned16(delta) || !aligned16(partials) || !aligned16(weight) || !aligned16(h_out) || !aligned16(y) ||
      !aligned16(staged) || !aligned16(col_scales))
    return E2H_ERR_MISALIGNED;
  launch_rmsnorm(x, delta, partials, partials ? slices : 0, partials ? col_scales : nullptr, weight, h_out, y, staged_out(staged, rows, dim), rows, dim,
                 eps, static_cast<hipStream_t>(stream));
  return launch_status();
}

extern "C" int e2h_rope_kv_write_seq(const uint16_t *qkv, const uint16_t *freqs_cis, uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache,
                                     const int64_t *input_pos, int64_t batch, int64_t seqlen, int64_t n_head, int64_t n_kv_head,
                                     int64_t cache_len, int64_t head_dim, int rows_by_token, void *stream) {
  if (!qkv || !freqs_cis || !q_out || !k_cache || !v_cache || !input_pos) return E2H_ERR_NULL_POINTER;
  if (batch < 1 || seqlen < 1 || n_head < 1 || n_kv_head < 1 || head_dim < 2 || head_dim % 2 != 0 || cache_len < 1 || cache_len > INT32_MAX)
    return E2H_ERR_BAD_SHAPE;
  const int64_t pairs = batch * seqlen * (n_head + 2 * n_kv_head) * head_dim / 2;
  if (batch * seqlen > INT32_MAX || (pairs + 255) / 256 > INT32_MAX) return E2H_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(qkv) & 3u) || (reinterpret_cast<uintptr_t>(freqs_cis) & 3u) || (reinterpret_cast<uintptr_t>(q_out) & 3u) ||
      (reinterpret_cast<uintptr_t>(k_cache) & 3u) || (reinterpret_cast<uintptr_t>(v_cache) & 3u) || (reinterpret_cast<uintptr_t>(input_pos) & 7u))
    return E2H_ERR_MISALIGNED;
  const bool vec = (head_dim % 8) == 0 && !((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(freqs_cis) | reinterpret_cast<uintptr_t>(q_out) |
                                            reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache)) & 15u);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (vec)
    hipLaunchKernelGGL(rope_kv_write_kernel<4>, dim3(static_cast<unsigned>((pairs / 4 + 255) / 256)), dim3(256), 0, st, qkv, freqs_cis, q_out, k_cache,
                       v_cache, input_pos, (int)batch, (int)seqlen, (int)n_head, (int)n_kv_head, (int)cache_len, (int)head_dim, rows_by_token ? 1 : 0);
  else
    hipLaunchKernelGGL(rope_kv_write_kernel<1>, dim3(static_cast<unsigned>((pairs + 255) / 256)), dim3(256), 0, st, qkv, freqs_cis, q_out, k_cache,
                       v_cache, input_pos, (int)batch, (int)seqlen, (int)n_head, (int)n_kv_head, (int)cache_len, (int)head_dim, rows_by_token ? 1 : 0);
  return launch_status();
}

extern "C" int e2h_rope_kv_write(const uint16_t *qkv, const uint16_t *freqs_cis, uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache,
                                 const int64_t *input_pos, int64_t batch, int64_t n_head, int64_t n_kv_head, int64_t cache_len,
                                 int64_t head_dim, void *stream) {
  return e2h_rope_kv_write_seq(qkv, freqs_cis, q_out, k_cache, v_cache, input_pos, batch, 1, n_head, n_kv_head, cache_len, head_dim, 0, stream);
}

extern "C" int e2h_silu_mul(const uint16_t *a, const uint16_t *b, uint16_t *y, int64_t n, void *stream) {
  if (!a || !b || !y) return E2H_ERR_NULL_POINTER;
  if (n < 8 || n % 8 != 0) return E2H_ERR_BAD_SHAPE;
  if (!aligned16(a) || !aligned16(b) || !aligned16(y)) return E2H_ERR_MISALIGNED;
  hipLaunchKernelGGL(silu_mul_kernel, dim3(static_cast<unsigned>((n / 8 + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream), a, b, y, n / 8);
  return launch_status();
}

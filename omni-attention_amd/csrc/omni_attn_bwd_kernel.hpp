// Backward of the block-sparse attention forward for gfx950 (MI355X, CDNA4).
//
// The reference has no backward (its operator is forward-only, omni-attn-mma/pybind/omni_attn.cc:70-77);
// what is differentiated here is exactly the function the forward kernel computes -- per
// query block the listed KV blocks with their FULL / CAUSAL / PARTIAL / MASKED semantics
// (omni-attn-mma/mma/attn_naive.cu:21-302), softmax scale 1/sqrt(D):
//
//   P_ij  = exp(q_i.k_j / sqrt(D) - LSE_i)   for allowed (i, j) of a listed block, else 0
//   delta_i = sum_d dO_id O_id
//   dV_j  = sum_i P_ij dO_i
//   dS_ij = P_ij (dO_i.v_j - delta_i)
//   dQ_i  = sum_j dS_ij k_j / sqrt(D)         dK_j = sum_i dS_ij q_i / sqrt(D)
//
// Two kernels, no atomics, bitwise reproducible:
//   bwd_dq_kernel    one workgroup per query block; walks that block's list like the forward;
//                    also writes delta for its rows (workspace, read by the second kernel).
//   bwd_dkdv_kernel  one workgroup per KV block; finds the (query block, slot) pairs that list
//                    it by scanning the slab's metadata (a bitmap of the matches is built in
//                    LDS first, then visited in ascending order).
// The dQ kernel runs two workgroups per compute unit (two waves per SIMD, each hides the other's
// loads); the dK/dV kernel needs more than 256 registers per lane and runs one.
// Both use the forward's building blocks with the operands exchanged: every product is a
// v_mfma_f32_32x32x16 whose A operand comes from an LDS tile (row-wise or transposed read)
// and whose B operand is in registers, and the accumulator of the first product of a step is
// the B operand of the second one, so P and dS never leave registers.
// Tiles are single-buffered: this is the straightforward schedule, not the forward's pipeline.
#pragma once

#include "omni_attn_fwd_kernel.hpp"

namespace omni_attn {

typedef __attribute__((ext_vector_type(4))) float f32x4_t;

struct BwdParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const uint16_t* o;
  const uint16_t* dout;
  const float* lse;  // [B,H,S] natural-log logsumexp written by the forward
  uint16_t* dq;
  uint16_t* dk;
  uint16_t* dv;
  float* delta;  // [B,H,S] workspace: written by the dQ kernel, read by the dK/dV kernel
  const int32_t* kv_num_blocks;
  const int32_t* kv_indices;
  const int32_t* types;
  const int32_t* partial_idx;
  const uint8_t* partial_masks;
  const uint32_t* partial_bits;
  int num_partial;
  int S, Tq, Tk, max_blocks, seqlen, n_slabs;
  float sl2;      // log2(e) / sqrt(D)
  float scale;    // 1 / sqrt(D)
  float softcap;  // > 0: the forward replaced x = s / sqrt(D) by softcap * tanh(x / softcap)
  float cap_c2;   // 2 * log2(e) / (sqrt(D) * softcap)
};

// Weight and score-gradient factor of one score.  Plain: p = exp2(s * sl2 - lse2), factor 1.
// Soft-capped: t = tanh(s / sqrt(D) / cap), p = exp2(cap * t * log2 e - lse2), factor 1 - t^2
// (the derivative of cap * tanh(x / cap) with respect to x).
__device__ __forceinline__ void bwd_weight(float s, float lse2, const BwdParams& p, float& w, float& dfac) {
  if (p.softcap > 0.f) {
    const float ex = __builtin_amdgcn_exp2f(s * p.cap_c2);
    const float t = __builtin_fmaf(__builtin_amdgcn_rcpf(ex + 1.f), -2.f, 1.f);
    w = __builtin_amdgcn_exp2f(__builtin_fmaf(t, p.softcap * 1.4426950408889634f, -lse2));
    dfac = __builtin_fmaf(-t, t, 1.f);
  } else {
    w = __builtin_amdgcn_exp2f(__builtin_fmaf(s, p.sl2, -lse2));
    dfac = 1.f;
  }
}

template <int QB>
struct BwdStep {
  // rows of a tile: the forward's rule (a 64-row block has half the threads)
  static constexpr int value = QB == 64 ? 32 : 64;
};

// [ROWS][D] tile from a slab into LDS, 16-byte chunks swizzled for row-wise (TR = false) or
// transposed (TR = true) operand reads.  Rows at or beyond the end of the slab read as zeros.
template <int D, int NT, int ROWS, bool TR>
__device__ __forceinline__ void bwd_load_tile(i32x4_t rsrc, int row0, uint32_t lds_tile, int tid, int w) {
  constexpr int CPR = D / 8;
  constexpr int NCH = ROWS * CPR / NT;
  static_assert(ROWS * CPR % NT == 0 && NCH >= 1, "tile must divide over the workgroup");
  constexpr int ROW_STRIDE = NT / CPR;
  const int ld_row = tid / CPR, ld_pch = tid % CPR;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int row = ld_row + i * ROW_STRIDE;
    uint32_t off;
    if constexpr (TR) {
      off = uint32_t(row * D + ((((ld_pch >> 1) ^ v_swizzle<D>(row)) << 1) | (ld_pch & 1)) * 8) * 2u;
    } else {
      off = uint32_t(row * D + (ld_pch ^ k_swizzle<D>(row)) * 8) * 2u;
    }
    buffer_to_lds_b128(rsrc, off, uint32_t(row0) * uint32_t(D * 2), lds_tile + uint32_t(w) * 1024u + uint32_t(i) * (NT * 16u));
  }
}

// A operand, row-wise: rows 32t + c of the tile, k-step s.
template <int D>
__device__ __forceinline__ u32x4_t bwd_row_frag(const uint16_t* tile, int s, int t, int g, int c) {
  const int row = 32 * t + c;
  const int ch = (2 * s + g) ^ k_swizzle<D>(row);
  return *reinterpret_cast<const u32x4_t*>(tile + row * D + ch * 8);
}
// A operand, transposed: rows 32 dt .. +31 of tile^T at tile rows 16 ts .. +15, the 16 rows
// taken in the accumulator order of the first product.
template <int D>
__device__ __forceinline__ u32x4_t bwd_tr_frag(const uint16_t* tile, int ts, int dt, int g, int c) {
  const int i16 = c & 15, j16 = c >> 4;
  const int vrow = 16 * ts + 4 * g + (i16 >> 2);
  const int unit = 2 * dt + j16;
  const int u0 = unit ^ v_swizzle<D>(vrow);
  const int u1 = unit ^ v_swizzle<D>(vrow + 8);
  const s16x4_t lo = lds_read_tr16(tile + vrow * D + u0 * 16 + (i16 & 3) * 4);
  const s16x4_t hi = lds_read_tr16(tile + (vrow + 8) * D + u1 * 16 + (i16 & 3) * 4);
  const u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo);
  const u32x2_t hi2 = __builtin_bit_cast(u32x2_t, hi);
  const u32x4_t a = {lo2[0], lo2[1], hi2[0], hi2[1]};
  return a;
}

// 32 mask bytes -> 32 bits (any non-zero byte = 1), byte i -> bit i.
__device__ __forceinline__ uint32_t bwd_pack32(const u32x4_t m0, const u32x4_t m1) {
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    uint32_t bytes = i < 4 ? m0[i] : m1[i - 4];
    bytes |= bytes >> 4;
    bytes |= bytes >> 2;
    bytes |= bytes >> 1;
    word |= (((bytes & 0x01010101u) * 0x01020408u) >> 24) << (4 * i);
  }
  return word;
}

// Effective mode of a slot, as the forward decides it.
__device__ __forceinline__ int32_t bwd_slot_mode(int32_t ty, int32_t pid, bool has_partial, int num_partial) {
  int32_t mode = (ty == kCausal || ty == kFull || ty == kPartial) ? ty : int32_t(kMasked);
  if (ty == kPartial && (!has_partial || pid < 0 || pid >= num_partial)) mode = kMasked;
  return mode;
}

// Transposed accumulators [D rows][32 columns] x factor -> 16-bit rows of the output, staged
// through LDS so that whole rows are stored (the forward's epilogue).
template <bool BF16, int D>
__device__ __forceinline__ void bwd_store_rows(const f32x16_t (&acc)[D / 32], float factor, uint16_t* stage,
                                               uint16_t* out_slab, int first_row, int n_rows_slab, int lane) {
  constexpr int CPR = D / 8, DT = D / 32;
  const int g = lane >> 5, c = lane & 31;
  static_for<DT * 4>([&](auto ic) {
    constexpr int dt = decltype(ic)::value / 4, r4 = decltype(ic)::value % 4;
    u32x2_t ov;
    ov[0] = pack2<BF16>(acc[dt][4 * r4 + 0] * factor, acc[dt][4 * r4 + 1] * factor);
    ov[1] = pack2<BF16>(acc[dt][4 * r4 + 2] * factor, acc[dt][4 * r4 + 3] * factor);
    const int ch = (4 * dt + r4) ^ k_swizzle<D>(c);
    *reinterpret_cast<u32x2_t*>(stage + c * D + ch * 8 + 4 * g) = ov;
  });
  constexpr int ROWS_PER_STORE = 64 / CPR;
  const int srow = lane / CPR, pch = lane % CPR;
#pragma unroll
  for (int i = 0; i < 32 / ROWS_PER_STORE; ++i) {
    const int row = i * ROWS_PER_STORE + srow;
    const u32x4_t val = *reinterpret_cast<const u32x4_t*>(stage + row * D + pch * 8);
    const int grow = first_row + row;
    if (grow < n_rows_slab)
      *reinterpret_cast<u32x4_t*>(out_slab + size_t(grow) * D + (pch ^ k_swizzle<D>(row)) * 8) = val;
  }
}

template <int D, int QB>
struct BwdDqTraits {
  static constexpr int kThreads = QB * 2;
  static constexpr int kStep = BwdStep<QB>::value;
  static constexpr int kTileElems = kStep * D;
  // three tiles (K row-wise, K transposed, V row-wise) or the output staging, whichever is larger
  static constexpr size_t kLdsBytes = (3 * kTileElems > QB * D ? 3 * kTileElems : QB * D) * sizeof(uint16_t);
};

template <bool BF16, int D, int QB, int KB>
__global__ void __launch_bounds__(QB * 2, 2) bwd_dq_kernel(const BwdParams p) {
  using Traits = BwdDqTraits<D, QB>;
  constexpr int NT = Traits::kThreads;
  constexpr int STEP = Traits::kStep;
  constexpr int SPB = KB / STEP;
  constexpr int NTL = STEP / 32;
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  constexpr int TILE = Traits::kTileElems;

  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  uint16_t* sKa = reinterpret_cast<uint16_t*>(lds_raw);
  uint16_t* sKt = sKa + TILE;
  uint16_t* sVa = sKt + TILE;

  const int bh = blockIdx.x / p.Tq;
  const int qb = p.Tq - 1 - (blockIdx.x - bh * p.Tq);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c = lane & 31;

  const size_t slab = size_t(bh) * size_t(p.S) * D;
  const uint32_t slab_bytes = uint32_t(p.S) * uint32_t(D * 2);
  const i32x4_t rK = make_buffer_resource(p.k + slab, slab_bytes);
  const i32x4_t rV = make_buffer_resource(p.v + slab, slab_bytes);
  const int q_row = qb * QB + 32 * w + c;
  const int q_wave_min = qb * QB + 32 * w;
  const int qr = q_row < p.S ? q_row : p.S - 1;
  const size_t meta_row = size_t(bh) * p.Tq + qb;
  const size_t meta_off = meta_row * p.max_blocks;
  const bool has_partial = p.partial_idx != nullptr && (p.partial_masks != nullptr || p.partial_bits != nullptr);

  int nb = load_uniform(p.kv_num_blocks + meta_row);
  nb = nb < 0 ? 0 : (nb > p.max_blocks ? p.max_blocks : nb);

  // Q and dO as B operands; delta = rowsum(dO . O) on the way.
  u32x4_t qf[KS], dof[KS];
  float dsum = 0.f;
  {
    const uint16_t* qp = p.q + slab + size_t(qr) * D + 8 * g;
    const uint16_t* dop = p.dout + slab + size_t(qr) * D + 8 * g;
    const uint16_t* op = p.o + slab + size_t(qr) * D + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      qf[s] = *reinterpret_cast<const u32x4_t*>(qp + 16 * s);
      dof[s] = *reinterpret_cast<const u32x4_t*>(dop + 16 * s);
      const u32x4_t of = *reinterpret_cast<const u32x4_t*>(op + 16 * s);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // (elements are copied to scalars first: a bit cast applied directly to a vector element
        // expression reads element 0)
        const uint32_t da = dof[s][e], ob = of[e];
        float a0, a1, b0, b1;
        if constexpr (BF16) {
          const uint32_t da_lo = da << 16, da_hi = da & 0xffff0000u, ob_lo = ob << 16, ob_hi = ob & 0xffff0000u;
          a0 = __builtin_bit_cast(float, da_lo);
          a1 = __builtin_bit_cast(float, da_hi);
          b0 = __builtin_bit_cast(float, ob_lo);
          b1 = __builtin_bit_cast(float, ob_hi);
        } else {
          const f16x2_t a = __builtin_bit_cast(f16x2_t, da);
          const f16x2_t b = __builtin_bit_cast(f16x2_t, ob);
          a0 = float(a[0]); a1 = float(a[1]); b0 = float(b[0]); b1 = float(b[1]);
        }
        dsum = __builtin_fmaf(a0, b0, dsum);
        dsum = __builtin_fmaf(a1, b1, dsum);
      }
    }
  }
  const float delta = pair_sum(dsum);  // the row lives in lanes c and c + 32
  const float lse = p.lse[size_t(bh) * p.S + qr];
  const bool row_live = q_row < p.seqlen && lse != -INFINITY;
  // exponent offset; +inf for rows without any allowed key so that every weight becomes 0
  const float lse2 = row_live ? lse * 1.4426950408889634f : INFINITY;
  if (q_row < p.S && g == 0) p.delta[size_t(bh) * p.S + q_row] = delta;

  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16_t dq[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) dq[dt] = zero16;

  for (int j = 0; j < nb; ++j) {
    const size_t o = meta_off + size_t(j);
    const int32_t kvb_raw = load_uniform(p.kv_indices + o);
    const int32_t ty = load_uniform(p.types + o);
    const int32_t pid = has_partial ? load_uniform(p.partial_idx + o) : -1;
    const int32_t kvb = kvb_raw < 0 ? 0 : (kvb_raw >= p.Tk ? p.Tk - 1 : kvb_raw);
    const int32_t mode = bwd_slot_mode(ty, pid, has_partial, p.num_partial);
    if (mode == kMasked) continue;
    for (int half = 0; half < SPB; ++half) {
      const int row0 = kvb * KB + half * STEP;
      if (row0 >= p.seqlen) continue;                                  // no allowed key
      if (mode == kCausal && row0 > qb * QB + QB - 1) continue;        // entirely above the diagonal
      __syncthreads();  // the previous step's operand reads are done
      bwd_load_tile<D, NT, STEP, false>(rK, row0, lds_offset_of(sKa), tid, w);
      bwd_load_tile<D, NT, STEP, true>(rK, row0, lds_offset_of(sKt), tid, w);
      bwd_load_tile<D, NT, STEP, false>(rV, row0, lds_offset_of(sVa), tid, w);
      // mask words of this lane's row: bit j of word t = key row0 + 32 t + j allowed
      uint32_t kw[NTL];
#pragma unroll
      for (int t = 0; t < NTL; ++t) kw[t] = 0xffffffffu;
      if (mode == kPartial) {
        const int q_local = q_row - qb * QB;
#pragma unroll
        for (int t = 0; t < NTL; ++t) {
          const int kcol = half * STEP + 32 * t;
          if (p.partial_bits != nullptr) {
            kw[t] = p.partial_bits[(size_t(pid) * QB + q_local) * (KB / 32) + kcol / 32];
          } else {
            const uint8_t* mp = p.partial_masks + (size_t(pid) * QB + q_local) * KB + kcol;
            kw[t] = bwd_pack32(*reinterpret_cast<const u32x4_t*>(mp), *reinterpret_cast<const u32x4_t*>(mp + 16));
          }
        }
      }
      int limit = p.seqlen - 1;
      if (mode == kCausal) limit = limit < q_row ? limit : q_row;
      const int lim_l = limit - row0 - 4 * g;
      static_for<NTL>([&](auto tc) {
        constexpr int t = decltype(tc)::value;
        kw[t] >>= 4 * g;
        const int n = lim_l - 32 * t + 1;
        const uint32_t low = n >= 32 ? 0xffffffffu : (n <= 0 ? 0u : ((1u << (n & 31)) - 1u));
        kw[t] &= low;
      });
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): tiles (and mask words) have landed
      __syncthreads();

      // S^T = K.Q^T and dP^T = V.dO^T : lane = query row, registers = keys
      f32x16_t st[NTL], dp[NTL];
      static_for<NTL>([&](auto tc) {
        constexpr int t = decltype(tc)::value;
        st[t] = zero16;
        dp[t] = zero16;
        static_for<KS>([&](auto sc) {
          constexpr int s = decltype(sc)::value;
          st[t] = mfma_32x32x16<BF16>(bwd_row_frag<D>(sKa, s, t, g, c), qf[s], st[t]);
          dp[t] = mfma_32x32x16<BF16>(bwd_row_frag<D>(sVa, s, t, g, c), dof[s], dp[t]);
        });
      });
      // dS^T = P^T (dP^T - delta), packed to 16 bits in the order the next product reads it
      u32x4_t dsb[NTL][2];
      static_for<8 * NTL>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        constexpr int t = i / 8, r = 2 * (i % 8);
        constexpr int kl0 = 8 * (r >> 2) + (r & 3), kl1 = 8 * ((r + 1) >> 2) + ((r + 1) & 3);
        const bool keep0 = (kw[t] >> kl0) & 1u, keep1 = (kw[t] >> kl1) & 1u;
        float w0, w1, f0, f1;
        bwd_weight(st[t][r], lse2, p, w0, f0);
        bwd_weight(st[t][r + 1], lse2, p, w1, f1);
        const float p0 = keep0 ? w0 : 0.f;
        const float p1 = keep1 ? w1 : 0.f;
        const float d0 = p0 * (dp[t][r] - delta) * f0;
        const float d1 = p1 * (dp[t][r + 1] - delta) * f1;
        dsb[t][r >> 3][(r & 7) >> 1] = pack2<BF16>(d0, d1);
      });
      // dQ^T += K^T.dS^T
      static_for<(STEP / 16) * DT>([&](auto jc) {
        constexpr int ts = decltype(jc)::value / DT, dt = decltype(jc)::value % DT;
        dq[dt] = mfma_32x32x16<BF16>(bwd_tr_frag<D>(sKt, ts, dt, g, c), dsb[ts >> 1][ts & 1], dq[dt]);
      });
    }
  }
  __syncthreads();  // tiles are dead: the staging area overlaps them
  uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + size_t(w) * 32 * D;
  bwd_store_rows<BF16, D>(dq, p.scale, stage, p.dq + slab, q_wave_min, p.S, lane);
}

template <int D, int KB>
struct BwdDkdvTraits {
  static constexpr int kThreads = KB * 2;
  // query rows per step: 32 where the tile still divides over the workgroup (two accumulator
  // pairs per wave already fill most of the register file), else the forward's rule
  static constexpr int kStep = (32 * (D / 8) % (KB * 2) == 0) ? 32 : BwdStep<KB>::value;
  static constexpr int kTileElems = kStep * D;
  static constexpr int kMaxBitmapWords = 4096;      // 64-slot words of the match bitmap (32 KiB)
  // four tiles (Q and dO, each row-wise and transposed) or the output staging, + lse and delta of a
  // step's rows, + the bitmap of (query block, slot) pairs that list this KV block
  static constexpr size_t kTileBytes = (4 * kTileElems > KB * D ? 4 * kTileElems : KB * D) * sizeof(uint16_t);
  static constexpr size_t kLdsBytes = kTileBytes + 2 * kStep * sizeof(float) + size_t(kMaxBitmapWords) * 8;
};

template <bool BF16, int D, int QB, int KB>
__global__ void __launch_bounds__(KB * 2, 1) bwd_dkdv_kernel(const BwdParams p) {
  using Traits = BwdDkdvTraits<D, KB>;
  constexpr int NT = Traits::kThreads;
  constexpr int NW = NT / 64;
  constexpr int STEP = Traits::kStep;
  constexpr int SPQ = QB / STEP;  // steps per query block (QB 64 with 64-row steps: one step, half used)
  constexpr int NSTEPS = SPQ > 0 ? SPQ : 1;
  constexpr int NTL = STEP / 32;
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  constexpr int TILE = Traits::kTileElems;

  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  uint16_t* sQa = reinterpret_cast<uint16_t*>(lds_raw);
  uint16_t* sQt = sQa + TILE;
  uint16_t* sDa = sQt + TILE;
  uint16_t* sDt = sDa + TILE;
  float* sLse = reinterpret_cast<float*>(lds_raw + Traits::kTileBytes);
  float* sDelta = sLse + STEP;
  uint64_t* sMatch = reinterpret_cast<uint64_t*>(sDelta + STEP);

  const int bh = blockIdx.x / p.Tk;
  const int kvb = blockIdx.x - bh * p.Tk;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c = lane & 31;

  const size_t slab = size_t(bh) * size_t(p.S) * D;
  const uint32_t slab_bytes = uint32_t(p.S) * uint32_t(D * 2);
  const i32x4_t rQ = make_buffer_resource(p.q + slab, slab_bytes);
  const i32x4_t rD = make_buffer_resource(p.dout + slab, slab_bytes);
  const int key_wave_min = kvb * KB + 32 * w;
  const int key = key_wave_min + c;  // this lane's key row inside the slab
  const int kr = key < p.S ? key : p.S - 1;
  const bool has_partial = p.partial_idx != nullptr && (p.partial_masks != nullptr || p.partial_bits != nullptr);
  const size_t meta_slab = size_t(bh) * p.Tq;
  const int chunks = (p.max_blocks + 63) / 64;  // 64-slot words per query block

  // K and V of this lane's key as B operands.
  u32x4_t kf[KS], vf[KS];
  {
    const uint16_t* kp = p.k + slab + size_t(kr) * D + 8 * g;
    const uint16_t* vp = p.v + slab + size_t(kr) * D + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      kf[s] = *reinterpret_cast<const u32x4_t*>(kp + 16 * s);
      vf[s] = *reinterpret_cast<const u32x4_t*>(vp + 16 * s);
    }
  }

  // Pass 1: which (query block, slot) pairs list this KV block (after the forward's clamping of
  // the block index) with a type the forward would visit?  One 64-bit word per query block and 64
  // slots; a wave takes one word at a time.
  for (int word = w; word < p.Tq * chunks; word += NW) {
    const int qb = word / chunks, ch = word - qb * chunks;
    int nb = load_uniform(p.kv_num_blocks + meta_slab + qb);
    nb = nb < 0 ? 0 : (nb > p.max_blocks ? p.max_blocks : nb);
    const int slot = ch * 64 + lane;
    bool hit = false;
    if (slot < nb) {
      const size_t o = (meta_slab + qb) * p.max_blocks + slot;
      const int32_t raw = p.kv_indices[o];
      const int32_t idx = raw < 0 ? 0 : (raw >= p.Tk ? p.Tk - 1 : raw);
      const int32_t ty = p.types[o];
      const int32_t pid = has_partial ? p.partial_idx[o] : -1;
      hit = idx == kvb && bwd_slot_mode(ty, pid, has_partial, p.num_partial) != kMasked;
    }
    const uint64_t bits = __builtin_amdgcn_ballot_w64(hit);
    if (lane == 0) sMatch[word] = bits;
  }
  __syncthreads();

  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16_t dk[DT], dv[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    dk[dt] = zero16;
    dv[dt] = zero16;
  }
  const bool key_live = key < p.seqlen;

  // Pass 2: visit the matches in ascending (query block, slot) order.
  for (int word = 0; word < p.Tq * chunks; ++word) {
    uint64_t bits = sMatch[word];
    // (readfirstlane returns a signed int: go through uint32_t so that bit 31 does not sign-extend)
    bits = (uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(bits >> 32))))) << 32) |
           uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(bits)))));
    const int qb = word / chunks, ch = word - qb * chunks;
    while (bits != 0) {
      const int b = __builtin_ctzll(bits);
      bits &= bits - 1;
      const size_t o = (meta_slab + qb) * p.max_blocks + ch * 64 + b;
      const int32_t ty = load_uniform(p.types + o);
      const int32_t pid = has_partial ? load_uniform(p.partial_idx + o) : -1;
      const int32_t mode = bwd_slot_mode(ty, pid, has_partial, p.num_partial);
      for (int half = 0; half < NSTEPS; ++half) {
        const int q0 = qb * QB + half * STEP;  // first query row of the step
        if (q0 >= p.seqlen) continue;
        if (mode == kCausal && q0 + STEP - 1 < kvb * KB) continue;  // entirely above the diagonal
        __syncthreads();
        bwd_load_tile<D, NT, STEP, false>(rQ, q0, lds_offset_of(sQa), tid, w);
        bwd_load_tile<D, NT, STEP, true>(rQ, q0, lds_offset_of(sQt), tid, w);
        bwd_load_tile<D, NT, STEP, false>(rD, q0, lds_offset_of(sDa), tid, w);
        bwd_load_tile<D, NT, STEP, true>(rD, q0, lds_offset_of(sDt), tid, w);
        if (tid < STEP) {
          const int row = q0 + tid;
          // rows of another query block (a 64-row block in a 64-row step never has any), rows
          // beyond the sequence and rows without any allowed key take no part
          const bool in_block = row < qb * QB + QB && row < p.seqlen;
          const float l = in_block ? p.lse[size_t(bh) * p.S + row] : -INFINITY;
          sLse[tid] = l == -INFINITY ? INFINITY : l * 1.4426950408889634f;
          sDelta[tid] = in_block ? p.delta[size_t(bh) * p.S + row] : 0.f;
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();

        // S = Q.K^T and dP = dO.V^T : lane = key, registers = query rows
        f32x16_t sc[NTL], dp[NTL];
        static_for<NTL>([&](auto tc) {
          constexpr int t = decltype(tc)::value;
          sc[t] = zero16;
          dp[t] = zero16;
          static_for<KS>([&](auto ks) {
            constexpr int s = decltype(ks)::value;
            sc[t] = mfma_32x32x16<BF16>(bwd_row_frag<D>(sQa, s, t, g, c), kf[s], sc[t]);
            dp[t] = mfma_32x32x16<BF16>(bwd_row_frag<D>(sDa, s, t, g, c), vf[s], dp[t]);
          });
        });
        u32x4_t pb[NTL][2], dsb[NTL][2];
        static_for<NTL * 4>([&](auto ic) {
          constexpr int t = decltype(ic)::value / 4, i4 = decltype(ic)::value % 4;
          // registers 4 i4 .. +3 of tile t are query rows 32 t + 8 i4 + 4 g .. +3 of the step
          const int ql = 32 * t + 8 * i4 + 4 * g;
          const f32x4_t l4 = *reinterpret_cast<const f32x4_t*>(sLse + ql);
          const f32x4_t d4 = *reinterpret_cast<const f32x4_t*>(sDelta + ql);
          float pv[4], dsv[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int qrow = q0 + ql + e;  // global query row
            bool keep = key_live;
            if (mode == kCausal) keep = keep && key <= qrow;
            if (mode == kPartial) {
              const int q_local = qrow - qb * QB, k_local = key - kvb * KB;
              bool bit = false;
              if (q_local < QB && key < p.S) {
                if (p.partial_bits != nullptr) {
                  bit = (p.partial_bits[(size_t(pid) * QB + q_local) * (KB / 32) + k_local / 32] >> (k_local & 31)) & 1u;
                } else {
                  bit = p.partial_masks[(size_t(pid) * QB + q_local) * KB + k_local] != 0;
                }
              }
              keep = keep && bit;
            }
            float wgt, fac;
            bwd_weight(sc[t][4 * i4 + e], l4[e], p, wgt, fac);
            pv[e] = keep ? wgt : 0.f;
            dsv[e] = pv[e] * (dp[t][4 * i4 + e] - d4[e]) * fac;
          }
          pb[t][i4 >> 1][2 * (i4 & 1) + 0] = pack2<BF16>(pv[0], pv[1]);
          pb[t][i4 >> 1][2 * (i4 & 1) + 1] = pack2<BF16>(pv[2], pv[3]);
          dsb[t][i4 >> 1][2 * (i4 & 1) + 0] = pack2<BF16>(dsv[0], dsv[1]);
          dsb[t][i4 >> 1][2 * (i4 & 1) + 1] = pack2<BF16>(dsv[2], dsv[3]);
        });
        // dV^T += dO^T.P and dK^T += Q^T.dS
        static_for<(STEP / 16) * DT>([&](auto jc) {
          constexpr int ts = decltype(jc)::value / DT, dt = decltype(jc)::value % DT;
          dv[dt] = mfma_32x32x16<BF16>(bwd_tr_frag<D>(sDt, ts, dt, g, c), pb[ts >> 1][ts & 1], dv[dt]);
          dk[dt] = mfma_32x32x16<BF16>(bwd_tr_frag<D>(sQt, ts, dt, g, c), dsb[ts >> 1][ts & 1], dk[dt]);
        });
      }
    }
  }
  __syncthreads();
  uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + size_t(w) * 32 * D;
  bwd_store_rows<BF16, D>(dk, p.scale, stage, p.dk + slab, key_wave_min, p.S, lane);
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the staging reads of dK are done before dV overwrites them
  bwd_store_rows<BF16, D>(dv, 1.f, stage, p.dv + slab, key_wave_min, p.S, lane);
}

constexpr int kBwdMaxDevices = 64;

template <bool BF16, int D, int QB, int KB>
int launch_bwd(const BwdParams& p, hipStream_t stream) {
  using TQ = BwdDqTraits<D, QB>;
  using TK = BwdDkdvTraits<D, KB>;
  auto kq = bwd_dq_kernel<BF16, D, QB, KB>;
  auto kk = bwd_dkdv_kernel<BF16, D, QB, KB>;
  static std::atomic<bool> lds_limit_set[kBwdMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return int(e);
  const bool cached = dev >= 0 && dev < kBwdMaxDevices;
  if (!cached || !lds_limit_set[dev].load(std::memory_order_acquire)) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kq), hipFuncAttributeMaxDynamicSharedMemorySize,
                            int(TQ::kLdsBytes));
    if (e != hipSuccess) return int(e);
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kk), hipFuncAttributeMaxDynamicSharedMemorySize,
                            int(TK::kLdsBytes));
    if (e != hipSuccess) return int(e);
    if (cached) lds_limit_set[dev].store(true, std::memory_order_release);
  }
  BwdParams params = p;
  void* args[] = {&params};
  e = hipLaunchKernel(reinterpret_cast<const void*>(kq), dim3(unsigned(p.n_slabs) * unsigned(p.Tq)),
                      dim3(TQ::kThreads), args, TQ::kLdsBytes, stream);
  if (e != hipSuccess) return int(e);
  e = hipLaunchKernel(reinterpret_cast<const void*>(kk), dim3(unsigned(p.n_slabs) * unsigned(p.Tk)),
                      dim3(TK::kThreads), args, TK::kLdsBytes, stream);
  return int(e);
}

}  // namespace omni_attn

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
//                    also writes -delta and the rows' score offsets (workspace, read by the
//                    second kernel).
//   bwd_dkdv_kernel  one workgroup per KV block; finds the (query block, slot) pairs that list
//                    it by scanning the slab's metadata (a bitmap of the matches is built in
//                    LDS -- in windows, where the metadata has more words than LDS holds --
//                    and visited in ascending order).  Each 32 keys have two waves
//                    with different work (weights and dV / dP, dS and dK), so two waves share
//                    a SIMD.
// Both use the forward's building blocks with the operands exchanged: every product is a
// v_mfma_f32_32x32x16 whose A operand comes from an LDS tile (row-wise or transposed read of
// the same tile) and whose B operand is in registers, and the accumulator of the first product
// of a step is the B operand of the second one, so P and dS never leave registers (the dK/dV
// kernel hands P from one wave to its partner through LDS).
// Tiles are loaded one step ahead (one barrier per step).  A step of 64 rows (or keys) is two
// 32-wide halves and runs as one sequence of slots like an iteration of the forward: one MFMA,
// the LDS fetch of an operand two or three slots ahead and a share of the vector work of the
// half whose first products have just finished, with a scheduling fence after every slot -- the
// exponentials of one half run under the products of the other inside one wave.  Offsets
// (-LSE sqrt(D), -delta) and masks (-inf) go into the accumulators the products start from, so a
// weight is one multiplication and one exp2 and an unmasked step carries no mask instruction.
// Workgroups are dealt to the XCDs by slab, so the workgroups that run together on an XCD share
// their operands through its L2.
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
  // workspace [2][B,H,S], written by the dQ kernel and read by the dK/dV kernel: plane 0 is
  // -delta = -rowsum(dO . O); plane 1 the offset of the row's scores, -LSE * sqrt(D), -inf for a
  // row without any allowed key or beyond the sequence (every weight of such a row becomes 0) --
  // or, in the soft-capped instances, the exponent offset LSE * log2(e), +inf for such a row
  float* ws;
  const int32_t* kv_num_blocks;
  const int32_t* kv_indices;
  const int32_t* types;
  const int32_t* partial_idx;
  const uint8_t* partial_masks;
  const uint32_t* partial_bits;
  int num_partial;
  int S, Tq, Tk, max_blocks, seqlen, n_slabs;
  int n_xcd;      // XCDs (L2 domains) of the device; workgroup ids go round-robin over them
  float sl2;      // log2(e) / sqrt(D)
  float scale;    // 1 / sqrt(D)
  float softcap;  // > 0: the forward replaced x = s / sqrt(D) by softcap * tanh(x / softcap)
  float cap_c2;   // 2 * log2(e) / (sqrt(D) * softcap)
};

// sqrt(D) for the head dimensions of the instances.
template <int D>
struct SqrtOf {
  static constexpr float value = D == 128 ? 11.313708498984761f : (D == 64 ? 8.f : 5.656854249492381f);
};

// Weight and score-gradient factor of one score.  Plain: p = exp2(s * sl2 - lse2), factor 1.
// Soft-capped: t = tanh(s / sqrt(D) / cap), p = exp2(cap * t * log2 e - lse2), factor 1 - t^2
// (the derivative of cap * tanh(x / cap) with respect to x).
template <bool CAP>
__device__ __forceinline__ void bwd_weight(float s, float lse2, const BwdParams& p, float& w, float& dfac) {
  if constexpr (CAP) {
    const float ex = __builtin_amdgcn_exp2f(s * p.cap_c2);
    const float t = __builtin_fmaf(__builtin_amdgcn_rcpf(ex + 1.f), -2.f, 1.f);
    w = __builtin_amdgcn_exp2f(__builtin_fmaf(t, p.softcap * 1.4426950408889634f, -lse2));
    dfac = __builtin_fmaf(-t, t, 1.f);
  } else {
    w = __builtin_amdgcn_exp2f(__builtin_fmaf(s, p.sl2, -lse2));
    dfac = 1.f;
  }
}

// LDS reads at a byte address.  A fragment's address is (tile + lane part) ^ (k-step bits) + a
// constant: the swizzles of both tile layouts only touch the chunk bits inside a row, and they
// repeat every 16 rows, so rows and tiles are immediate offsets and a fragment costs one XOR.
__device__ __forceinline__ u32x4_t lds_b128_at(uint32_t addr) {
  return *(const __attribute__((address_space(3))) u32x4_t*)(addr);
}
__device__ __forceinline__ f32x4_t lds_f32x4_at(uint32_t addr) {
  return *(const __attribute__((address_space(3))) f32x4_t*)(addr);
}
__device__ __forceinline__ u32x4_t lds_tr_pair_at(uint32_t lo_addr, uint32_t hi_addr) {
  const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(lo_addr));
  const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(hi_addr));
  const u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo);
  const u32x2_t hi2 = __builtin_bit_cast(u32x2_t, hi);
  const u32x4_t a = {lo2[0], lo2[1], hi2[0], hi2[1]};
  return a;
}
// A transposed A fragment at (tile + lane part of its first half) ^ (column bits) + a constant:
// the second half lies 8 tile rows further, where every swizzle differs by chunk bit 1 (32 bytes).
template <int D>
__device__ __forceinline__ u32x4_t lds_tr_frag(uint32_t lo_lane, uint32_t col_bits, uint32_t off) {
  return lds_tr_pair_at((lo_lane ^ col_bits) + off, (lo_lane ^ (col_bits ^ 32u)) + off + 8u * D * 2u);
}

// One LDS layout serves both kinds of operand reads of a backward tile ([rows][D] 16-bit, the
// 16-byte chunk index of a row XORed with a function of the row, period 16 rows):
//   row-wise (ds_read_b128): 16 lanes read the same chunk of 16 consecutive rows -- the 16 XOR
//   values of 16 consecutive rows put them on 16 different 16-byte bank groups;
//   transposed (ds_read_b64_tr_b16): 32 lanes read 4 consecutive chunks of 4 consecutive rows
//   (starting at a multiple of 4) -- those 16 chunks land on 16 different bank groups too.
// So a tile is loaded once however it is read.
template <int D>
__device__ __forceinline__ int bwd_swizzle(int row) {
  if constexpr (D == 128) return ((row & 3) << 2) | ((row >> 2) & 3);
  if constexpr (D == 64) return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
  return (row >> 2) & 3;
}
// Lane part (bytes) of a row-wise A fragment: row 32 t + c of the tile, k-step s at
// ((tile + lane part) ^ 32 s) + 32 t rows.
template <int D>
__device__ __forceinline__ uint32_t bwd_row_lane(int g, int c) {
  return uint32_t(c * D + (g ^ bwd_swizzle<D>(c)) * 8) * 2u;
}
// Lane part (bytes) of a transposed A fragment: rows 32 dt .. +31 of tile^T at tile rows
// 16 ts .. +15 (taken in the accumulator order of the first product) at
// ((tile + lane part) ^ 64 dt) + 16 ts rows; `upper` selects the second half, 8 rows further.
template <int D>
__device__ __forceinline__ uint32_t bwd_tr_lane(int g, int c, int upper) {
  const int i16 = c & 15, j16 = c >> 4, r = 4 * g + (i16 >> 2) + 8 * upper;
  const int chunk = 2 * j16 + ((i16 & 3) >> 1);
  return uint32_t(r * D * 2 + (chunk ^ bwd_swizzle<D>(r)) * 16 + (i16 & 1) * 8);
}

// [ROWS][D] tile from a slab into LDS in that layout.  Rows at or beyond the end of the slab
// read as zeros.
template <int D, int NT, int ROWS>
__device__ __forceinline__ void bwd_load_tile(i32x4_t rsrc, int row0, uint32_t lds_tile, int tid, int w) {
  constexpr int CPR = D / 8;
  constexpr int TOTAL = ROWS * CPR;  // 16-byte chunks of the tile
  constexpr int NCH = TOTAL >= NT ? TOTAL / NT : 1;
  static_assert(TOTAL >= NT ? TOTAL % NT == 0 : TOTAL % 64 == 0, "tile must divide over the threads (or whole waves)");
  constexpr int ROW_STRIDE = NT / CPR;
  if (TOTAL < NT && tid >= TOTAL) return;  // a small tile is loaded by the first waves only
  const int ld_row = tid / CPR, ld_pch = tid % CPR;
  // The swizzle repeats every 16 rows and a thread's loads are ROW_STRIDE rows apart: one or two
  // per-lane offsets serve all of them, the rest of the address is wave-uniform.
  constexpr int PER = (NCH == 1 || ROW_STRIDE % 16 == 0) ? 1 : 2;
  static_assert(NCH == 1 || (PER * ROW_STRIDE) % 16 == 0, "swizzle must repeat over a thread's loads");
  uint32_t lane_off[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int row = ld_row + i * ROW_STRIDE;
    lane_off[i] = uint32_t(row * D + (ld_pch ^ bwd_swizzle<D>(row)) * 8) * 2u - uint32_t(i * ROW_STRIDE * D * 2);
  }
#pragma unroll
  for (int i = 0; i < NCH; ++i)
    buffer_to_lds_b128(rsrc, lane_off[i % PER], uint32_t(row0 + i * ROW_STRIDE) * uint32_t(D * 2),
                       lds_tile + uint32_t(w) * 1024u + uint32_t(i) * (NT * 16u));
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


// One step of a backward walk.
struct BwdStepInfo {
  int row0;   // first key row (dQ kernel) / first query row (dK/dV kernel) of the step
  int mode;   // effective block mode
  int pid;    // partial tile
  int blk;    // dK/dV kernel: query block of the step
  int sub;    // index of the step inside its block
  bool valid;
};

template <int D, int QB>
struct BwdDqTraits {
  static constexpr int kThreads = QB * 2;
  // keys per step: two 32-key halves whose products and vector work overlap inside a wave
  static constexpr int kStep = 64;
  static constexpr int kTileElems = kStep * D;
  // two sets of two tiles (K, V), or the output staging
  static constexpr size_t kLdsBytes = (4 * kTileElems > QB * D ? 4 * kTileElems : QB * D) * sizeof(uint16_t);
};

template <bool BF16, bool CAP, int D, int QB, int KB>
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
  uint16_t* const lds16 = reinterpret_cast<uint16_t*>(lds_raw);  // [2 sets][K, V][TILE]

  // Workgroup -> (slab, query block): XCD x takes the slabs bh with bh % n_xcd == x one after
  // the other, longest query block first, so the workgroups that run together on an XCD walk the
  // K/V rows of one or two slabs and share them through that XCD's L2.
  const int slot = blockIdx.x / p.n_xcd;
  const int xcd = blockIdx.x - slot * p.n_xcd;
  if (slot >= ((p.n_slabs - xcd + p.n_xcd - 1) / p.n_xcd) * p.Tq) return;
  const int bh = xcd + p.n_xcd * (slot / p.Tq);
  const int qb = p.Tq - 1 - slot % p.Tq;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c = lane & 31;

  // Rows at or beyond the sequence are never used: the resources of K and V end there (those
  // rows arrive as zeros) and the query rows beyond it are replaced by zeros below, whatever the
  // caller left in the padding.
  const size_t slab = size_t(bh) * size_t(p.S) * D;
  const uint32_t live_bytes = uint32_t(p.seqlen) * uint32_t(D * 2);
  const i32x4_t rK = make_buffer_resource(p.k + slab, live_bytes);
  const i32x4_t rV = make_buffer_resource(p.v + slab, live_bytes);
  const int q_row = qb * QB + 32 * w + c;
  const int q_wave_min = qb * QB + 32 * w;
  const int qr = q_row < p.S ? q_row : p.S - 1;
  const size_t meta_row = size_t(bh) * p.Tq + qb;
  const size_t meta_off = meta_row * p.max_blocks;
  const bool has_partial = p.partial_idx != nullptr && (p.partial_masks != nullptr || p.partial_bits != nullptr);

  // Block metadata in registers, as in the forward: lane i holds block 64 * chunk + i of the list.
  int32_t mv_kvb = 0, mv_info = kMasked;  // info: effective mode in the low two bits, tile index above
  auto load_chunk = [&](int chunk) {
    const int j = chunk * 64 + lane;
    const size_t o = meta_off + size_t(j < p.max_blocks ? j : 0);
    const int32_t raw = p.kv_indices[o];
    const int32_t ty = p.types[o];
    const int32_t pid = has_partial ? p.partial_idx[o] : -1;
    mv_kvb = raw < 0 ? 0 : (raw >= p.Tk ? p.Tk - 1 : raw);
    const int32_t mode = bwd_slot_mode(ty, pid, has_partial, p.num_partial);
    mv_info = (mode == kPartial ? pid << 2 : 0) | mode;
  };
  load_chunk(0);
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
      const u32x4_t none4 = {0u, 0u, 0u, 0u};
      const bool row_in = q_row < p.seqlen;
      qf[s] = row_in ? *reinterpret_cast<const u32x4_t*>(qp + 16 * s) : none4;
      dof[s] = row_in ? *reinterpret_cast<const u32x4_t*>(dop + 16 * s) : none4;
      const u32x4_t of = row_in ? *reinterpret_cast<const u32x4_t*>(op + 16 * s) : none4;
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
  if (q_row < p.S && g == 0) {
    p.ws[size_t(bh) * p.S + q_row] = -delta;
    // The dK/dV kernel starts the accumulator of a row's scores at -LSE * sqrt(D), so that the
    // exponent of a weight is the score times log2(e) / sqrt(D) and nothing else (-inf: every
    // weight of the row is 0).  A soft-capped score is not linear in the product: there the
    // plane holds the offset itself.
    p.ws[size_t(p.n_slabs) * p.S + size_t(bh) * p.S + q_row] =
        CAP ? lse2 : (row_live ? -lse * SqrtOf<D>::value : -INFINITY);
  }

  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16_t dq[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) dq[dt] = zero16;

  // The steps of the walk in order, skipping what contributes nothing: MASKED slots, keys at or
  // beyond the sequence, CAUSAL steps entirely above the diagonal of this query block.
  // Inside a KV block the next step is the previous one moved on by STEP keys (both reasons to
  // skip a step only get truer with the key index, so a block's steps are a prefix of it): that
  // path is a handful of scalar instructions; the slots of the list are only read at the first
  // step of a block.
  int gj = 0;  // next slot of the list to look at
  BwdStepInfo g_last = {0, kMasked, -1, 0, 0, false};
  const int q_last = qb * QB + QB - 1;
  auto next_step = [&]() {
    if (g_last.valid) {
      const int r = g_last.row0 + STEP, sb = g_last.sub + 1;
      const bool inside = bool(int(sb < SPB) & int(r < p.seqlen) & int(!(g_last.mode == kCausal && r > q_last)));
      if (inside) {
        g_last.row0 = r;
        g_last.sub = sb;
        return g_last;
      }
    }
    g_last.valid = false;
    while (gj < nb) {
      if ((gj & 63) == 0 && gj > 0) load_chunk(gj >> 6);
      const int ln = gj & 63;
      const int kvb = __builtin_amdgcn_readlane(mv_kvb, ln);
      const int info = __builtin_amdgcn_readlane(mv_info, ln);
      const int mode = info & 3, pid = info >> 2;
      ++gj;
      const int row0 = kvb * KB;
      if (mode == kMasked || row0 >= p.seqlen || (mode == kCausal && row0 > q_last)) continue;
      g_last.row0 = row0;
      g_last.mode = mode;
      g_last.pid = pid;
      g_last.sub = 0;
      g_last.valid = true;
      break;
    }
    return g_last;
  };
  const uint32_t lds_tiles = lds_offset_of(lds16);
  auto issue_loads = [&](const BwdStepInfo& st, int set) {
    const uint32_t base = lds_tiles + uint32_t(set) * (2u * TILE * 2u);
    bwd_load_tile<D, NT, STEP>(rK, st.row0, base, tid, w);
    bwd_load_tile<D, NT, STEP>(rV, st.row0, base + TILE * 2u, tid, w);
  };
  const uint32_t row_lane = bwd_row_lane<D>(g, c);
  const uint32_t tr_lo = bwd_tr_lane<D>(g, c, 0);
  // One step, as one sequence of slots -- first the products S^T = K.Q^T and dP^T = V.dO^T of the
  // 32-key halves (lane = query row, registers = keys; the two products of a k-step alternate),
  // then the products dQ^T += K^T.dS^T of the halves -- each slot one MFMA, the LDS fetch of the
  // operand three slots ahead and a share of the vector work of the half whose first products
  // have just finished: dS^T = P^T (dP^T - delta), packed to 16 bits in the order the last
  // product reads it, is computed for half u under the first products of half u + 1 (or under the
  // last products of half 0).  The accumulator of S^T starts at the row's offset -LSE * sqrt(D) --
  // at -inf where the step's mask forbids the pair (`masked`, wave-uniform) -- so that a weight is
  // exp2(score * sl2); that of dP^T starts at -delta.  A soft-capped score is not linear in the
  // product: there S^T starts at zero and offset and mask are applied to the weights.
  constexpr int NSUB = NTL;
  constexpr int NTR = 2 * DT;                    // last products of a half
  constexpr int NS = NSUB * (2 * KS + NTR);      // slots of a step
  constexpr int PF = D == 128 ? 2 : 3;           // operand fetch distance in slots (registers are tight at 128)
  const float row_off = CAP ? lse2 : (row_live ? -lse * SqrtOf<D>::value : -INFINITY);
  const float neg_delta = -delta;
  auto compute = [&](int set, const uint32_t (&kw)[NTL], bool masked) {
    const uint32_t base = lds_tiles + uint32_t(set) * (2u * TILE * 2u);
    const uint32_t aK = base + row_lane, aV = aK + TILE * 2u, tK0 = base + tr_lo;
    f32x16_t st[NSUB], dp[NSUB];
    u32x4_t dsb[NSUB][2];
    auto operand = [&](auto nc) {
      constexpr int n = decltype(nc)::value;
      if constexpr (n < NSUB * 2 * KS) {
        constexpr int u = n / (2 * KS), s = (n % (2 * KS)) / 2, which = n % 2;
        return lds_b128_at(((which ? aV : aK) ^ uint32_t(32 * s)) + uint32_t(u) * (32u * D * 2u));
      } else {
        constexpr int m = n - NSUB * 2 * KS, u = m / NTR, ts = (m % NTR) / DT, dt = m % DT;
        constexpr uint32_t off = uint32_t(2 * u + ts) * (16u * D * 2u);
        return lds_tr_frag<D>(tK0, uint32_t(64 * dt), off);
      }
    };
    auto keep_bits = [&](auto uc, auto rc) {  // 0 or ~0 for register r of half u
      constexpr int u = decltype(uc)::value, r = decltype(rc)::value;
      return uint32_t(__builtin_amdgcn_sbfe(int(kw[u]), 8 * (r >> 2) + (r & 3), 1));
    };
    // the score gradients of registers r, r + 1 of half u
    auto grads = [&](auto uc, auto rc) {
      constexpr int u = decltype(uc)::value, r = decltype(rc)::value;
      float w0, w1, f0 = 1.f, f1 = 1.f;
      if constexpr (CAP) {
        bwd_weight<true>(st[u][r], row_off, p, w0, f0);
        bwd_weight<true>(st[u][r + 1], row_off, p, w1, f1);
        const uint32_t b0 = __builtin_bit_cast(uint32_t, w0) & keep_bits(uc, rc);
        const uint32_t b1 = __builtin_bit_cast(uint32_t, w1) & keep_bits(uc, IntC<r + 1>{});
        w0 = __builtin_bit_cast(float, b0) * f0;
        w1 = __builtin_bit_cast(float, b1) * f1;
      } else {
        w0 = __builtin_amdgcn_exp2f(st[u][r] * p.sl2);
        w1 = __builtin_amdgcn_exp2f(st[u][r + 1] * p.sl2);
      }
      dsb[u][r >> 3][(r & 7) >> 1] = pack2<BF16>(w0 * dp[u][r], w1 * dp[u][r + 1]);
    };
    u32x4_t opq[PF];
    static_for<PF>([&](auto nc) { opq[decltype(nc)::value] = operand(nc); });
    __builtin_amdgcn_s_setprio(1);  // products first: the other wave of the SIMD fills the gaps
    static_for<NS>([&](auto nc) {
      constexpr int n = decltype(nc)::value;
      constexpr bool first = n < NSUB * 2 * KS;
      constexpr int ch = first ? n / (2 * KS) : NSUB + (n - NSUB * 2 * KS) / NTR;  // chain of the slot
      constexpr int sl = first ? n % (2 * KS) : (n - NSUB * 2 * KS) % NTR;          // slot inside it
      constexpr int len = first ? 2 * KS : NTR;
      if constexpr (first) {
        constexpr int s = sl / 2;
        if constexpr (sl == 0) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            st[ch][r] = CAP ? 0.f : row_off;
            dp[ch][r] = neg_delta;
          }
          if constexpr (!CAP) {
            if (masked) {
              static_for<16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                const uint32_t keep = keep_bits(IntC<ch>{}, rc);
                const uint32_t bits = __builtin_bit_cast(uint32_t, float(st[ch][r]));
                st[ch][r] = __builtin_bit_cast(float, (bits & keep) | (0xff800000u & ~keep));
              });
            }
          }
        }
        if constexpr (sl % 2 == 0) {
          st[ch] = mfma_32x32x16<BF16>(opq[n % PF], qf[s], st[ch]);
        } else {
          dp[ch] = mfma_32x32x16<BF16>(opq[n % PF], dof[s], dp[ch]);
        }
      } else {
        constexpr int u = ch - NSUB, ts = sl / DT, dt = sl % DT;
        dq[dt] = mfma_32x32x16<BF16>(opq[n % PF], dsb[u][ts], dq[dt]);
      }
      if constexpr (n + PF < NS) opq[n % PF] = operand(IntC<n + PF>{});
      // the score gradients of half ch - 1 go beside the products of chain ch: 8 register pairs
      // spread over the chain's slots
      if constexpr (ch >= 1 && ch <= NSUB) {
        constexpr int lo = sl * 8 / len, hi = (sl + 1) * 8 / len;
        static_for<hi - lo>([&](auto ic) { grads(IntC<ch - 1>{}, IntC<2 * (lo + decltype(ic)::value)>{}); });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_s_setprio(0);
  };

  // Tiles of step i + 1 are loaded while step i is computed: one barrier per step.
  BwdStepInfo cur = next_step();
  int set = 0;
  if (cur.valid) issue_loads(cur, 0);
  while (cur.valid) {
    const BwdStepInfo nxt = next_step();
    // mask words of this lane's row: bit j of word t = key row0 + 32 t + j allowed
    uint32_t kw[NTL];
#pragma unroll
    for (int t = 0; t < NTL; ++t) kw[t] = 0xffffffffu;
    if (cur.mode == kPartial) {
      const int q_local = q_row - qb * QB;
#pragma unroll
      for (int t = 0; t < NTL; ++t) {
        const int kcol = cur.sub * STEP + 32 * t;
        if (p.partial_bits != nullptr) {
          kw[t] = p.partial_bits[(size_t(cur.pid) * QB + q_local) * (KB / 32) + kcol / 32];
        } else {
          const uint8_t* mp = p.partial_masks + (size_t(cur.pid) * QB + q_local) * KB + kcol;
          kw[t] = bwd_pack32(*reinterpret_cast<const u32x4_t*>(mp), *reinterpret_cast<const u32x4_t*>(mp + 16));
        }
      }
    }
    int limit = p.seqlen - 1;
    if (cur.mode == kCausal) limit = limit < q_row ? limit : q_row;
    const int lim_l = limit - cur.row0 - 4 * g;
    static_for<NTL>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      kw[t] >>= 4 * g;
      const int n = lim_l - 32 * t + 1;
      const uint32_t low = n >= 32 ? 0xffffffffu : (n <= 0 ? 0u : ((1u << (n & 31)) - 1u));
      kw[t] &= low;
    });
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this step's tiles (and mask words) have landed
    __syncthreads();                     // ... for every wave; and the other set is no longer read
    if (nxt.valid) issue_loads(nxt, set ^ 1);
    compute(set, kw, !(cur.mode == kFull && cur.row0 + STEP <= p.seqlen));
    set ^= 1;
    cur = nxt;
  }
  __syncthreads();  // tiles are dead: the staging area overlaps them
  uint16_t* stage = lds16 + size_t(w) * 32 * D;
  // (the lane number goes through an empty asm: the addresses of the epilogue are then computed
  // here and not kept in registers across the walk, where every register counts)
  int lane_out = lane;
  asm volatile("" : "+v"(lane_out));
  bwd_store_rows<BF16, D>(dq, p.scale, stage, p.dq + slab, q_wave_min, p.S, lane_out);
}

// First step of STEP query rows of query block qb that can contribute to KV block kvb: a CAUSAL
// step whose rows all lie above the block's first key contributes nothing (the dK/dV kernel starts
// a block's walk there, and never stores score gradients for the steps before it).
template <int QB, int KB, int STEP>
__device__ __forceinline__ int bwd_first_step(int mode, int kvb, int qb) {
  if (mode != kCausal) return 0;
  const int below = kvb * KB - (qb * QB + STEP - 1);  // rows of the block before the first useful step
  return below > 0 ? (below + STEP - 1) / STEP : 0;
}

template <int D, int KB>
struct BwdDkdvTraits {
  static constexpr int kKeyGroups = KB / 32;       // 32 keys per wave
  static constexpr int kRoleThreads = KB * 2;      // one wave per key group in each of the two roles
  static constexpr int kThreads = KB * 4;
  // Query rows per step.  At head_dim 128 with 128-key blocks: 64, worked as two 32-row halves
  // whose products and vector work overlap inside a wave (one workgroup of eight waves per
  // compute unit, two waves per SIMD).  Elsewhere 32, so that two workgroups share a compute
  // unit: a 64-key workgroup has four waves, and at head_dim <= 64 the products of a step are so
  // short that four waves per SIMD hide more than longer steps gain (measured at head_dim 64:
  // 64-row steps at two waves per SIMD take 1.3 x the time of 32-row steps at four).
  static constexpr int kStep = (KB == 128 && D == 128) ? 64 : 32;
  static constexpr int kSub = kStep / 32;
  static constexpr int kTileElems = kStep * D;
  // three sets of two tiles (Q, dO) -- the output staging overlaps them
  static constexpr size_t kTileBytes = size_t(6) * kTileElems * sizeof(uint16_t);
  // the weights one role hands to the other, 16-bit and in B-operand order:
  // [2 steps in flight][key group][32-row half][2][64 lanes] 16-byte words
  static constexpr size_t kHandBytes = size_t(2) * kKeyGroups * kSub * 2 * 64 * 16;
  // -delta and the exponent offsets of the rows of three steps
  static constexpr size_t kRowBytes = size_t(6) * kStep * sizeof(float);
  static constexpr size_t kFixedBytes = kTileBytes + kHandBytes + kRowBytes;
  // per 64-slot word of a slab's metadata: the bitmap of the slots that list this KV block (8
  // bytes) and mode / tile index of the first (4 bytes).  The launch asks for the words its
  // metadata needs, so small problems fit two workgroups per compute unit; metadata with more
  // words than fit is worked through in windows of kMaxBitmapWords.
  static constexpr size_t kLdsLimit = size_t(160) * 1024;
  static constexpr int kMaxBitmapWords =
      (kLdsLimit - kFixedBytes) / 12 < 4096 ? int((kLdsLimit - kFixedBytes) / 12) : 4096;
  static constexpr size_t lds_bytes(size_t bitmap_words) { return kFixedBytes + bitmap_words * 12; }
  static constexpr size_t kLdsBytes = lds_bytes(kMaxBitmapWords);
};

// Two 16-bit values of a word -> fp32 (exact).
template <bool BF16>
__device__ __forceinline__ void unpack2(uint32_t w, float& lo, float& hi) {
  if constexpr (BF16) {
    const uint32_t l = w << 16, h = w & 0xffff0000u;
    lo = __builtin_bit_cast(float, l);
    hi = __builtin_bit_cast(float, h);
  } else {
    const f16x2_t v = __builtin_bit_cast(f16x2_t, w);
    lo = float(v[0]);
    hi = float(v[1]);
  }
}

// One workgroup per KV block, two waves per 32 keys with different work, so that two waves
// share each SIMD and the vector work of one runs under the matrix work of the other:
//   the "weight" wave of a key group holds K, computes S = Q.K^T and P for a step, hands P
//   (times the soft-cap derivative factor, when capped) to its partner through LDS -- rounded to
//   16 bits, in the order the partner's product reads it -- and accumulates dV^T += dO^T.P;
//   the "gradient" wave holds V, computes dP - delta = dO.V^T - delta, and one step later
//   dS = P (dP - delta) and dK^T += Q^T.dS.
// The gradient waves run one step behind the weight waves, so one barrier per step orders
// the hand-over, the tile loads (the weight waves load Q, the gradient waves dO, one step ahead)
// and the reuse of the three tile sets.
// A step is kStep query rows.  Its products form one sequence of slots -- first products of the
// 32-row halves, then second products of the halves -- each slot one MFMA, the LDS fetch of
// the operand three slots ahead and a share of the vector work of the half whose first
// product has just finished, with a scheduling fence after each slot: the weights of half u are
// computed under the products of half u + 1 (or under the second products of half 0).
template <bool BF16, bool CAP, int D, int QB, int KB>
__global__ void __launch_bounds__(KB * 4, D == 128 ? 2 : 4) bwd_dkdv_kernel(const BwdParams p) {
  using Traits = BwdDkdvTraits<D, KB>;
  constexpr int NKG = Traits::kKeyGroups;
  constexpr int RT = Traits::kRoleThreads;
  constexpr int NW = Traits::kThreads / 64;
  constexpr int STEP = Traits::kStep;
  constexpr int NSUB = Traits::kSub;
  constexpr int NSTEPS = QB / STEP;  // steps per query block
  constexpr int KS = D / 16;         // products of a 32-row half: KS for S (or dP) ...
  constexpr int DT = D / 32;
  constexpr int NTR = 2 * DT;        // ... and as many for dV^T (or dK^T)
  constexpr int NS = 2 * NSUB * KS;  // slots of a step
  constexpr int SPC = 16 / KS;       // scores of a half whose vector work goes beside one product
  constexpr int TILE = Traits::kTileElems;
  constexpr int PF = 3 < NS ? 3 : NS;  // operand fetch distance in slots
  constexpr bool PRIO = KB == 64;      // raise the wave priority around the products (it pays
                                       // with two workgroups per compute unit)
  static_assert(NTR == KS && QB % STEP == 0 && 16 % KS == 0, "slot layout");

  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  uint16_t* const lds16 = reinterpret_cast<uint16_t*>(lds_raw);  // [3 sets][Q, dO][TILE]
  uint32_t* const sHand = reinterpret_cast<uint32_t*>(lds_raw + Traits::kTileBytes);
  float* const sNd = reinterpret_cast<float*>(lds_raw + Traits::kTileBytes + Traits::kHandBytes);  // [3 sets][STEP] -delta
  float* const sL2 = sNd + 3 * STEP;                                         // [3 sets][STEP] exponent offsets
  uint64_t* const sMatch = reinterpret_cast<uint64_t*>(sL2 + 3 * STEP);

  // Workgroup -> (slab, KV block): XCD x takes the slabs bh with bh % n_xcd == x one after the
  // other, so the workgroups that run together on an XCD read the Q and dO rows of one slab and
  // share them through that XCD's L2.
  const int slot = blockIdx.x / p.n_xcd;
  const int xcd = blockIdx.x - slot * p.n_xcd;
  if (slot >= ((p.n_slabs - xcd + p.n_xcd - 1) / p.n_xcd) * p.Tk) return;
  const int bh = xcd + p.n_xcd * (slot / p.Tk);
  const int kvb = slot % p.Tk;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool grad_role = w >= NKG;        // wave-uniform
  const int kg = grad_role ? w - NKG : w;  // key group of the wave
  const int rtid = tid - (grad_role ? RT : 0);
  const int g = lane >> 5, c = lane & 31;

  // Rows at or beyond the sequence are never read: the resources of Q and dO end there, so
  // those rows arrive as zeros whatever the caller left in them.
  const size_t slab = size_t(bh) * size_t(p.S) * D;
  const uint32_t live_bytes = uint32_t(p.seqlen) * uint32_t(D * 2);
  const i32x4_t rQ = make_buffer_resource(p.q + slab, live_bytes);
  const i32x4_t rD = make_buffer_resource(p.dout + slab, live_bytes);
  const i32x4_t rNd = make_buffer_resource(p.ws + size_t(bh) * p.S, uint32_t(p.S) * 4u);
  const i32x4_t rL2 = make_buffer_resource(p.ws + size_t(p.n_slabs) * p.S + size_t(bh) * p.S, uint32_t(p.S) * 4u);
  const int key_wave_min = kvb * KB + 32 * kg;
  const int key = key_wave_min + c;  // this lane's key row inside the slab
  const int kr = key < p.S ? key : p.S - 1;
  const bool key_live = key < p.seqlen;
  const bool has_partial = p.partial_idx != nullptr && (p.partial_masks != nullptr || p.partial_bits != nullptr);
  const size_t meta_slab = size_t(bh) * p.Tq;
  const int chunks = (p.max_blocks + 63) / 64;  // 64-slot words per query block
  const int n_words = p.Tq * chunks;
  // words of the bitmap held in LDS at a time (what the launch sized the allocation for)
  const int win_words = n_words < Traits::kMaxBitmapWords ? n_words : Traits::kMaxBitmapWords;
  int32_t* const sFirst = reinterpret_cast<int32_t*>(sMatch + win_words);

  // This lane's key as B operand: K for a weight wave, V for a gradient wave (zeros for a key
  // beyond the sequence).
  u32x4_t bop[KS];
  {
    const uint16_t* src = (grad_role ? p.v : p.k) + slab + size_t(kr) * D + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const u32x4_t val = *reinterpret_cast<const u32x4_t*>(src + 16 * s);
      bop[s] = key_live ? val : u32x4_t{0u, 0u, 0u, 0u};
    }
  }

  // The scan: which (query block, slot) pairs list this KV block (after the forward's clamping of
  // the block index) with a type the forward would visit?  One 64-bit word per query block and 64
  // slots.  Mode and tile index of a word's first match are
  // kept beside it (a list names a block once, except for duplicates and clamped indices).  The
  // words [base, end) of the slab go to entries 0 .. end - base of the window; every wave of the
  // workgroup calls this at the same point (the barriers are the workgroup's).
  auto scan_window = [&](auto scan_c, int base, int end) {
    __syncthreads();  // nobody reads the previous window any more
    // A wave takes SCAN consecutive words per pass and has the loads of all of them in flight
    // together (every slot inside the list's width is loaded; kv_num_blocks cuts afterwards).
    // The first window, scanned while few registers are live, takes four; later ones one.
    constexpr int SCAN = decltype(scan_c)::value;
    for (int word0 = base + w * SCAN; word0 < end; word0 += NW * SCAN) {
      int32_t raw[SCAN], ty[SCAN], pid[SCAN], nbv[SCAN];
#pragma unroll
      for (int u = 0; u < SCAN; ++u) {
        const int word = word0 + u < end ? word0 + u : end - 1;  // (a repeat of the last word: ignored below)
        const int qb = word / chunks, ch = word - qb * chunks;
        const int slot = ch * 64 + lane;
        const size_t o = (meta_slab + qb) * p.max_blocks + (slot < p.max_blocks ? slot : p.max_blocks - 1);
        raw[u] = p.kv_indices[o];
        ty[u] = p.types[o];
        pid[u] = has_partial ? p.partial_idx[o] : -1;
        nbv[u] = p.kv_num_blocks[meta_slab + qb];
      }
#pragma unroll
      for (int u = 0; u < SCAN; ++u) {
        const int word = word0 + u;
        if (word >= end) break;
        const int ch = word % chunks;
        const int nb = nbv[u] < 0 ? 0 : (nbv[u] > p.max_blocks ? p.max_blocks : nbv[u]);
        const int32_t idx = raw[u] < 0 ? 0 : (raw[u] >= p.Tk ? p.Tk - 1 : raw[u]);
        const int32_t mode = bwd_slot_mode(ty[u], pid[u], has_partial, p.num_partial);
        const bool hit = ch * 64 + lane < nb && idx == kvb && mode != kMasked;
        const int32_t info = (mode == kPartial ? pid[u] << 2 : 0) | mode;
        const uint64_t bits = __builtin_amdgcn_ballot_w64(hit);
        if (lane == 0) sMatch[word - base] = bits;
        if (bits != 0 && lane == __builtin_ctzll(bits)) sFirst[word - base] = info;
      }
    }
    __syncthreads();
  };

  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16_t acc[DT];  // dV^T of a weight wave, dK^T of a gradient wave
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc[dt] = zero16;

  // The walk: the matches in ascending (query block, slot) order, each as NSTEPS steps of STEP
  // query rows, skipping steps beyond the sequence and CAUSAL steps entirely above the diagonal.
  // Inside a match the next step is the previous one moved on by STEP query rows (a CAUSAL step
  // that is valid stays valid further down; only the end of the sequence can end a match early):
  // that path is a handful of scalar instructions; the bitmap is only read at the first step of a
  // match.  The generator ends at the end of the window LDS holds and goes on from there once the
  // next window has been scanned.
  int gw = -1, g_qb = 0, g_ch = -1;  // word gw = (g_qb, g_ch)
  int win_base = 0, win_end = win_words;  // the words of the slab the window holds
  scan_window(IntC<4>{}, 0, win_end);
  uint64_t gbits = 0;
  bool g_first = true;
  BwdStepInfo g_last = {0, kMasked, -1, 0, 0, false};
  auto next_step = [&]() {
    if (g_last.valid) {
      const int r = g_last.row0 + STEP, sb = g_last.sub + 1;
      if (bool(int(sb < NSTEPS) & int(r < p.seqlen))) {
        g_last.row0 = r;
        g_last.sub = sb;
        return g_last;
      }
    }
    g_last.valid = false;
    for (;;) {
      while (gbits == 0) {
        if (++gw >= win_end) return g_last;
        if (++g_ch == chunks) {
          g_ch = 0;
          ++g_qb;
        }
        const uint64_t m = sMatch[gw - win_base];
        // (readfirstlane returns a signed int: go through uint32_t so that bit 31 does not sign-extend)
        gbits = (uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(m >> 32))))) << 32) |
                uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(m)))));
        g_first = true;
      }
      int mode, pid;
      if (g_first) {
        const int32_t info = __builtin_amdgcn_readfirstlane(sFirst[gw - win_base]);
        mode = info & 3;
        pid = mode == kPartial ? info >> 2 : -1;
      } else {  // a further match in the same 64 slots
        const size_t o = (meta_slab + g_qb) * p.max_blocks + g_ch * 64 + __builtin_ctzll(gbits);
        const int32_t ty = load_uniform(p.types + o);
        pid = has_partial ? load_uniform(p.partial_idx + o) : -1;
        mode = bwd_slot_mode(ty, pid, has_partial, p.num_partial);
      }
      gbits &= gbits - 1;
      g_first = false;
      // first step of the match that contributes: CAUSAL steps entirely above the diagonal and
      // steps beyond the sequence do not
      const int sub = bwd_first_step<QB, KB, STEP>(mode, kvb, g_qb);
      const int q0 = g_qb * QB + sub * STEP;
      if (sub >= NSTEPS || q0 >= p.seqlen) continue;
      g_last.row0 = q0;
      g_last.mode = mode;
      g_last.pid = pid;
      g_last.blk = g_qb;
      g_last.sub = sub;
      g_last.valid = true;
      return g_last;
    }
  };
  const uint32_t lds_tiles = lds_offset_of(lds16);
  const uint32_t hand_lane = lds_offset_of(sHand) + uint32_t(kg) * (NSUB * 2048u) + uint32_t(lane) * 16u;
  const uint32_t lds_nd = lds_offset_of(sNd), lds_l2 = lds_offset_of(sL2);
  auto tile_at = [&](int set, int which) { return lds_tiles + uint32_t(set * 2 + which) * (TILE * 2u); };
  // the four words of half `half` of 32-row half u of the step with parity par
  auto hand_at = [&](int par, int u, int half) {
    return hand_lane + uint32_t(par) * (NKG * NSUB * 2048u) + uint32_t(u) * 2048u + uint32_t(half) * 1024u;
  };
  // The rows of step j + 1 are loaded during iteration j: Q and the exponent offsets by the
  // weight waves, dO and -delta by the gradient waves.
  auto load_q = [&](const BwdStepInfo& st, int set) {
    bwd_load_tile<D, RT, STEP>(rQ, st.row0, tile_at(set, 0), rtid, kg);
    if (rtid < STEP)
      buffer_to_lds_b32(rL2, uint32_t(rtid) * 4u, uint32_t(st.row0) * 4u, lds_l2 + uint32_t(set * STEP) * 4u);
  };
  auto load_do = [&](const BwdStepInfo& st, int set) {
    bwd_load_tile<D, RT, STEP>(rD, st.row0, tile_at(set, 1), rtid, kg);
    if (rtid < STEP)
      buffer_to_lds_b32(rNd, uint32_t(rtid) * 4u, uint32_t(st.row0) * 4u, lds_nd + uint32_t(set * STEP) * 4u);
  };
  const uint32_t row_lane = bwd_row_lane<D>(g, c);
  const uint32_t tr_lo = bwd_tr_lane<D>(g, c, 0);

  // Operand n of a step's slot sequence, from the tile read row-wise (first products: rows
  // 32 u + lane of the tile at k-step s) or transposed (second products: columns 32 dt .. +31
  // at rows 32 u + 16 ts .. +15).
  auto operand = [&](auto nc, uint32_t a_rows, uint32_t a_tr0) {
    constexpr int n = decltype(nc)::value;
    constexpr int ch = n / KS, s = n % KS;
    if constexpr (ch < NSUB) {
      return lds_b128_at((a_rows ^ uint32_t(32 * s)) + uint32_t(ch) * (32u * D * 2u));
    } else {
      constexpr int u = ch - NSUB, ts = s / DT, dt = s % DT;
      constexpr uint32_t off = uint32_t(2 * u + ts) * (16u * D * 2u);
      return lds_tr_frag<D>(a_tr0, uint32_t(64 * dt), off);
    }
  };

  // Weight wave, one step: S = Q.K^T (lane = key, registers = query rows), P, dV^T += dO^T.P.
  // The accumulator of a half's scores starts at the rows' offsets -LSE * sqrt(D) -- at -inf where
  // the step's mask (`masked`, wave-uniform: the words kw are only looked at then) forbids the
  // pair -- so a weight is exp2(score * sl2) and the mask costs nothing inside the slots.  A
  // soft-capped score is not linear in the product: there the accumulator starts at zero, the
  // offsets are fetched when the weights are computed and the mask is applied to the weights.
  auto weight_step = [&](int set, int par, const uint32_t (&kw)[NSUB], bool masked) {
    const uint32_t aQ = tile_at(set, 0) + row_lane, tD0 = tile_at(set, 1) + tr_lo;
    // The row offsets of the workspace: registers 4 i .. +3 of a half are its query rows
    // 8 i + 4 g .. +3.
    auto row_offsets = [&](int u, int i4) {
      return lds_f32x4_at(lds_l2 + uint32_t(set * STEP + 32 * u + 8 * i4) * 4u + 16u * g);
    };
    // 0 or ~0: may register r of half u keep its value?  (kw is already shifted by 4 g: bit
    // 8 (r / 4) + r % 4 is the row of register r)
    auto keep_bits = [&](auto uc, auto rc) {
      constexpr int u = decltype(uc)::value, r = decltype(rc)::value;
      return uint32_t(__builtin_amdgcn_sbfe(int(kw[u]), 8 * (r >> 2) + (r & 3), 1));
    };
    f32x16_t sc[NSUB];
    u32x4_t pb[NSUB][2];   // P packed to 16 bits, B-operand order
    u32x4_t hb[NSUB][2];   // what the partner gets when capped: P times the soft-cap factor
    f32x4_t lq = {0.f, 0.f, 0.f, 0.f};
    auto weights = [&](auto uc, auto ic) {
      constexpr int u = decltype(uc)::value, i = decltype(ic)::value;
      static_for<SPC / 2>([&](auto jc) {
        constexpr int r = SPC * i + 2 * decltype(jc)::value;
        float w0, w1;
        if constexpr (CAP) {
          float f0, f1;
          if constexpr ((r & 3) == 0) lq = row_offsets(u, r >> 2);
          bwd_weight<true>(sc[u][r], lq[r & 3], p, w0, f0);
          bwd_weight<true>(sc[u][r + 1], lq[(r + 1) & 3], p, w1, f1);
          const uint32_t b0 = __builtin_bit_cast(uint32_t, w0) & keep_bits(uc, IntC<r>{});
          const uint32_t b1 = __builtin_bit_cast(uint32_t, w1) & keep_bits(uc, IntC<r + 1>{});
          w0 = __builtin_bit_cast(float, b0);
          w1 = __builtin_bit_cast(float, b1);
          hb[u][r >> 3][(r & 7) >> 1] = pack2<BF16>(w0 * f0, w1 * f1);
        } else {  // the scores already carry their row's offset and the mask
          w0 = __builtin_amdgcn_exp2f(sc[u][r] * p.sl2);
          w1 = __builtin_amdgcn_exp2f(sc[u][r + 1] * p.sl2);
        }
        pb[u][r >> 3][(r & 7) >> 1] = pack2<BF16>(w0, w1);
      });
      if constexpr (((i + 1) * SPC) % 8 == 0) {  // four words are complete: to the partner
        constexpr int half = (i + 1) * SPC / 8 - 1;
        if constexpr (CAP) {
          *(__attribute__((address_space(3))) u32x4_t*)(hand_at(par, u, half)) = hb[u][half];
        } else {
          *(__attribute__((address_space(3))) u32x4_t*)(hand_at(par, u, half)) = pb[u][half];
        }
      }
    };
    u32x4_t opq[PF];
    static_for<PF>([&](auto nc) { opq[decltype(nc)::value] = operand(nc, aQ, tD0); });
    if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
    static_for<NS>([&](auto nc) {
      constexpr int n = decltype(nc)::value;
      constexpr int ch = n / KS, s = n % KS;
      if constexpr (ch < NSUB) {
        if constexpr (s == 0) {
          if constexpr (CAP) {
            sc[ch] = zero16;
          } else {
            static_for<4>([&](auto ic) {
              constexpr int i4 = decltype(ic)::value;
              const f32x4_t o4 = row_offsets(ch, i4);
              sc[ch][4 * i4 + 0] = o4[0];
              sc[ch][4 * i4 + 1] = o4[1];
              sc[ch][4 * i4 + 2] = o4[2];
              sc[ch][4 * i4 + 3] = o4[3];
            });
            if (masked) {
              static_for<16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                const uint32_t keep = keep_bits(IntC<ch>{}, rc);
                const uint32_t bits = __builtin_bit_cast(uint32_t, float(sc[ch][r]));
                sc[ch][r] = __builtin_bit_cast(float, (bits & keep) | (0xff800000u & ~keep));
              });
            }
          }
        }
        sc[ch] = mfma_32x32x16<BF16>(opq[n % PF], bop[s], sc[ch]);
      } else {
        constexpr int u = ch - NSUB, ts = s / DT, dt = s % DT;
        acc[dt] = mfma_32x32x16<BF16>(opq[n % PF], pb[u][ts], acc[dt]);
      }
      if constexpr (n + PF < NS) opq[n % PF] = operand(IntC<n + PF>{}, aQ, tD0);
      // the weights of half ch - 1 go beside the products of chain ch
      if constexpr (NSUB > 1 && ch >= 1 && ch <= NSUB) weights(IntC<ch - 1>{}, IntC<s>{});
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (NSUB == 1 && n == KS - 1) {  // a one-half step: nothing to put them under
        if constexpr (PRIO) __builtin_amdgcn_s_setprio(0);
        static_for<KS>([&](auto ic) { weights(IntC<0>{}, ic); });
        if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    if constexpr (PRIO) __builtin_amdgcn_s_setprio(0);
  };
  // Gradient wave, one step: dP - delta = dO.V^T - delta (the accumulator starts at -delta),
  // dS = P (dP - delta) with the partner's P, dK^T += Q^T.dS.
  auto grad_step = [&](int set, int par) {
    const uint32_t aD = tile_at(set, 1) + row_lane, tQ0 = tile_at(set, 0) + tr_lo;
    f32x16_t dp[NSUB];
    u32x4_t hand[NSUB][2], dsb[NSUB][2];
    static_for<4 * NSUB>([&](auto ic) {
      constexpr int u = decltype(ic)::value / 4, i4 = decltype(ic)::value % 4;
      const f32x4_t nd = lds_f32x4_at(lds_nd + uint32_t(set * STEP + 32 * u + 8 * i4) * 4u + 16u * g);
      dp[u][4 * i4 + 0] = nd[0];
      dp[u][4 * i4 + 1] = nd[1];
      dp[u][4 * i4 + 2] = nd[2];
      dp[u][4 * i4 + 3] = nd[3];
    });
    auto score_grads = [&](auto uc, auto ic) {
      constexpr int u = decltype(uc)::value, i = decltype(ic)::value;
      static_for<SPC / 2>([&](auto jc) {
        constexpr int r = SPC * i + 2 * decltype(jc)::value;
        float h0, h1;
        unpack2<BF16>(hand[u][r >> 3][(r & 7) >> 1], h0, h1);
        dsb[u][r >> 3][(r & 7) >> 1] = pack2<BF16>(h0 * dp[u][r], h1 * dp[u][r + 1]);
      });
    };
    u32x4_t opq[PF];
    static_for<PF>([&](auto nc) { opq[decltype(nc)::value] = operand(nc, aD, tQ0); });
    if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
    static_for<NS>([&](auto nc) {
      constexpr int n = decltype(nc)::value;
      constexpr int ch = n / KS, s = n % KS;
      if constexpr (ch < NSUB) {
        if constexpr (s == 0) {
          hand[ch][0] = lds_b128_at(hand_at(par, ch, 0));
          hand[ch][1] = lds_b128_at(hand_at(par, ch, 1));
        }
        dp[ch] = mfma_32x32x16<BF16>(opq[n % PF], bop[s], dp[ch]);
      } else {
        constexpr int u = ch - NSUB, ts = s / DT, dt = s % DT;
        acc[dt] = mfma_32x32x16<BF16>(opq[n % PF], dsb[u][ts], acc[dt]);
      }
      if constexpr (n + PF < NS) opq[n % PF] = operand(IntC<n + PF>{}, aD, tQ0);
      if constexpr (NSUB > 1 && ch >= 1 && ch <= NSUB) score_grads(IntC<ch - 1>{}, IntC<s>{});
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (NSUB == 1 && n == KS - 1) {
        if constexpr (PRIO) __builtin_amdgcn_s_setprio(0);
        static_for<KS>([&](auto ic) { score_grads(IntC<0>{}, ic); });
        if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    if constexpr (PRIO) __builtin_amdgcn_s_setprio(0);
  };

  // Bits of one partial tile for this lane's key: bit j = query row q_local0 + j of the tile
  // attends the key.  Lane j of the wave fetches the 32 key bits of row j; the column of this
  // lane's key is then collected from the 32 rows.
  auto partial_column = [&](int pid, int q_local0) {
    const int rl = lane & 31;
    uint32_t roww;
    if (p.partial_bits != nullptr) {
      roww = p.partial_bits[(size_t(pid) * QB + q_local0 + rl) * (KB / 32) + kg];
    } else {
      const uint8_t* mp = p.partial_masks + (size_t(pid) * QB + q_local0 + rl) * KB + 32 * kg;
      roww = bwd_pack32(*reinterpret_cast<const u32x4_t*>(mp), *reinterpret_cast<const u32x4_t*>(mp + 16));
    }
    uint32_t col = 0;
    static_for<32>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      const uint32_t r = uint32_t(__builtin_amdgcn_readlane(int(roww), j));
      col |= ((r >> c) & 1u) << j;
    });
    return col;
  };

  // Iteration j: the weight waves do step j, the gradient waves step j - 1.  The two roles
  // run separate copies of the loop (same trip count, one barrier per trip), so that each keeps
  // its accumulators in place.  Metadata of more words than the bitmap holds takes several
  // windows: the steps of a window are worked off completely before the next one is scanned.
  auto run = [&](auto role_c) {
    constexpr bool GRAD = decltype(role_c)::value;
    const BwdStepInfo none = {0, kMasked, -1, 0, 0, false};
    for (;;) {
      BwdStepInfo prev = none, cur = next_step();
      int s_prev = 2, s_cur = 0, s_nxt = 1;  // tile sets of steps j - 1, j, j + 1
      if (cur.valid) {
        if constexpr (!GRAD) load_q(cur, 0); else load_do(cur, 0);
      }
      for (int j = 0; cur.valid || prev.valid; ++j) {
        const BwdStepInfo nxt = cur.valid ? next_step() : none;
        // mask words of this lane's key: bit i of word u = query row row0 + 32 u + i attends it
        uint32_t kw[NSUB];
  #pragma unroll
        for (int u = 0; u < NSUB; ++u) kw[u] = 0;
        if constexpr (!GRAD) {
          if (cur.valid) {
  #pragma unroll
            for (int u = 0; u < NSUB; ++u) {
              uint32_t m = key_live ? 0xffffffffu : 0u;
              if (cur.mode == kCausal) {  // rows at or after the key
                const int n = key - (cur.row0 + 32 * u);
                m &= n <= 0 ? 0xffffffffu : (n >= 32 ? 0u : (0xffffffffu << (n & 31)));
              }
              if (cur.mode == kPartial) m &= partial_column(cur.pid, cur.row0 + 32 * u - cur.blk * QB);
              kw[u] = m >> (4 * g);
            }
          }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the tile this wave loaded has landed
        __syncthreads();  // ... everybody's have; the hand-over of step j - 1 is written; the set
                          // about to be overwritten (step j - 2) is no longer read
        if constexpr (!GRAD) {
          if (nxt.valid) load_q(nxt, s_nxt);
          if (cur.valid) {
            // (wave-uniform) a FULL step whose keys are all inside the sequence needs no mask
            weight_step(s_cur, j & 1, kw, !(cur.mode == kFull && key_wave_min + 32 <= p.seqlen));
          }
        } else {
          if (nxt.valid) load_do(nxt, s_nxt);
          if (prev.valid) grad_step(s_prev, (j + 1) & 1);
        }
        prev = cur;
        cur = nxt;
        const int t3 = s_prev;
        s_prev = s_cur;
        s_cur = s_nxt;
        s_nxt = t3;
      }
      if (__builtin_expect(win_end >= n_words, 1)) break;
      // (rare) more words of metadata than the bitmap holds: the next window
      win_base = win_end;
      win_end = win_base + win_words < n_words ? win_base + win_words : n_words;
      scan_window(IntC<1>{}, win_base, win_end);
      gw = win_base - 1;
    }
    __syncthreads();
    uint16_t* stage = lds16 + size_t(w) * 32 * D;
    if constexpr (!GRAD) {
      bwd_store_rows<BF16, D>(acc, 1.f, stage, p.dv + slab, key_wave_min, p.S, lane);
    } else {
      bwd_store_rows<BF16, D>(acc, p.scale, stage, p.dk + slab, key_wave_min, p.S, lane);
    }
  };
  if (grad_role) {
    run(std::integral_constant<bool, true>{});
  } else {
    run(std::integral_constant<bool, false>{});
  }
}

constexpr int kBwdMaxDevices = 64;

template <bool BF16, bool CAP, int D, int QB, int KB>
int launch_bwd_cap(const BwdParams& p, hipStream_t stream) {
  using TQ = BwdDqTraits<D, QB>;
  using TK = BwdDkdvTraits<D, KB>;
  auto kq = bwd_dq_kernel<BF16, CAP, D, QB, KB>;
  auto kk = bwd_dkdv_kernel<BF16, CAP, D, QB, KB>;
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
  const unsigned slabs_per_xcd = unsigned(p.n_slabs + p.n_xcd - 1) / unsigned(p.n_xcd);
  BwdParams params = p;
  void* args[] = {&params};
  const size_t n_words = size_t(p.Tq) * size_t((p.max_blocks + 63) / 64);
  const size_t dkdv_lds = TK::lds_bytes(n_words < size_t(TK::kMaxBitmapWords) ? n_words : size_t(TK::kMaxBitmapWords));
  const dim3 dkdv_grid(unsigned(p.n_xcd) * slabs_per_xcd * unsigned(p.Tk));
  const dim3 dq_grid(unsigned(p.n_xcd) * slabs_per_xcd * unsigned(p.Tq));
  e = hipLaunchKernel(reinterpret_cast<const void*>(kq), dq_grid, dim3(TQ::kThreads), args, TQ::kLdsBytes, stream);
  if (e != hipSuccess) return int(e);
  e = hipLaunchKernel(reinterpret_cast<const void*>(kk), dkdv_grid, dim3(TK::kThreads), args, dkdv_lds, stream);
  return int(e);
}

// The soft-capped instances are separate kernels: the extra arithmetic per score would
// otherwise cost the plain ones registers.
template <bool BF16, int D, int QB, int KB>
int launch_bwd(const BwdParams& p, hipStream_t stream) {
  return p.softcap > 0.f ? launch_bwd_cap<BF16, true, D, QB, KB>(p, stream)
                         : launch_bwd_cap<BF16, false, D, QB, KB>(p, stream);
}

}  // namespace omni_attn

// Block-sparse FlashAttention-2 forward for gfx950 (MI355X, CDNA4).
//
// One workgroup owns one query block (QB rows) of one (batch, head) and walks only
// the KV blocks listed for it, like the reference's per-Q-block CTA
// (omni-attn-mma/mma/omni_attn_shared_kv.cu:33-647); the mask semantics are those of
// the reference's scalar kernel (omni-attn-mma/mma/attn_naive.cu:21-302).
//
// Everything is computed transposed so that one lane owns one query row:
//   S^T[kv, q] = K[kv, :] . Q[q, :]      A = K tile (LDS), B = Q (registers)
//   O^T[d,  q] = V^T[d, kv] . P^T[kv, q]  A = V^T (LDS transpose read), B = P^T
// With v_mfma_f32_32x32x16 the accumulator of S^T puts query row (lane % 32) in a
// lane and 16 kv positions in its registers, which is exactly the B-operand layout
// the second product needs: P never leaves registers, row max / row sum are in-lane
// reductions plus one exchange with lane ^ 32, and the online-softmax rescale is a
// per-lane scalar.
//
// A wave owns 32 query rows; a workgroup has QB/32 waves.  KV blocks are consumed in
// steps of 64 keys (a 128-key block is two steps).  K and V tiles are double-buffered
// in LDS and filled by direct global->LDS loads (no register staging); the K tile runs
// one step ahead of the V tile so that S^T of step i+1 is issued to the matrix cores
// before the softmax of step i runs on the vector ALU.  One workgroup barrier per step.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace omni_attn {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

enum : int { kMasked = 0, kCausal = 1, kFull = 2, kPartial = 3 };

struct FwdParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* o;
  float* lse;                    // may be null
  const int32_t* kv_num_blocks;  // [B,H,Tq]
  const int32_t* kv_indices;     // [B,H,Tq,max_blocks]
  const int32_t* types;          // [B,H,Tq,max_blocks]
  const int32_t* partial_idx;    // [B,H,Tq,max_blocks] or null
  const uint8_t* partial_masks;  // [P,QB,KB] bytes or null
  int S;           // padded sequence length (rows per (b,h) slab)
  int Tq;          // query blocks per slab
  int Tk;          // ceil(S / KB)
  int max_blocks;  // slots per query block
  int seqlen;      // min(seqlen_orig, S): rows/keys at or beyond it are padding
  int n_slabs;     // B*H
  int slab_group;  // slabs of one XCD that are walked together (>= 1)
  float sl2;       // log2(e) / sqrt(D)
};

template <bool BF16>
__device__ __forceinline__ f32x16_t mfma_32x32x16(u32x4_t a, u32x4_t b, f32x16_t c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
}

// Two fp32 values -> two 16-bit values (round to nearest even), low half first.
template <bool BF16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (BF16) {
    bf16x2_t v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  } else {
    f16x2_t v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
}

// LDS tiles are [64 rows][D] 16-bit elements with no padding; 16-byte chunks are
// XOR-swizzled inside a row so that the operand reads are bank-conflict free.
// K is read with ds_read_b128 by 32 consecutive rows at one chunk column: the chunk
// index is XORed with the row so 16 consecutive rows cover all 64 banks.
template <int D>
__device__ __forceinline__ int k_swizzle(int row) {
  constexpr int C = D / 8;  // 16-byte chunks per row
  return (row / (16 / C)) % C;
}
// V is read with ds_read_b64_tr_b16: within 16 lanes, 4 lanes read 32 contiguous bytes
// of one row and the next 4 lanes the next row; lanes 16-31 read the neighbouring 32-byte
// unit of the same 4 rows.  Bit 0 of the unit index (which half-wave group) is left
// alone and the higher bits are XORed with the row, so the 32 lanes that are served
// together touch 8 different 32-byte bank groups.
template <int D>
__device__ __forceinline__ int v_swizzle(int row) {
  constexpr int U = D / 16;  // 32-byte units per row
  if constexpr (U <= 2) return 0;
  return 2 * ((row / (8 / U)) % (U / 2));
}

__device__ __forceinline__ s16x4_t lds_read_tr16(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s16x4_t*)(p));
}

// Exchange between the lane pair (l, l ^ 32) without touching LDS: v_permlane32_swap
// swaps the upper 32 lanes of its first operand with the lower 32 lanes of its second,
// so with x in both operands one result holds {lo, lo} and the other {hi, hi}.
// (The elements are copied to scalars before the bit cast: a bit cast applied directly
// to a vector element expression reads element 0 for both.)
__device__ __forceinline__ void pair_split(float x, float& lo, float& hi) {
  typedef __attribute__((ext_vector_type(2))) unsigned u2;
  const unsigned a = __builtin_bit_cast(unsigned, x);
  const u2 r = __builtin_amdgcn_permlane32_swap(a, a, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  lo = __builtin_bit_cast(float, r0);
  hi = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float pair_max(float x) {
  float lo, hi;
  pair_split(x, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float pair_sum(float x) {
  float lo, hi;
  pair_split(x, lo, hi);
  return lo + hi;
}

template <bool BF16, int D, int QB, int KB>
struct FwdTraits {
  static constexpr int kThreads = QB * 2;  // QB/32 waves of 64 lanes
  static constexpr int kStep = 64;
  static constexpr int kTileElems = kStep * D;
  static constexpr size_t kLdsBytes =
      size_t(2) * 2 * kTileElems * sizeof(uint16_t) + size_t(QB) * 2 * sizeof(uint32_t);
};

// One step of the walk: 64 keys starting at row0, with the effective block mode.
struct StepInfo {
  int row0;
  int mode;
  int pid;
};
// The metadata words of a step as loaded; interpreted one iteration later so that no
// instruction waits on a metadata load it has just issued.
struct RawStep {
  int kvb;
  int ty;
  int pid;
};

typedef __attribute__((address_space(3))) void lds_void_t;

// 16 bytes per lane from global memory straight into LDS: the wave's 64 chunks land at
// lds_base + 16 * lane.  The global address is a wave-uniform 64-bit base plus a per-lane
// 32-bit byte offset.  Written as inline asm so that the compiler does not order later
// LDS reads of *other* buffers behind it with a vmcnt(0) wait; completion is waited for
// explicitly (vmcnt(0) + workgroup barrier) before the filled buffer is read.
__device__ __forceinline__ void global_to_lds_b128(const void* gbase_uniform, uint32_t byte_off,
                                                   uint32_t lds_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(lds_base), "v"(byte_off), "s"(gbase_uniform)
      : "memory", "m0");
}
// Block-mask metadata is read-only for the whole launch and every read of it is
// wave-uniform: reading it through the constant address space makes these scalar loads
// (SGPR results, no vector-memory latency in the instruction stream).
__device__ __forceinline__ int32_t load_uniform(const int32_t* p) {
  return *reinterpret_cast<const __attribute__((address_space(4))) int32_t*>(
      reinterpret_cast<size_t>(p));
}
__device__ __forceinline__ uint32_t lds_offset_of(const void* p) {
  return uint32_t(size_t((lds_void_t*)p));
}

template <bool BF16, int D, int QB, int KB>
__global__ void __launch_bounds__(QB * 2, 2) fwd_kernel(const FwdParams p) {
  using Traits = FwdTraits<BF16, D, QB, KB>;
  constexpr int NT = Traits::kThreads;
  constexpr int STEP = Traits::kStep;
  constexpr int SPB = KB / STEP;        // steps per KV block
  constexpr int CPR = D / 8;            // 16-byte chunks per row
  constexpr int NCH = STEP * CPR / NT;  // 16-byte chunks per thread per tile
  constexpr int KS = D / 16;            // MFMA k-steps of Q.K
  constexpr int DT = D / 32;            // 32-row tiles of O^T
  constexpr int TILE = Traits::kTileElems;
  static_assert(STEP * CPR % NT == 0, "tile must divide over the workgroup");

  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  uint16_t* sK = reinterpret_cast<uint16_t*>(lds_raw);           // [2][TILE]
  uint16_t* sV = sK + 2 * TILE;                                  // [2][TILE]
  uint32_t* sBits = reinterpret_cast<uint32_t*>(sV + 2 * TILE);  // [QB*2]

  // Workgroup -> (slab, query block).  Consecutive workgroup ids go round-robin over
  // the 8 XCDs.  XCD x takes the slabs bh with bh % 8 == x (every batch element's heads
  // are spread over all XCDs, which balances batches with different masks) and works
  // through them in groups of p.slab_group slabs, sized so that one group's query
  // blocks just fill the XCD's workgroup slots: the workgroups that run together then
  // belong to one or two slabs and walk the same K/V rows at about the same time, so
  // each K/V tile is fetched from HBM once and served from the XCD's L2 to the other
  // query blocks.  Inside a group the order is longest-first: query block Tq-1 of each
  // slab of the group, then Tq-2, ...
  const int wg = blockIdx.x;
  const int xcd = wg & 7;
  const int slot = wg >> 3;
  const int slabs_here = (p.n_slabs - xcd + 7) >> 3;
  if (slot >= slabs_here * p.Tq) return;
  const int per_group = p.slab_group * p.Tq;
  const int gi = slot / per_group;
  const int in_group = slot - gi * per_group;
  const int g_left = slabs_here - gi * p.slab_group;
  const int g_eff = g_left < p.slab_group ? g_left : p.slab_group;
  const int qrank = in_group / g_eff;
  const int bh = xcd + 8 * (gi * p.slab_group + (in_group - qrank * g_eff));
  const int qb = p.Tq - 1 - qrank;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int c = lane & 31;

  const size_t slab = size_t(bh) * size_t(p.S) * D;
  const uint16_t* __restrict__ gK = p.k + slab;
  const uint16_t* __restrict__ gV = p.v + slab;

  const int q_row = qb * QB + 32 * w + c;  // this lane's query row inside the slab
  const int q_wave_min = qb * QB + 32 * w;

  // Q as the B operand of S^T = K.Q^T: lane holds Q[q_row][16s + 8g .. +7].
  u32x4_t qf[KS];
  {
    const int qr = q_row < p.S ? q_row : p.S - 1;
    const uint16_t* qp = p.q + slab + size_t(qr) * D + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const u32x4_t*>(qp + 16 * s);
  }

  const size_t meta_row = size_t(bh) * p.Tq + qb;
  const size_t meta_off = meta_row * p.max_blocks;
  int nb = load_uniform(p.kv_num_blocks + meta_row);
  nb = nb < 0 ? 0 : (nb > p.max_blocks ? p.max_blocks : nb);
  const int nsteps = nb * SPB;

  // Metadata of step `it`: issue the (scalar) loads ...
  const bool has_partial = p.partial_idx != nullptr && p.partial_masks != nullptr;
  auto fetch_raw = [&](int it) {
    RawStep r = {0, kMasked, -1};
    if (it < nsteps) {
      const int j = it / SPB;
      r.kvb = load_uniform(p.kv_indices + meta_off + j);
      r.ty = load_uniform(p.types + meta_off + j);
      if (has_partial) r.pid = load_uniform(p.partial_idx + meta_off + j);
    }
    return r;
  };
  // ... and interpret them: first key row, effective mode, partial-mask index.
  auto interpret = [&](int it, const RawStep& r) {
    StepInfo si;
    const int half = it % SPB;
    const int kvb = r.kvb < 0 ? 0 : (r.kvb >= p.Tk ? p.Tk - 1 : r.kvb);
    si.mode = (r.ty == kCausal || r.ty == kFull || r.ty == kPartial) ? r.ty : kMasked;
    si.pid = r.pid;
    if (r.ty == kPartial && r.pid < 0) si.mode = kMasked;
    si.row0 = kvb * KB + half * STEP;
    return si;
  };

  // Direct global->LDS tile load: every lane fetches 16 bytes, the wave's 64 chunks land
  // at consecutive LDS addresses: one wave-wide load fills 64 / CPR rows of the tile.
  // The swizzle is applied on the global side: the lane that fills physical chunk
  // (row, pch) fetches the logical chunk that belongs there.  The swizzle only depends
  // on row modulo 16 (at most) and the loads of one thread are a multiple of 16 rows
  // apart in every configuration except (QB=64, D=128), so one per-lane byte offset
  // serves all loads of a thread and the rest of the address is wave-uniform.  A tile
  // that would run past the last row of the slab clamps its rows instead.
  constexpr int ROWS_PER_CALL = 64 / CPR;           // rows filled by one wave-wide load
  constexpr int ROW_STRIDE = ROWS_PER_CALL * (NT / 64);  // rows between a thread's loads
  constexpr bool kUniformSwizzle = ROW_STRIDE % 16 == 0;
  const int ld_row = tid / CPR;  // row of this thread's first load
  const int ld_pch = tid % CPR;
  auto k_off = [&](int row) { return uint32_t(row * D + (ld_pch ^ k_swizzle<D>(row)) * 8) * 2u; };
  auto v_off = [&](int row) {
    return uint32_t(row * D + ((((ld_pch >> 1) ^ v_swizzle<D>(row)) << 1) | (ld_pch & 1)) * 8) * 2u;
  };
  const uint32_t koff0 = k_off(ld_row), voff0 = v_off(ld_row);
  const uint32_t lds_k0 = lds_offset_of(sK) + uint32_t(w) * 1024u;
  const uint32_t lds_v0 = lds_offset_of(sV) + uint32_t(w) * 1024u;
  auto issue_tile = [&](const uint16_t* gsrc, bool is_v, uint32_t lds0, int buf, int kv_row0) {
    const uint32_t dst = lds0 + uint32_t(buf) * (TILE * 2u);
    const uint32_t off0 = is_v ? voff0 : koff0;
    if (kv_row0 + STEP <= p.S) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        uint32_t off = off0;
        if constexpr (!kUniformSwizzle) {
          const int row = ld_row + i * ROW_STRIDE;
          off = (is_v ? v_off(row) : k_off(row)) - uint32_t(i * ROW_STRIDE * D * 2);
        }
        global_to_lds_b128(gsrc + size_t(kv_row0 + i * ROW_STRIDE) * D, off,
                           dst + uint32_t(i) * (NT * 16u));
      }
    } else {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int row = ld_row + i * ROW_STRIDE;
        int gr = kv_row0 + row;
        gr = gr < p.S ? gr : p.S - 1;
        const uint32_t off = (is_v ? v_off(row) : k_off(row)) - uint32_t(row * D * 2);
        global_to_lds_b128(gsrc, off + uint32_t(gr) * (D * 2u), dst + uint32_t(i) * (NT * 16u));
      }
    }
  };
  auto issue_k = [&](int buf, int kv_row0) { issue_tile(gK, false, lds_k0, buf, kv_row0); };
  auto issue_v = [&](int buf, int kv_row0) { issue_tile(gV, true, lds_v0, buf, kv_row0); };

  // PARTIAL blocks: thread tid fetches 32 mask bytes of row tid/2 (a row of its own
  // wave), packs them to 32 bits and parks the word in LDS for the two lanes that own
  // the row.  Writer and readers are the same wave, so no workgroup barrier is needed.
  // Done at the top of the step that needs it: no registers are held across steps for
  // it, at the price of one exposed load latency per PARTIAL step.
  auto stage_mask_bits = [&](int it, const StepInfo& si) {
    const int half = it % SPB;
    const uint8_t* mp = p.partial_masks + size_t(si.pid) * (QB * KB) + size_t(tid >> 1) * KB +
                        half * STEP + (tid & 1) * 32;
    const u32x4_t m0 = *reinterpret_cast<const u32x4_t*>(mp);
    const u32x4_t m1 = *reinterpret_cast<const u32x4_t*>(mp + 16);
    uint32_t word = 0;  // byte i (0 or 1) of the 32 -> bit i
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t bytes = i < 4 ? m0[i] : m1[i - 4];
      const uint32_t nib = ((bytes & 0x01010101u) * 0x01020408u) >> 24;
      word |= nib << (4 * i);
    }
    sBits[tid] = word;
  };

  // Wave-uniform classification of this wave's 32x64 tile of a step:
  // 0 = nothing to do, 1 = no mask needed, 2 = masked path.
  auto classify = [&](const StepInfo& si) {
    if (si.mode == kMasked) return 0;
    const bool clip = si.row0 + STEP > p.seqlen;
    if (si.mode == kCausal) {
      if (si.row0 > q_wave_min + 31) return 0;                       // all in the future
      if (si.row0 + STEP - 1 <= q_wave_min && !clip) return 1;       // all in the past
      return 2;
    }
    return (si.mode == kFull && !clip) ? 1 : 2;
  };

  // S^T = K . Q^T for the 64 keys of one LDS tile: two 32-key accumulator tiles.
  auto qk_tile = [&](const uint16_t* tK, f32x16_t (&st)[2]) {
    const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int row = 32 * t + c;
        const int ch = (2 * s + g) ^ k_swizzle<D>(row);
        const u32x4_t a = *reinterpret_cast<const u32x4_t*>(tK + row * D + ch * 8);
        st[t] = mfma_32x32x16<BF16>(a, qf[s], s == 0 ? zero : st[t]);
      }
    }
  };

  f32x16_t ot[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) ot[dt][r] = 0.f;
  float m_run = -INFINITY;  // reference point of the exponentials, log2 domain (score * sl2)
  float l_run = 0.f;        // this lane's share of the running row sum

  // Mask (if needed) + online softmax of one step; leaves P (fp32) in st.
  auto softmax_step = [&](f32x16_t (&st)[2], const StepInfo& si, bool masked_path) {
    if (masked_path) {
      // Register r of tile t holds key  row0 + 32t + 8(r/4) + 4g + r%4.
      int limit = p.seqlen - 1;
      if (si.mode == kCausal) limit = limit < q_row ? limit : q_row;
      const int lim_l = limit - si.row0 - 4 * g;
      uint32_t kw0 = 0xffffffffu, kw1 = 0xffffffffu;
      if (si.mode == kPartial) {
        const u32x2_t bw = *reinterpret_cast<const u32x2_t*>(sBits + (32 * w + c) * 2);
        kw0 = bw[0];
        kw1 = bw[1];
      }
      kw0 >>= 4 * g;
      kw1 >>= 4 * g;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const uint32_t kw = t == 0 ? kw0 : kw1;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kl = 8 * (r >> 2) + (r & 3);
          const bool keep = (32 * t + kl <= lim_l) && ((kw >> kl) & 1u);
          st[t][r] = keep ? st[t][r] : -INFINITY;
        }
      }
    }
    // The row lives in lanes c and c+32.
    float mx = st[0][0];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, st[t][r]);
    mx = pair_max(mx);
    // The reference point m_run of the exponentials only has to stay within 2^kSlack of
    // the true running max (P then stays below 2^kSlack, exact in fp32 and well inside
    // the 16-bit types' range), so it is moved -- and O, l rescaled -- only when some
    // row of the wave outgrows it by more than that.  The decision is wave-uniform; the
    // result is the same sum with a different common factor.
    constexpr float kSlack = 6.f;
    const float m_cand = mx * p.sl2;
    if (__builtin_amdgcn_ballot_w64(m_cand > m_run + kSlack) != 0) {
      const float m_new = fmaxf(m_run, m_cand);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);  // m_run = -inf -> 0
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) ot[dt][r] *= alpha;
    }
    const float m_ref = m_run == -INFINITY ? 0.f : m_run;
    float rs = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(st[t][r], p.sl2, -m_ref));
        st[t][r] = pv;
        rs += pv;
      }
    l_run += rs;
  };

  // O^T += V^T . P^T.  k-slot e of lane group g in k-step (t, s2) is key
  // 32t + 16 s2 + 8(e/4) + 4g + e%4 -- the accumulator order of S^T.
  auto pv_tile = [&](const uint16_t* tV, const f32x16_t (&st)[2]) {
    const int i16 = c & 15;
    const int j16 = c >> 4;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        u32x4_t pb;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          pb[e] = pack2<BF16>(st[t][8 * s2 + 2 * e], st[t][8 * s2 + 2 * e + 1]);
        const int vrow = 32 * t + 16 * s2 + 4 * g + (i16 >> 2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const int unit = 2 * dt + j16;
          const int u0 = unit ^ v_swizzle<D>(vrow);
          const int u1 = unit ^ v_swizzle<D>(vrow + 8);
          const s16x4_t lo = lds_read_tr16(tV + vrow * D + u0 * 16 + (i16 & 3) * 4);
          const s16x4_t hi = lds_read_tr16(tV + (vrow + 8) * D + u1 * 16 + (i16 & 3) * 4);
          const u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo);
          const u32x2_t hi2 = __builtin_bit_cast(u32x2_t, hi);
          const u32x4_t a = {lo2[0], lo2[1], hi2[0], hi2[1]};
          ot[dt] = mfma_32x32x16<BF16>(a, pb, ot[dt]);
        }
      }
    }
  };

  // ---- software pipeline ----------------------------------------------------------
  // Top of iteration `it` (before the barrier): in flight are K(it+1) -> sK[(it+1)&1] and
  // V(it) -> sV[it&1]; st_cur holds S^T of step it.  After the barrier every wave has
  // finished reading sK[it&1] (S^T of step it) and sV[(it-1)&1] (PV of step it-1), so
  // those two buffers are refilled with K(it+2) and V(it+1).
  // Step descriptors: raw metadata words are loaded three steps ahead and interpreted
  // one iteration later, two steps ahead of their first use (the K tile load).
  StepInfo cur = interpret(0, fetch_raw(0));
  StepInfo nxt = interpret(1, fetch_raw(1));
  StepInfo nn = interpret(2, fetch_raw(2));
  RawStep raw3 = fetch_raw(3);
  int cls_cur = classify(cur), cls_nxt = nsteps > 1 ? classify(nxt) : 0;
  f32x16_t st_cur[2], st_nxt[2];
  if (nsteps > 0) {
    issue_k(0, cur.row0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    if (nsteps > 1) issue_k(1, nxt.row0);
    issue_v(0, cur.row0);
    if (cls_cur != 0) qk_tile(sK, st_cur);
  }

  for (int it = 0; it < nsteps; ++it) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this thread's tile loads have landed
    __syncthreads();
    if (it + 2 < nsteps) issue_k(it & 1, nn.row0);
    if (it + 1 < nsteps) issue_v((it + 1) & 1, nxt.row0);
    const StepInfo n3 = interpret(it + 3, raw3);
    raw3 = fetch_raw(it + 4);
    if (cur.mode == kPartial) stage_mask_bits(it, cur);

    if (cls_nxt != 0) qk_tile(sK + ((it + 1) & 1) * TILE, st_nxt);
    if (cls_cur != 0) {
      softmax_step(st_cur, cur, cls_cur == 2);
      pv_tile(sV + (it & 1) * TILE, st_cur);
    }

#pragma unroll
    for (int t = 0; t < 2; ++t) st_cur[t] = st_nxt[t];
    cur = nxt;
    cls_cur = cls_nxt;
    nxt = nn;
    cls_nxt = (it + 2 < nsteps) ? classify(nn) : 0;
    nn = n3;
  }

  // Epilogue: O = O^T / l, zeros for rows without any allowed key or beyond seqlen.
  const float l_tot = pair_sum(l_run);
  const bool live = (q_row < p.seqlen) && (l_tot > 0.f);
  const float inv = live ? 1.f / l_tot : 0.f;
  if (q_row < p.S) {
    uint16_t* op = p.o + slab + size_t(q_row) * D + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        u32x2_t ov;
        ov[0] = pack2<BF16>(ot[dt][4 * r4 + 0] * inv, ot[dt][4 * r4 + 1] * inv);
        ov[1] = pack2<BF16>(ot[dt][4 * r4 + 2] * inv, ot[dt][4 * r4 + 3] * inv);
        *reinterpret_cast<u32x2_t*>(op + 32 * dt + 8 * r4) = ov;
      }
    }
    if (p.lse != nullptr && g == 0) {
      const float lse = live ? (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f : -INFINITY;
      p.lse[size_t(bh) * p.S + q_row] = lse;
    }
  }
}

// Host-side launch of one instance; returns the hipError_t of the launch.
template <bool BF16, int D, int QB, int KB>
int launch_fwd(const FwdParams& p, hipStream_t stream) {
  using Traits = FwdTraits<BF16, D, QB, KB>;
  auto kern = fwd_kernel<BF16, D, QB, KB>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     int(Traits::kLdsBytes));
  if (e != hipSuccess) return int(e);
  const unsigned slabs_per_xcd = unsigned(p.n_slabs + 7) / 8u;
  const dim3 grid(8u * slabs_per_xcd * unsigned(p.Tq));
  const dim3 block(Traits::kThreads);
  hipLaunchKernelGGL(kern, grid, block, Traits::kLdsBytes, stream, p);
  return int(hipGetLastError());
}

}  // namespace omni_attn

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
// steps of 64 keys (a 128-key block is two steps; 32 keys for 64-row query blocks).  K and
// V tiles are double-buffered in LDS and filled by direct buffer->LDS loads (no register
// staging, out-of-range rows read as zeros).
//
// The walk is software-pipelined so that the matrix cores and the vector ALU work on
// different steps inside ONE instruction stream: iteration i of a wave issues the 2*D/16
// MFMAs of S^T(i+1) and the D/8 MFMAs of O^T += V^T.P^T(i-1) while its vector
// instructions do the online softmax of step i.  None of the three depends on another
// inside the iteration, and the source spells the interleaving out: the iteration is a
// sequence of slots, each with one MFMA, the LDS fetch of the operand three slots ahead, a
// share of the softmax and -- in the early slots -- one tile load, with a scheduling fence
// after every slot.  (A wave that issues MFMAs back to back leaves other waves of its
// SIMD almost no vector issue slots; vector instructions placed between the MFMAs of the
// same wave are nearly free.)  Two iterations are unrolled so that the accumulators of
// S^T and the packed P alternate between two register sets without copies.
// One workgroup barrier per step.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <utility>

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

// The hipError_t of the last HIP call of this thread that made an entry point return
// OMNI_ATTN_ERR_LAUNCH (read back through omni_attn_last_hip_error()); defined beside that function.
void record_hip_error(int hip_error);

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
  const uint32_t* partial_bits;  // [P,QB,KB/32] words (bit j of word c = key 32c + j) or null;
                                 // at most one of partial_masks / partial_bits is set
  int num_partial; // P: tiles stored in partial_masks
  int S;           // padded sequence length (rows per (b,h) slab)
  int Tq;          // query blocks per slab
  int Tk;          // ceil(S / KB)
  int max_blocks;  // slots per query block
  int seqlen;      // min(seqlen_orig, S): rows/keys at or beyond it are padding
  int n_slabs;     // B*H
  int n_xcd;       // XCDs (L2 domains) of the device; workgroup ids go round-robin over them
  int slab_group;  // slabs of one XCD that are walked together (>= 1)
  float sl2;       // log2(e) / sqrt(D); log2(e) when scores are soft-capped (they are scaled there)
  float softcap;   // > 0: scores s / sqrt(D) are replaced by softcap * tanh(s / sqrt(D) / softcap)
  float cap_c2;    // 2 * log2(e) / (sqrt(D) * softcap)
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
// Maximum of values that are never NaN, as exactly one v_max_f32 / v_max3_f32 (the library
// function also quiets signalling NaNs: one more instruction for every operand the compiler
// knows nothing about).
__device__ __forceinline__ float vmax(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float vmax3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float pair_max(float x) {
  float lo, hi;
  pair_split(x, lo, hi);
  return vmax(lo, hi);
}
__device__ __forceinline__ float pair_sum(float x) {
  float lo, hi;
  pair_split(x, lo, hi);
  return lo + hi;
}

template <bool BF16, int D, int QB, int KB>
struct FwdTraits {
  static constexpr int kThreads = QB * 2;  // QB/32 waves of 64 lanes
  // Keys per step.  A 64-row query block has half the waves; at D = 128 its 64-key tiles would
  // leave LDS room for only two workgroups per CU (one wave per SIMD): it steps by 32 keys, four
  // workgroups fit and every SIMD has two waves again.  At D <= 64 four workgroups fit with 64-key
  // tiles, and a step has twice the matrix work per barrier.
  static constexpr int kStep = (QB == 64 && D == 128) ? 32 : 64;
  static constexpr int kTileElems = kStep * D;
  // K tiles, V tiles, one mask word per row and 32 keys, one mask byte per row and key in transit
  static constexpr size_t kLdsBytes = size_t(2) * 2 * kTileElems * sizeof(uint16_t) +
                                      size_t(QB) * (kStep / 32) * sizeof(uint32_t) + size_t(QB) * kStep;
};

// One step of the walk: kStep keys starting at row0, with the effective block mode.
struct StepInfo {
  int row0;
  int mode;
  int pid;
};

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((ext_vector_type(4))) int32_t i32x4_t;

// Buffer resource for a slab of `bytes` bytes: raw (unstructured) addressing, so a lane
// whose byte offset is at or beyond `bytes` reads zeros instead of faulting.
__device__ __forceinline__ i32x4_t make_buffer_resource(const void* base, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  i32x4_t r;
  r[0] = __builtin_amdgcn_readfirstlane(int32_t(uint32_t(a)));
  r[1] = __builtin_amdgcn_readfirstlane(int32_t(uint32_t(a >> 32) & 0xffffu));
  r[2] = __builtin_amdgcn_readfirstlane(int32_t(bytes));
  r[3] = 0x00020000;
  return r;
}
// 16 bytes per lane from a buffer straight into LDS: the wave's 64 chunks land at
// lds_base + 16 * lane.  The source offset is a wave-uniform part plus a per-lane part.
// Written as inline asm so that the compiler does not order later LDS reads of *other*
// buffers behind it with a vmcnt(0) wait; completion is waited for explicitly (vmcnt(0) +
// workgroup barrier) before the filled buffer is read.
__device__ __forceinline__ void buffer_to_lds_b128(i32x4_t rsrc, uint32_t lane_off,
                                                   uint32_t uniform_off, uint32_t lds_base) {
  // (Every scalar operand goes through readfirstlane: that is free for a value that is
  // already in scalar registers and keeps the operand legal if the compiler has chosen
  // to compute a uniform value with vector instructions.)
  i32x4_t r;
  r[0] = __builtin_amdgcn_readfirstlane(rsrc[0]);
  r[1] = __builtin_amdgcn_readfirstlane(rsrc[1]);
  r[2] = __builtin_amdgcn_readfirstlane(rsrc[2]);
  r[3] = __builtin_amdgcn_readfirstlane(rsrc[3]);
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen lds"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(lane_off), "s"(r),
        "s"(__builtin_amdgcn_readfirstlane(uniform_off))
      : "memory", "m0");
}
// 4 bytes per lane: the dword of lane l lands at lds_base + 4 * l (lanes switched off by the
// execution mask neither load nor store).
__device__ __forceinline__ void buffer_to_lds_b32(i32x4_t rsrc, uint32_t lane_off,
                                                  uint32_t uniform_off, uint32_t lds_base) {
  i32x4_t r;
  r[0] = __builtin_amdgcn_readfirstlane(rsrc[0]);
  r[1] = __builtin_amdgcn_readfirstlane(rsrc[1]);
  r[2] = __builtin_amdgcn_readfirstlane(rsrc[2]);
  r[3] = __builtin_amdgcn_readfirstlane(rsrc[3]);
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dword %1, %2, %3 offen lds"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(lane_off), "s"(r),
        "s"(__builtin_amdgcn_readfirstlane(uniform_off))
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

// An empty asm that "modifies" its operands: the values have to be computed before
// this point of the instruction stream (the optimizer would otherwise sink work whose
// results are only needed much later out of the place it was written in).
__device__ __forceinline__ void pin(float& a) { asm volatile("" : "+v"(a)); }
__device__ __forceinline__ void pin(uint32_t& a) { asm volatile("" : "+v"(a)); }
__device__ __forceinline__ void pin(float& a, float& b) { asm volatile("" : "+v"(a), "+v"(b)); }

template <int V>
struct IntC {
  static constexpr int value = V;
};
// f(IntC<0>{}), f(IntC<1>{}), ... f(IntC<N-1>{}): a loop whose index is a compile-time
// constant inside the body (register arrays indexed with it never go to scratch memory).
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(IntC<Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <bool BF16, int D, int QB, int KB>
__global__ void __launch_bounds__(QB * 2, 2) fwd_kernel(const FwdParams p) {
  using Traits = FwdTraits<BF16, D, QB, KB>;
  constexpr int NT = Traits::kThreads;
  constexpr int STEP = Traits::kStep;
  constexpr int SPB = KB / STEP;        // steps per KV block
  constexpr int NTL = STEP / 32;        // 32-key accumulator tiles of S^T per step
  constexpr int CPR = D / 8;            // 16-byte chunks per row
  constexpr int NCH = STEP * CPR / NT;  // 16-byte chunks per thread per tile
  constexpr int KS = D / 16;            // MFMA k-steps of Q.K
  constexpr int DT = D / 32;            // 32-row tiles of O^T
  constexpr int TILE = Traits::kTileElems;
  static_assert(STEP * CPR % NT == 0, "tile must divide over the workgroup");

  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  uint16_t* sK = reinterpret_cast<uint16_t*>(lds_raw);           // [2][TILE]
  uint16_t* sV = sK + 2 * TILE;                                  // [2][TILE]
  uint32_t* sBits = reinterpret_cast<uint32_t*>(sV + 2 * TILE);  // [QB][NTL]
  uint8_t* sMaskBytes = reinterpret_cast<uint8_t*>(sBits + QB * NTL);  // [QB][STEP]

  // Workgroup -> (slab, query block).  Consecutive workgroup ids go round-robin over
  // the XCDs.  XCD x takes the slabs bh with bh % n_xcd == x (every batch element's heads
  // are spread over all XCDs, which balances batches with different masks) and works
  // through them in groups of p.slab_group slabs, sized so that one group's query
  // blocks just fill the XCD's workgroup slots: the workgroups that run together then
  // belong to one or two slabs and walk the same K/V rows at about the same time, so
  // each K/V tile is fetched from HBM once and served from the XCD's L2 to the other
  // query blocks.  Inside a group the order is longest-first: query block Tq-1 of each
  // slab of the group, then Tq-2, ...
  const int wg = blockIdx.x;
  const int slot = wg / p.n_xcd;
  const int xcd = wg - slot * p.n_xcd;
  const int slabs_here = (p.n_slabs - xcd + p.n_xcd - 1) / p.n_xcd;
  if (slot >= slabs_here * p.Tq) return;
  const int per_group = p.slab_group * p.Tq;
  const int gi = slot / per_group;
  const int in_group = slot - gi * per_group;
  const int g_left = slabs_here - gi * p.slab_group;
  const int g_eff = g_left < p.slab_group ? g_left : p.slab_group;
  const int qrank = in_group / g_eff;
  const int bh = xcd + p.n_xcd * (gi * p.slab_group + (in_group - qrank * g_eff));
  const int qb = p.Tq - 1 - qrank;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int c = lane & 31;

  // Rows at or beyond the sequence are never used: the resources of K and V end there (those
  // rows arrive as zeros) and the query rows beyond it are replaced by zeros, whatever the caller
  // left in the padding.
  const size_t slab = size_t(bh) * size_t(p.S) * D;
  const uint32_t live_bytes = uint32_t(p.seqlen) * uint32_t(D * 2);
  const i32x4_t rK = make_buffer_resource(p.k + slab, live_bytes);
  const i32x4_t rV = make_buffer_resource(p.v + slab, live_bytes);

  const int q_row = qb * QB + 32 * w + c;  // this lane's query row inside the slab
  const int q_wave_min = qb * QB + 32 * w;

  const size_t meta_row = size_t(bh) * p.Tq + qb;
  const size_t meta_off = meta_row * p.max_blocks;

  // Block metadata lives in registers: lane i of every wave holds the (validated) words of
  // block 64 * chunk + i of this query block's list -- first key row, effective mode,
  // partial-mask index -- and a step's words are picked out with v_readlane: no memory
  // instruction per step.  A new chunk is fetched when the walk reaches it (every 64
  // blocks).  The loads of a chunk do not depend on the block count, so the first chunk,
  // the count and Q are all in flight together at the start of the kernel.
  const bool packed_tiles = p.partial_bits != nullptr;
  const bool has_partial = p.partial_idx != nullptr && (p.partial_masks != nullptr || packed_tiles);
  int32_t mv_row0 = 0, mv_mode = kMasked, mv_pid = -1;
  auto load_chunk = [&](int chunk) {
    const int j = chunk * 64 + lane;
    const size_t o = meta_off + size_t(j < p.max_blocks ? j : 0);
    const int32_t kvb_raw = p.kv_indices[o];
    const int32_t ty = p.types[o];
    const int32_t pid = has_partial ? p.partial_idx[o] : -1;
    const int32_t kvb = kvb_raw < 0 ? 0 : (kvb_raw >= p.Tk ? p.Tk - 1 : kvb_raw);
    int32_t mode = (ty == kCausal || ty == kFull || ty == kPartial) ? ty : int32_t(kMasked);
    if (ty == kPartial && (pid < 0 || pid >= p.num_partial)) mode = kMasked;
    mv_row0 = kvb * KB;
    mv_mode = mode;
    mv_pid = pid;
  };
  load_chunk(0);
  int nb = load_uniform(p.kv_num_blocks + meta_row);
  nb = nb < 0 ? 0 : (nb > p.max_blocks ? p.max_blocks : nb);
  const int nsteps = nb * SPB;

  // Q as the B operand of S^T = K.Q^T: lane holds Q[q_row][16s + 8g .. +7].
  u32x4_t qf[KS];
  {
    const int qr = q_row < p.S ? q_row : p.S - 1;
    const uint16_t* qp = p.q + slab + size_t(qr) * D + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s)
      qf[s] = q_row < p.seqlen ? *reinterpret_cast<const u32x4_t*>(qp + 16 * s) : u32x4_t{0u, 0u, 0u, 0u};
  }
  // Step `it` (clamped to the last step of the walk; steps past the end are only ever
  // used as the address of a tile load whose data nobody reads).
  auto step_info = [&](int it) {
    const int itc = it < nsteps ? it : nsteps - 1;
    const int j = itc / SPB;
    if (itc == it && itc % SPB == 0 && (j & 63) == 0 && j > 0) load_chunk(j >> 6);
    const int ln = j & 63;
    StepInfo si;
    si.row0 = __builtin_amdgcn_readlane(mv_row0, ln) + (itc % SPB) * STEP;
    si.mode = __builtin_amdgcn_readlane(mv_mode, ln);
    si.pid = __builtin_amdgcn_readlane(mv_pid, ln);
    return si;
  };

  // Direct buffer->LDS tile load: every lane fetches 16 bytes, the wave's 64 chunks land
  // at consecutive LDS addresses: one wave-wide load fills 64 / CPR rows of the tile.
  // The swizzle is applied on the source side: the lane that fills physical chunk
  // (row, pch) fetches the logical chunk that belongs there.  The swizzle depends on the
  // row modulo 16 at most and a thread's loads are ROW_STRIDE rows apart, so one or two
  // per-lane byte offsets serve all loads of a thread; the rest of the address is
  // wave-uniform and goes through the scalar offset of the load.
  constexpr int ROWS_PER_CALL = 64 / CPR;                // rows filled by one wave-wide load
  constexpr int ROW_STRIDE = ROWS_PER_CALL * (NT / 64);  // rows between a thread's loads
  constexpr int KPER = ROW_STRIDE % 16 == 0 ? 1 : 2;     // distinct K lane offsets
  static_assert((KPER * ROW_STRIDE) % 16 == 0, "K swizzle must repeat over a thread's loads");
  static_assert(ROW_STRIDE % 8 == 0, "V swizzle must be the same for all loads of a thread");
  const int ld_row = tid / CPR;  // row of this thread's first load
  const int ld_pch = tid % CPR;
  auto k_off = [&](int row) { return uint32_t(row * D + (ld_pch ^ k_swizzle<D>(row)) * 8) * 2u; };
  auto v_off = [&](int row) {
    return uint32_t(row * D + ((((ld_pch >> 1) ^ v_swizzle<D>(row)) << 1) | (ld_pch & 1)) * 8) * 2u;
  };
  uint32_t koff[KPER];
#pragma unroll
  for (int i = 0; i < KPER; ++i)
    koff[i] = k_off(ld_row + i * ROW_STRIDE) - uint32_t(i * ROW_STRIDE * D * 2);
  const uint32_t voff = v_off(ld_row);
  const uint32_t lds_k0 = lds_offset_of(sK) + uint32_t(w) * 1024u;
  const uint32_t lds_v0 = lds_offset_of(sV) + uint32_t(w) * 1024u;
  // Load number n of a tile pair: n < NCH is part n of the V tile, the rest the K tile.
  auto issue_load = [&](int n, int buf, int k_row0, int v_row0) {
    const bool is_v = n < NCH;
    const int i = is_v ? n : n - NCH;
    const uint32_t dst = (is_v ? lds_v0 : lds_k0) + uint32_t(buf) * (TILE * 2u) + uint32_t(i) * (NT * 16u);
    const uint32_t row = uint32_t(is_v ? v_row0 : k_row0) + uint32_t(i * ROW_STRIDE);
    buffer_to_lds_b128(is_v ? rV : rK, is_v ? voff : koff[i % KPER], row * uint32_t(D * 2), dst);
  };

  // PARTIAL blocks, in two stages so that no load latency is exposed.  One iteration ahead
  // each wave fetches the STEP mask bytes of its 32 rows for that step straight into LDS
  // (buffer->LDS loads, no registers; the resource covers exactly the tile); at the end of
  // that iteration a lane packs 32 of the bytes of a row to 32 bits and parks the word in LDS
  // for the two lanes that own the row.  Writer and readers of both stages are the same wave,
  // so no workgroup barrier is needed.
  constexpr int MCPR = STEP / 16;  // 16-byte chunks per row of mask bytes
  auto prefetch_mask_bytes = [&](int it, const StepInfo& si) {
    const int half = it % SPB;
    const i32x4_t rM = make_buffer_resource(p.partial_masks + size_t(si.pid) * (QB * KB), uint32_t(QB * KB));
    const uint32_t dst = lds_offset_of(sMaskBytes) + uint32_t(w) * uint32_t(32 * STEP);
#pragma unroll
    for (int i = 0; i < MCPR / 2; ++i) {  // 64 / MCPR rows per load
      const uint32_t row = uint32_t(32 * w + i * (64 / MCPR)) + uint32_t(lane / MCPR);
      buffer_to_lds_b128(rM, row * uint32_t(KB) + uint32_t(lane % MCPR) * 16u, uint32_t(half * STEP),
                         dst + uint32_t(i) * 1024u);
    }
  };
  // Tiles that arrive already packed (one 32-bit word per row and 32 keys) need no second
  // stage: one 4-byte buffer->LDS load per lane puts the step's words of the wave's 32 rows
  // where the byte path parks the words it packs.
  auto prefetch_mask_words = [&](int it, const StepInfo& si) {
    constexpr uint32_t TILE_WORDS = uint32_t(QB) * (KB / 32);
    const int half = it % SPB;
    const i32x4_t rM = make_buffer_resource(p.partial_bits + size_t(si.pid) * TILE_WORDS, TILE_WORDS * 4u);
    if (lane < 32 * NTL) {
      const uint32_t row = uint32_t(32 * w + lane / NTL);
      buffer_to_lds_b32(rM, (row * uint32_t(KB / 32) + uint32_t(lane % NTL)) * 4u, uint32_t(half * NTL) * 4u,
                        lds_offset_of(sBits) + uint32_t(32 * w * NTL) * 4u);
    }
  };
  auto stage_mask_bits = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the bytes have landed
    // word NTL * row + h of the wave's 32 rows; with one word per row the upper half-wave
    // repeats the lower one
    const int wi = lane % (32 * NTL);
    const uint8_t* mp = sMaskBytes + size_t(32 * w) * STEP + size_t(wi) * 32;
    const u32x4_t m0 = *reinterpret_cast<const u32x4_t*>(mp);
    const u32x4_t m1 = *reinterpret_cast<const u32x4_t*>(mp + 16);
    uint32_t word = 0;  // byte i of the 32 (any non-zero value = attend, attn_naive.cu:151) -> bit i
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t bytes = i < 4 ? m0[i] : m1[i - 4];
      bytes |= bytes >> 4;  // fold each byte onto its lowest bit
      bytes |= bytes >> 2;
      bytes |= bytes >> 1;
      const uint32_t nib = ((bytes & 0x01010101u) * 0x01020408u) >> 24;
      word |= nib << (4 * i);
    }
    sBits[32 * w * NTL + wi] = word;
  };

  // Does this wave's 32 x STEP tile of the step need no mask at all?  (wave-uniform)
  auto unmasked = [&](const StepInfo& si) {
    const bool inside = si.row0 + STEP <= p.seqlen;  // (written without branches: scalar selects)
    const bool full = si.mode == kFull;
    const bool below = (si.mode == kCausal) & (si.row0 + STEP - 1 <= q_wave_min);
    return inside & (full | below);
  };

  // LDS operand fetches.  K: rows 32t + c of the tile at k-step s.
  auto k_frag = [&](const uint16_t* tK, int s, int t) {
    const int row = 32 * t + c;
    const int ch = (2 * s + g) ^ k_swizzle<D>(row);
    return *reinterpret_cast<const u32x4_t*>(tK + row * D + ch * 8);
  };
  // V^T: operand j = (ts, dt) is rows 32 dt .. +31 of V^T (d) at keys 16 ts .. +15; k-slot e
  // of lane group g in k-step ts = (t, s2) is key 32t + 16 s2 + 8(e/4) + 4g + e%4 -- the
  // accumulator order of S^T.
  const int i16 = c & 15;
  const int j16 = c >> 4;
  auto v_frag = [&](const uint16_t* tV, int j) {
    const int ts = j / DT, dt = j % DT;
    const int vrow = 16 * ts + 4 * g + (i16 >> 2);
    const int unit = 2 * dt + j16;
    const int u0 = unit ^ v_swizzle<D>(vrow);
    const int u1 = unit ^ v_swizzle<D>(vrow + 8);
    const s16x4_t lo = lds_read_tr16(tV + vrow * D + u0 * 16 + (i16 & 3) * 4);
    const s16x4_t hi = lds_read_tr16(tV + (vrow + 8) * D + u1 * 16 + (i16 & 3) * 4);
    const u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo);
    const u32x2_t hi2 = __builtin_bit_cast(u32x2_t, hi);
    const u32x4_t a = {lo2[0], lo2[1], hi2[0], hi2[1]};
    return a;
  };

  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16_t ot[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) ot[dt] = zero16;
  f32x16_t st[2][NTL];   // [set][32-key tile]: S^T of the current / next step, alternating
  u32x4_t pb[2][NTL][2];  // [set][tile][16-key half]: P^T packed to 16 bits, B-operand order
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int t = 0; t < NTL; ++t) {
      st[a][t] = zero16;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) pb[a][t][s2] = u32x4_t{0u, 0u, 0u, 0u};
    }
  float m_run = -INFINITY;  // reference point of the exponentials, log2 domain (score * sl2)
  float l_run = 0.f;        // this lane's share of the running row sum
  // When the reference point moves, the rescale of O waits until the top of the next
  // iteration: the PV product that is in flight still belongs to the old reference.
  float alpha_pending = 1.f;
  uint64_t rescale_pending = 0;  // wave-uniform: lanes whose row outgrew the reference

  // ---- one iteration of the pipeline ----------------------------------------------------
  // SET = it % 2.  Reads K(it+1) from sK[SET^1] into st[SET^1], V(it-1) from sV[SET^1] with
  // pb[SET^1]; softmax of st[SET] into pb[SET]; loads K(it+2) into sK[SET] and V(it) into
  // sV[SET] (both last read one iteration ago).
  constexpr int NQK = NTL * KS;            // MFMAs of S^T
  constexpr int NPV_ALL = (STEP / 16) * DT; // MFMAs of O^T
  constexpr int NL = 2 * NCH;     // tile loads per thread
  constexpr int PF_ALL = 3;       // operand fetch distance in slots
  constexpr float kSlack = 6.f;

  // Mask of a step whose 32x64 tile is not entirely allowed, applied to S^T before the
  // iteration that does its softmax: disallowed scores become -inf.  Register r of tile t
  // holds key  row0 + 32t + 8(r/4) + 4g + r%4.
  auto apply_mask = [&](auto set_c, const StepInfo& si) {
    constexpr int SET = decltype(set_c)::value;
    int limit = p.seqlen - 1;
    if (si.mode == kCausal) limit = limit < q_row ? limit : q_row;
    if (si.mode == kMasked) limit = -1;
    const int lim_l = limit - si.row0 - 4 * g;
    uint32_t kw[NTL];
#pragma unroll
    for (int t = 0; t < NTL; ++t) kw[t] = 0xffffffffu;
    if (si.mode == kPartial) {
#pragma unroll
      for (int t = 0; t < NTL; ++t) kw[t] = sBits[(32 * w + c) * NTL + t];
    }
    // the limit becomes part of the bit words: positions 0 .. lim_l - 32t of word t stay
    static_for<NTL>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      kw[t] >>= 4 * g;
      const int n = lim_l - 32 * t + 1;  // allowed low positions of word t
      const uint32_t low = n >= 32 ? 0xffffffffu : (n <= 0 ? 0u : ((1u << (n & 31)) - 1u));
      kw[t] &= low;
    });
    // two instructions per score: the bit, sign-extended to a full word, selects between the
    // score and -inf
    static_for<16 * NTL>([&](auto ec) {
      constexpr int e = decltype(ec)::value;
      constexpr int t = e / 16, r = e % 16;
      constexpr int kl = 8 * (r >> 2) + (r & 3);
      const uint32_t keep = uint32_t(__builtin_amdgcn_sbfe(int(kw[t]), kl, 1));  // 0 or ~0
      const uint32_t bits = __builtin_bit_cast(uint32_t, float(st[SET][t][r]));
      st[SET][t][r] = __builtin_bit_cast(float, (bits & keep) | (0xff800000u & ~keep));
    });
  };

  // Soft-capped scores (the score_mod of transfusion_pytorch/transfusion.py:358-364, applied to the
  // scaled score as at :958-959 and :968): cap * tanh(x / cap) = cap * (1 - 2 / (exp(2 x / cap) + 1)),
  // written into S^T before the mask and the softmax of the step; the softmax then runs on
  // scores that are already scaled (sl2 = log2 e).
  auto apply_softcap = [&](auto set_c) {
    constexpr int SET = decltype(set_c)::value;
    const float cap = p.softcap, c2 = p.cap_c2;
    static_for<16 * NTL>([&](auto ec) {
      constexpr int e = decltype(ec)::value;
      constexpr int t = e / 16, r = e % 16;
      const float ex = __builtin_amdgcn_exp2f(st[SET][t][r] * c2);
      const float rc = __builtin_amdgcn_rcpf(ex + 1.f);
      st[SET][t][r] = __builtin_fmaf(rc, -2.f * cap, cap);
    });
  };

  // The first operands of an iteration are fetched right after the barrier, ahead of everything
  // else that happens between two bodies: their LDS latency runs under that bookkeeping.
  auto body_prefetch = [&](auto set_c, auto first_c, u32x4_t* opq) {
    constexpr int SET = decltype(set_c)::value;
    constexpr int NPV = decltype(first_c)::value != 0 ? 0 : NPV_ALL;
    constexpr int NS = NQK + NPV;
    constexpr int PF = PF_ALL < NS ? PF_ALL : NS;
    const uint16_t* tK = sK + (SET ^ 1) * TILE;
    const uint16_t* tV = sV + (SET ^ 1) * TILE;
    static_for<PF>([&](auto nc) {
      constexpr int n = decltype(nc)::value;
      if constexpr (n < NPV) {
        opq[n] = v_frag(tV, n);
      } else {
        opq[n] = k_frag(tK, (n - NPV) / NTL, (n - NPV) % NTL);
      }
    });
  };
  auto body = [&](auto set_c, auto first_c, int k_row0, int v_row0, u32x4_t* opq) {
    constexpr int SET = decltype(set_c)::value;
    // The first iteration of a walk has no previous step: no PV slots.
    constexpr int NPV = decltype(first_c)::value != 0 ? 0 : NPV_ALL;
    constexpr int NS = NQK + NPV;  // slots
    constexpr int LSP = (NS / 2) / NL > 0 ? (NS / 2) / NL : 1;  // slots between tile loads
    static_assert(NL * LSP <= NS, "tile loads must fit in the slots");
    constexpr int PF = PF_ALL < NS ? PF_ALL : NS;
    constexpr int NMX = 2 * NTL;          // max chunks of 8 scores
    constexpr int NPR = 8 * NTL;          // pairs of exponentials
    constexpr int NV = NMX + 1 + NPR;     // vector chunks: max, reference, exponentials
    const uint16_t* tK = sK + (SET ^ 1) * TILE;
    const uint16_t* tV = sV + (SET ^ 1) * TILE;
    auto operand = [&](int n) { return n < NPV ? v_frag(tV, n) : k_frag(tK, (n - NPV) / NTL, (n - NPV) % NTL); };

    float mxa, mxb, m_ref = 0.f, rs0, rs1;
    auto vector_chunk = [&](auto uc) {
      constexpr int u = decltype(uc)::value;
      if constexpr (u < 0) {
      } else if constexpr (u < NMX) {
        static_for<4>([&](auto ec) {
          constexpr int e = 8 * u + 2 * decltype(ec)::value;
          if constexpr (u == 0 && e == 0) {
            mxa = vmax(st[SET][0][0], st[SET][0][1]);
          } else if constexpr (u == 1 && e == 8) {
            mxb = vmax(st[SET][0][8], st[SET][0][9]);
          } else if constexpr ((u & 1) != 0) {
            mxb = vmax3(mxb, st[SET][e / 16][e % 16], st[SET][e / 16][e % 16 + 1]);
          } else {
            mxa = vmax3(mxa, st[SET][e / 16][e % 16], st[SET][e / 16][e % 16 + 1]);
          }
        });
      } else if constexpr (u == NMX) {
        // The reference point m_run of the exponentials only has to stay within 2^kSlack of
        // the true running max (P then stays below 2^kSlack, exact in fp32 and well inside
        // the 16-bit types' range), so it is moved -- and O, l rescaled -- only when some
        // row of the wave outgrows it by more than that.  The decision is wave-uniform; the
        // result is the same sum with a different common factor.  (Written without
        // branches: an unmoved reference gives a factor of exactly 1, or of 0 for a row that
        // has not seen a key yet and whose sums are still 0.)
        const float mx = pair_max(vmax(mxa, mxb));  // the row lives in lanes c and c+32
        const float m_cand = mx * p.sl2;
        const uint64_t movers = __builtin_amdgcn_ballot_w64(m_cand > m_run + kSlack);
        const bool move = movers != 0;
        const float m_new = move ? vmax(m_run, m_cand) : m_run;
        m_ref = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
        l_run *= alpha;
        m_run = m_new;
        alpha_pending = move ? alpha : alpha_pending;
        rescale_pending |= movers;
        pin(l_run, alpha_pending);
      } else {
        constexpr int i = u - NMX - 1;
        constexpr int t = i / 8, r = 2 * (i % 8);
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[SET][t][r], p.sl2, -m_ref));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[SET][t][r + 1], p.sl2, -m_ref));
        if constexpr (i == 0) {
          rs0 = p0;
          rs1 = p1;
        } else {
          rs0 += p0;
          rs1 += p1;
        }
        uint32_t packed = pack2<BF16>(p0, p1);
        pin(packed);
        pb[SET][t][r >> 3][(r & 7) >> 1] = packed;
        pin(rs0, rs1);
        if constexpr (i == NPR - 1) l_run += rs0 + rs1;
      }
    };

    // The slots run at a raised wave priority and everything between two bodies (barrier, rescale,
    // mask, metadata of the next steps) at the default one: the other wave of the SIMD, from the
    // other workgroup of the compute unit, is then not held up by this wave's bookkeeping while
    // it has matrix instructions to issue.
    __builtin_amdgcn_s_setprio(1);
    static_for<NS>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      if constexpr (j < NPV) {
        constexpr int ts = j / DT, dt = j % DT;
        ot[dt] = mfma_32x32x16<BF16>(opq[j % PF], pb[SET ^ 1][ts >> 1][ts & 1], ot[dt]);
      } else {
        constexpr int s = (j - NPV) / NTL, t = (j - NPV) % NTL;
        st[SET ^ 1][t] = mfma_32x32x16<BF16>(opq[j % PF], qf[s], s == 0 ? zero16 : st[SET ^ 1][t]);
      }
      if constexpr (j + PF < NS) opq[j % PF] = operand(j + PF);
      if constexpr (j % LSP == 0 && j / LSP < NL) issue_load(j / LSP, SET, k_row0, v_row0);
      constexpr int u_lo = j * NV / NS, u_hi = (j + 1) * NV / NS;
      static_for<u_hi - u_lo>([&](auto dc) { vector_chunk(IntC<u_lo + decltype(dc)::value>{}); });
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_s_setprio(0);
  };

  // ---- the walk -------------------------------------------------------------------------
  StepInfo cur = {0, kMasked, -1}, nxt = cur, nn = cur;
  if (nsteps > 0) {
    cur = step_info(0);
    nxt = step_info(1);
    nn = step_info(2);
    // Prologue: K(0) and K(1).
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      issue_load(NCH + i, 0, cur.row0, 0);
      issue_load(NCH + i, 1, nxt.row0, 0);
    }
    if (cur.mode == kPartial) {
      if (packed_tiles) {
        prefetch_mask_words(0, cur);
      } else {
        prefetch_mask_bytes(0, cur);
        stage_mask_bits();
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int t = 0; t < NTL; ++t)
        st[0][t] = mfma_32x32x16<BF16>(k_frag(sK, s, t), qf[s], s == 0 ? zero16 : st[0][t]);
  }

  auto iteration = [&](auto set_c, auto first_c, int it) {
    constexpr int SET = decltype(set_c)::value;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this thread's tile loads have landed
    __syncthreads();
    u32x4_t opq[PF_ALL];
    body_prefetch(IntC<SET>{}, first_c, opq);
    // The common step -- every score allowed, no rescale owed, no PARTIAL tile ahead, no soft cap
    // -- goes from the barrier into the slots over one scalar condition and one branch.
    const bool next_partial = it + 1 < nsteps && nxt.mode == kPartial;
    const bool plain = (rescale_pending == 0) & !(p.softcap > 0.f) & unmasked(cur) & !next_partial;
    if (!plain) {
      if (rescale_pending != 0) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) ot[dt][r] *= alpha_pending;
        rescale_pending = 0;
      }
      if (p.softcap > 0.f) apply_softcap(IntC<SET>{});
      if (!unmasked(cur)) apply_mask(IntC<SET>{}, cur);
      if (next_partial) {
        if (packed_tiles) {
          prefetch_mask_words(it + 1, nxt);
        } else {
          prefetch_mask_bytes(it + 1, nxt);
        }
      }
    }
    body(IntC<SET>{}, first_c, nn.row0, cur.row0, opq);
    if (next_partial && !packed_tiles) stage_mask_bits();
    const StepInfo n3 = step_info(it + 3);
    cur = nxt;
    nxt = nn;
    nn = n3;
  };
  if (nsteps > 0) {
    iteration(IntC<0>{}, IntC<1>{}, 0);
    if (1 < nsteps) iteration(IntC<1>{}, IntC<0>{}, 1);
  }
  for (int it = 2; it < nsteps; it += 2) {
    iteration(IntC<0>{}, IntC<0>{}, it);
    if (it + 1 < nsteps) iteration(IntC<1>{}, IntC<0>{}, it + 1);
  }

  // Drain: O^T += V^T . P^T of the last step.
  if (nsteps > 0) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (rescale_pending != 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) ot[dt][r] *= alpha_pending;
    }
    auto drain = [&](auto set_c) {
      constexpr int SET = decltype(set_c)::value;
#pragma unroll
      for (int j = 0; j < NPV_ALL; ++j) {
        const int ts = j / DT, dt = j % DT;
        ot[dt] = mfma_32x32x16<BF16>(v_frag(sV + SET * TILE, j), pb[SET][ts >> 1][ts & 1], ot[dt]);
      }
    };
    if ((nsteps - 1) & 1) {
      drain(IntC<1>{});
    } else {
      drain(IntC<0>{});
    }
  }

  // Epilogue: O = O^T / l, zeros for rows without any allowed key or beyond seqlen.
  // A lane holds 4 consecutive d of its row per accumulator group; stored directly, one
  // store instruction would touch 32 rows with 16 bytes each.  So the wave transposes its
  // 32 x D output through LDS -- its own 32 rows of the K buffers, which nobody reads after
  // the barrier of the drain, 16-byte chunks swizzled like a K tile -- and stores whole
  // rows: 64 lanes x 16 bytes = 64 / CPR complete rows per instruction.
  const float l_tot = pair_sum(l_run);
  const bool live = (q_row < p.seqlen) && (l_tot > 0.f);
  const float inv = live ? 1.f / l_tot : 0.f;
  {
    uint16_t* stage = sK + size_t(w) * 32 * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        u32x2_t ov;
        ov[0] = pack2<BF16>(ot[dt][4 * r4 + 0] * inv, ot[dt][4 * r4 + 1] * inv);
        ov[1] = pack2<BF16>(ot[dt][4 * r4 + 2] * inv, ot[dt][4 * r4 + 3] * inv);
        const int ch = (4 * dt + r4) ^ k_swizzle<D>(c);
        *reinterpret_cast<u32x2_t*>(stage + c * D + ch * 8 + 4 * g) = ov;
      }
    }
    constexpr int ROWS_PER_STORE = 64 / CPR;
    const int srow = lane / CPR, pch = lane % CPR;
#pragma unroll
    for (int i = 0; i < 32 / ROWS_PER_STORE; ++i) {
      const int row = i * ROWS_PER_STORE + srow;  // row of the wave
      const u32x4_t val = *reinterpret_cast<const u32x4_t*>(stage + row * D + pch * 8);
      const int grow = q_wave_min + row;
      if (grow < p.S)
        *reinterpret_cast<u32x4_t*>(p.o + slab + size_t(grow) * D + (pch ^ k_swizzle<D>(row)) * 8) = val;
    }
  }
  if (q_row < p.S && p.lse != nullptr && g == 0) {
    const float lse = live ? (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f : -INFINITY;
    p.lse[size_t(bh) * p.S + q_row] = lse;
  }
}

// Host-side launch of one instance; returns the hipError_t of the launch itself (the
// thread's sticky "last error" of earlier, unrelated HIP calls is neither read nor cleared).
// The dynamic-LDS limit of an instance is raised once per device, not on every launch.
constexpr int kMaxDevices = 64;
template <bool BF16, int D, int QB, int KB>
int launch_fwd(const FwdParams& p, hipStream_t stream) {
  using Traits = FwdTraits<BF16, D, QB, KB>;
  auto kern = fwd_kernel<BF16, D, QB, KB>;
  static std::atomic<bool> lds_limit_set[kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return int(e);
  const bool cached = dev >= 0 && dev < kMaxDevices;
  if (!cached || !lds_limit_set[dev].load(std::memory_order_acquire)) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, int(Traits::kLdsBytes));
    if (e != hipSuccess) return int(e);
    if (cached) lds_limit_set[dev].store(true, std::memory_order_release);
  }
  const unsigned slabs_per_xcd = unsigned(p.n_slabs + p.n_xcd - 1) / unsigned(p.n_xcd);
  const dim3 grid(unsigned(p.n_xcd) * slabs_per_xcd * unsigned(p.Tq));
  const dim3 block(Traits::kThreads);
  FwdParams params = p;
  void* args[] = {&params};
  return int(hipLaunchKernel(reinterpret_cast<const void*>(kern), grid, block, args,
                             Traits::kLdsBytes, stream));
}

}  // namespace omni_attn

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
// steps of 64 keys (a 128-key block is two steps) from a double-buffered LDS tile
// pair; the next step's K/V (and, for PARTIAL blocks, its mask bytes) are fetched
// into registers while the current step computes.
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
  int total_work;  // B*H*Tq
  int work_per_xcd;
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
// V is read with ds_read_b64_tr_b16: 4 lanes read 32 contiguous bytes of one row, the
// next 4 lanes the next row.  The 32-byte unit index is XORed with the row.
template <int D>
__device__ __forceinline__ int v_swizzle(int row) {
  constexpr int U = D / 16;  // 32-byte units per row
  return (row / (8 / U)) % U;
}

__device__ __forceinline__ s16x4_t lds_read_tr16(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s16x4_t*)(p));
}

template <bool BF16, int D, int QB, int KB>
struct FwdTraits {
  static constexpr int kThreads = QB * 2;  // QB/32 waves of 64 lanes
  static constexpr int kStep = 64;
  static constexpr int kTileElems = kStep * D;
  static constexpr size_t kLdsBytes =
      size_t(2) * 2 * kTileElems * sizeof(uint16_t) + size_t(2) * QB * 2 * sizeof(uint32_t);
};

template <bool BF16, int D, int QB, int KB>
__global__ void __launch_bounds__(QB * 2, 2) fwd_kernel(const FwdParams p) {
  using Traits = FwdTraits<BF16, D, QB, KB>;
  constexpr int NT = Traits::kThreads;
  constexpr int STEP = Traits::kStep;
  constexpr int SPB = KB / STEP;        // steps per KV block
  constexpr int CPR = D / 8;            // 16-byte chunks per row
  constexpr int NCH = STEP * CPR / NT;  // chunks per thread per tile
  constexpr int KS = D / 16;            // MFMA k-steps of Q.K
  constexpr int DT = D / 32;            // 32-row tiles of O^T
  constexpr int TILE = Traits::kTileElems;
  static_assert(STEP * CPR % NT == 0, "tile must divide over the workgroup");

  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  uint16_t* sK = reinterpret_cast<uint16_t*>(lds_raw);  // [2][TILE]
  uint16_t* sV = sK + 2 * TILE;                         // [2][TILE]
  uint32_t* sBits = reinterpret_cast<uint32_t*>(sV + 2 * TILE);  // [2][QB*2]

  // Workgroup -> (slab, query block).  Consecutive workgroup ids go round-robin over
  // the 8 XCDs, so give each XCD one contiguous range of the work list: all query
  // blocks of a (b,h) slab then share one XCD's L2 for that slab's K and V.  Inside a
  // slab the last (longest, under causal masks) query block is issued first.
  const int wg = blockIdx.x;
  const int work = (wg & 7) * p.work_per_xcd + (wg >> 3);
  if (work >= p.total_work) return;
  const int bh = work / p.Tq;
  const int qb = p.Tq - 1 - (work - bh * p.Tq);

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
  int nb = p.kv_num_blocks[meta_row];
  nb = nb < 0 ? 0 : (nb > p.max_blocks ? p.max_blocks : nb);
  const int nsteps = nb * SPB;

  // Decode step `it` of the walk: first key row, effective mode, partial-mask index.
  auto decode = [&](int it, int& kv_row0, int& mode, int& pid) {
    const int j = it / SPB;
    const int half = it - j * SPB;
    int kvb = p.kv_indices[meta_off + j];
    kvb = kvb < 0 ? 0 : (kvb >= p.Tk ? p.Tk - 1 : kvb);
    const int ty = p.types[meta_off + j];
    mode = (ty == kCausal || ty == kFull || ty == kPartial) ? ty : kMasked;
    pid = -1;
    if (ty == kPartial) {
      if (p.partial_idx != nullptr && p.partial_masks != nullptr) pid = p.partial_idx[meta_off + j];
      if (pid < 0) mode = kMasked;
    }
    kv_row0 = kvb * KB + half * STEP;
  };

  u32x4_t kreg[NCH], vreg[NCH], mreg[2];

  auto global_fetch = [&](int it, int kv_row0, int mode, int pid) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int x = tid + i * NT;
      const int row = x / CPR;
      const int ch = x % CPR;
      int gr = kv_row0 + row;
      gr = gr < p.S ? gr : p.S - 1;
      const size_t off = size_t(gr) * D + ch * 8;
      kreg[i] = *reinterpret_cast<const u32x4_t*>(gK + off);
      vreg[i] = *reinterpret_cast<const u32x4_t*>(gV + off);
    }
    if (mode == kPartial) {
      const int half = it % SPB;
      const uint8_t* mp = p.partial_masks + size_t(pid) * (QB * KB) + size_t(tid >> 1) * KB +
                          half * STEP + (tid & 1) * 32;
      mreg[0] = *reinterpret_cast<const u32x4_t*>(mp);
      mreg[1] = *reinterpret_cast<const u32x4_t*>(mp + 16);
    }
  };

  auto lds_commit = [&](int buf, int mode) {
    uint16_t* dK = sK + buf * TILE;
    uint16_t* dV = sV + buf * TILE;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int x = tid + i * NT;
      const int row = x / CPR;
      const int ch = x % CPR;
      const int kch = ch ^ k_swizzle<D>(row);
      const int vch = (((ch >> 1) ^ v_swizzle<D>(row)) << 1) | (ch & 1);
      *reinterpret_cast<u32x4_t*>(dK + row * D + kch * 8) = kreg[i];
      *reinterpret_cast<u32x4_t*>(dV + row * D + vch * 8) = vreg[i];
    }
    if (mode == kPartial) {
      // 32 mask bytes (each 0 or 1) -> 32 bits; byte i of a dword lands in bit i.
      uint32_t word = 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t bytes = i < 4 ? mreg[0][i] : mreg[1][i - 4];
        const uint32_t nib = ((bytes & 0x01010101u) * 0x01020408u) >> 24;
        word |= nib << (4 * i);
      }
      sBits[buf * (QB * 2) + tid] = word;
    }
  };

  f32x16_t ot[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) ot[dt][r] = 0.f;
  float m_run = -INFINITY;  // running row max, log2 domain (score * sl2)
  float l_run = 0.f;        // this lane's share of the running row sum

  int cur_row0 = 0, cur_mode = kMasked, cur_pid = -1;
  if (nsteps > 0) {
    decode(0, cur_row0, cur_mode, cur_pid);
    global_fetch(0, cur_row0, cur_mode, cur_pid);
    lds_commit(0, cur_mode);
  }
  __syncthreads();

  for (int it = 0; it < nsteps; ++it) {
    const int buf = it & 1;
    int nxt_row0 = 0, nxt_mode = kMasked, nxt_pid = -1;
    const bool has_next = it + 1 < nsteps;
    if (has_next) {
      decode(it + 1, nxt_row0, nxt_mode, nxt_pid);
      global_fetch(it + 1, nxt_row0, nxt_mode, nxt_pid);
    }

    // Wave-uniform classification of this wave's 32x64 tile.
    const bool clip = cur_row0 + STEP > p.seqlen;
    bool skip = cur_mode == kMasked;
    bool masked_path = cur_mode != kFull || clip;
    if (cur_mode == kCausal) {
      if (cur_row0 > q_wave_min + 31) skip = true;                      // all in the future
      else if (cur_row0 + STEP - 1 <= q_wave_min && !clip) masked_path = false;  // all in the past
    }

    if (!skip) {
      const uint16_t* tK = sK + buf * TILE;
      const uint16_t* tV = sV + buf * TILE;

      // S^T = K . Q^T : two 32-key tiles.
      f32x16_t st[2];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) st[t][r] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int row = 32 * t + c;
          const int ch = (2 * s + g) ^ k_swizzle<D>(row);
          const u32x4_t a = *reinterpret_cast<const u32x4_t*>(tK + row * D + ch * 8);
          st[t] = mfma_32x32x16<BF16>(a, qf[s], st[t]);
        }
      }

      if (masked_path) {
        // Register r of tile t holds key  cur_row0 + 32t + 8(r/4) + 4g + r%4.
        int limit = p.seqlen - 1;
        if (cur_mode == kCausal) limit = limit < q_row ? limit : q_row;
        const int lim_l = limit - cur_row0 - 4 * g;
        uint32_t kw0 = 0xffffffffu, kw1 = 0xffffffffu;
        if (cur_mode == kPartial) {
          const u32x2_t bw = *reinterpret_cast<const u32x2_t*>(sBits + buf * (QB * 2) + (32 * w + c) * 2);
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

      // Online softmax (log2 domain).  The row lives in lanes c and c+32.
      float mx = st[0][0];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, st[t][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run, mx * p.sl2);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
      m_run = m_new;
      float rs = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(st[t][r], p.sl2, -m_safe));
          st[t][r] = pv;
          rs += pv;
        }
      l_run = l_run * alpha + rs;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) ot[dt][r] *= alpha;

      // O^T += V^T . P^T.  k-slot e of lane group g in k-step (t, s2) is key
      // 32t + 16 s2 + 8(e/4) + 4g + e%4 -- the accumulator order of S^T.
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          u32x4_t pb;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            pb[e] = pack2<BF16>(st[t][8 * s2 + 2 * e], st[t][8 * s2 + 2 * e + 1]);
          const int i16 = c & 15;
          const int j16 = c >> 4;
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
    }

    if (has_next) lds_commit(buf ^ 1, nxt_mode);
    __syncthreads();
    cur_row0 = nxt_row0;
    cur_mode = nxt_mode;
    cur_pid = nxt_pid;
  }

  // Epilogue: O = O^T / l, zeros for rows without any allowed key or beyond seqlen.
  const float l_tot = l_run + __shfl_xor(l_run, 32);
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
  const dim3 grid(unsigned(p.work_per_xcd) * 8u);
  const dim3 block(Traits::kThreads);
  hipLaunchKernelGGL(kern, grid, block, Traits::kLdsBytes, stream, p);
  return int(hipGetLastError());
}

}  // namespace omni_attn

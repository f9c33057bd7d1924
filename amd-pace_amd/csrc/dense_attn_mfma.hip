// Dense bf16 attention on the matrix cores for head_dim 64 / 96 / 128 / 256: the fast path of the torch op
// pace::attention (dense_attn.hip holds the general kernel and the entry point).
#include <type_traits>

#include "attn_core.h"

namespace pace_kv {

// ---------------------------------------------------------------------------------
// Up to 64 query rows per head (decode, verify).  K and V are the reference's row-major
// [B][N][L][D] tensors.  K rows feed the first product directly (16 bytes of a row per
// lane); V rows are staged per wave in LDS and read back token-minor for the second.
// One workgroup of 4 waves per (batch, head, group of 16*NQT query rows); the waves split
// the L axis and merge through LDS like the paged kernel.
// ---------------------------------------------------------------------------------
struct DenseMfmaParams {
  PagedAttnParams base;  // q / out / mask fields and scale are shared with the paged kernel
  const uint16_t* k;
  const uint16_t* v;
  int32_t B, N, S, L;
  int32_t H;  // the tensors' head size: the kernel's D, or less (a multiple of 8) where the kernel is built PADDED
  int32_t mB, mN, mS;
  int32_t n_qgroups;
  // Optional summary of the mask, one entry per mask line ((mb * mN + mn) * mS + ms), written by
  // dense_mask_lines_kernel just before the attention launch: the last column above the floor (-1: none) and the
  // first one if the line is plain (see mask_line_summary), else -1.
  const int32_t* line_last;
  const int32_t* line_first;
};

// One wave per mask line.
__global__ __launch_bounds__(64) void dense_mask_lines_kernel(const void* mask, int is_f32, int L, int32_t* last_out, int32_t* first_out) {
  int last, first;
  mask_line_summary(mask, is_f32 != 0, (int64_t)blockIdx.x * L, 0, L, threadIdx.x, last, first);
  if (threadIdx.x == 0) last_out[blockIdx.x] = last, first_out[blockIdx.x] = first;
}

// ONCE: one group of query rows per (batch, head), so K / V are read once and fetched non-temporally.
// Waves per workgroup: four; two with head_dim 256, where a wave has a SIMD (and its 512 registers) to itself
// and the V stages of four would not fit the LDS a workgroup may have.
template <int D>
constexpr int dense_split_waves() { return D > 128 ? 2 : 4; }

// OCC: waves per SIMD the registers are budgeted for.  At head_dim 256 a wave with a SIMD to itself (OCC 1) spills
// nothing and is the faster form while the launch has no more workgroups than fit at that rate; a launch with more
// (decode steps of a batch) is bound by the loads in flight and gains from a second wave per SIMD.
// PADDED: the tensors' head size is dp.H < D, a multiple of 8: rows are dp.H elements apart, the 16-byte chunks past
// dp.H read as zero (they change neither a score nor an output dim that exists) and are not written.
template <int D, int NQT, bool HAS_MASK, bool ONCE, int OCC = (D > 128 ? 1 : 2), bool PADDED = false>
__global__ __launch_bounds__(64 * dense_split_waves<D>()) __attribute__((amdgpu_waves_per_eu(OCC))) void dense_attn_mfma_kernel(
    const DenseMfmaParams dp) {
  constexpr int KK = D / 32;
  constexpr int MT = D / 16;
  constexpr int NW = dense_split_waves<D>();
  constexpr int VROW = D + 24;                    // padded LDS row (elements): keeps the transposed reads off each other's banks
  constexpr int STAGE = 32 * VROW;                // one wave's V unit
  constexpr int MERGE_FLOATS = (NW / 2) * 16 * NQT * (D + 2);
  constexpr int LDS_BYTES = (NW * STAGE * 2 > MERGE_FLOATS * 4) ? NW * STAGE * 2 : MERGE_FLOATS * 4;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[LDS_BYTES];
  const PagedAttnParams& p = dp.base;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, g = lane >> 4;
  const int qg = blockIdx.x % dp.n_qgroups;
  const int head = (blockIdx.x / dp.n_qgroups) % dp.N;
  const int b = blockIdx.x / (dp.n_qgroups * dp.N);
  const int L = dp.L, S = dp.S;
  const int RS = PADDED ? dp.H : D;  // row stride of the tensors, in elements
  const uint16_t* kbase = dp.k + ((int64_t)b * dp.N + head) * (int64_t)L * RS;
  const uint16_t* vbase = dp.v + ((int64_t)b * dp.N + head) * (int64_t)L * RS;
  uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + wave * STAGE;

  u32x4 qreg[NQT][KK];
  RowState<D, NQT> st;
  int row_s[NQT];
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int s = (qg * NQT + qt) * 16 + n;
    const bool valid = s < S;
    row_s[qt] = s;
    st.limit[qt] = valid ? L - 1 : -1;
    if (HAS_MASK) {
      const int64_t mb = dp.mB == 1 ? 0 : b, mn = dp.mN == 1 ? 0 : head, ms = dp.mS == 1 ? 0 : (valid ? s : 0);
      st.mask_off[qt] = ((mb * dp.mN + mn) * dp.mS + ms) * (int64_t)L;
    } else {
      st.mask_off[qt] = 0;
    }
    st.m[qt] = kNegInf, st.m_top[qt] = kNegInf, st.m_neg[qt] = 0.f;
    st.l[qt] = 0.f;
    const uint16_t* qp = p.q + (((int64_t)b * dp.N + head) * S + (valid ? s : 0)) * RS + 8 * g;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qreg[qt][kk] = (valid && (!PADDED || 32 * kk + 8 * g < dp.H)) ? *reinterpret_cast<const u32x4*>(qp + kk * 32) : z;
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) st.o[qt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int units = (L + 31) / 32;
  const int per_wave = (units + NW - 1) / NW;
  const int u_begin = min(units, wave * per_wave);
  const int n_units = min(units, u_begin + per_wave) - u_begin;
  UnitRegs<D> buf;
  MaskRegs<NQT> mregs;
  constexpr int CH = D / 8;            // chunks per row
  constexpr int VCH = 32 * CH / 64;    // V chunks of a unit per lane
  // A wave that has a SIMD to itself has the registers to fetch a unit ahead: its loads then travel while the unit
  // before is worked on, instead of every unit waiting out its own memory latency with nothing else in flight.
  constexpr bool AHEAD = OCC == 1;
  // K: token 8*(n/4) + 4*tile + n%4 of the unit, dims 32*kk + 8g.. (clamped rows are masked later).
  auto fetch_k = [&](int t0, u32x4 (&kx)[2][KK]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int tok = min(L - 1, t0 + 8 * (n >> 2) + 4 * t + (n & 3));
      const uint16_t* kp = kbase + (int64_t)tok * RS + 8 * g;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        kx[t][kk] = u32x4{0u, 0u, 0u, 0u};
        if (!PADDED || 32 * kk + 8 * g < dp.H) kx[t][kk] = ONCE ? load16_stream(kp + kk * 32) : *reinterpret_cast<const u32x4*>(kp + kk * 32);
      }
    }
  };
  // V: the unit's 32 rows, coalesced 16-byte chunks
  auto fetch_v = [&](int t0, u32x4 (&vx)[VCH]) {
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int c = i * 64 + lane, r = c / CH, ch = c % CH;
      const uint16_t* vp = vbase + (int64_t)min(L - 1, t0 + r) * RS + ch * 8;
      vx[i] = u32x4{0u, 0u, 0u, 0u};
      if (!PADDED || ch * 8 < dp.H) vx[i] = ONCE ? load16_stream(vp) : *reinterpret_cast<const u32x4*>(vp);
    }
  };
  u32x4 k_next[AHEAD ? 2 : 1][AHEAD ? KK : 1], v_next[AHEAD ? VCH : 1];
  MaskRaw<NQT> m_next;
  if constexpr (AHEAD) {
    if (n_units > 0) {
      if (HAS_MASK) load_mask_raw<NQT>(m_next, p, st.mask_off, 32 * u_begin, g);
      fetch_k(32 * u_begin, k_next);
      fetch_v(32 * u_begin, v_next);
    }
  }
  for (int uu = 0; uu < n_units; ++uu) {
    const int t0 = 32 * (u_begin + uu);
    // ... V goes to this wave's LDS stage ...
    if constexpr (AHEAD) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) buf.k[t][kk] = k_next[t][kk];
      if (HAS_MASK) mask_regs_from_raw<NQT>(mregs, m_next, p);
#pragma unroll
      for (int i = 0; i < VCH; ++i) {
        const int c = i * 64 + lane, r = c / CH, ch = c % CH;
        *reinterpret_cast<u32x4*>(stage + r * VROW + ch * 8) = v_next[i];
      }
      if (uu + 1 < n_units) {
        if (HAS_MASK) load_mask_raw<NQT>(m_next, p, st.mask_off, t0 + 32, g);
        fetch_k(t0 + 32, k_next);
        fetch_v(t0 + 32, v_next);
      }
    } else {
      if (HAS_MASK) load_mask_regs<NQT>(mregs, p, st.mask_off, t0, g);  // travels with the unit's K / V
      fetch_k(t0, buf.k);
      u32x4 vx[VCH];
      fetch_v(t0, vx);
#pragma unroll
      for (int i = 0; i < VCH; ++i) {
        const int c = i * 64 + lane, r = c / CH, ch = c % CH;
        *reinterpret_cast<u32x4*>(stage + r * VROW + ch * 8) = vx[i];
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes have landed
    __builtin_amdgcn_wave_barrier();
    // ... and come back token-minor: lane (n, g) takes dim 16j + n of tokens 8g..8g+7.  The LDS
    // transpose read hands lane i of a 16-lane group element i % 4 of the 8-byte pieces that
    // lanes 4j + i / 4 (j = 0..3) point at; with lane s of the group pointing at token
    // 8g + s / 4, dims 16j + 4 (s % 4) .. +3, lane n receives tokens 8g .. 8g+3 of dim 16j + n,
    // and a second read four token rows further down completes the operand.
    typedef short tr_v4 __attribute__((ext_vector_type(4)));
    typedef tr_v4 __attribute__((address_space(3))) * tr_ptr;
    const uint16_t* tr_base = stage + (8 * g + (n >> 2)) * VROW + 4 * (n & 3);
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const tr_v4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(tr_base + 16 * j));
      const tr_v4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(tr_base + 4 * VROW + 16 * j));
      const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      buf.v[j] = u32x4{l2[0], l2[1], h2[0], h2[1]};
    }
    __builtin_amdgcn_wave_barrier();
    const bool full = t0 + 32 <= L;
    compute_unit<D, NQT, HAS_MASK>(buf, qreg, st, p, t0, L, 0, full, g, mregs);
  }
  finish_rows<D, NQT, HAS_MASK>(st, p);
  __syncthreads();  // every wave is done with its V stage; the space becomes the merge buffer
  float* merge_buf = reinterpret_cast<float*>(lds_raw);
  constexpr int ROW_F = D + 2;
  constexpr int SLOT_F = 16 * NQT * ROW_F;
#pragma unroll
  for (int stride = 1; stride < NW; stride *= 2) {
    const int slot = wave / (2 * stride);
    const bool sender = (wave & (2 * stride - 1)) == stride;
    const bool receiver = (wave & (2 * stride - 1)) == 0;
    if (sender) {
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) {
        float* rowp = merge_buf + slot * SLOT_F + (qt * 16 + n) * ROW_F;
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) rowp[16 * j + 4 * g + i] = st.o[qt][j][i];
        if (g == 0) rowp[D] = st.m[qt], rowp[D + 1] = st.l[qt];
      }
    }
    __syncthreads();
    if (receiver) {
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) {
        const float* rowp = merge_buf + slot * SLOT_F + (qt * 16 + n) * ROW_F;
        const float m_b = rowp[D], l_b = rowp[D + 1];
        const float m_new = fmaxf(st.m[qt], m_b);
        const float m_use = (m_new == kNegInf) ? 0.f : m_new;
        const float wa = __builtin_amdgcn_exp2f(st.m[qt] - m_use), wb = __builtin_amdgcn_exp2f(m_b - m_use);
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) st.o[qt][j][i] = st.o[qt][j][i] * wa + rowp[16 * j + 4 * g + i] * wb;
        st.l[qt] = st.l[qt] * wa + l_b * wb;
        st.m[qt] = m_new;
      }
    }
    __syncthreads();
  }
  if (wave != 0) return;
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    if (row_s[qt] >= S) continue;
    const float l = st.l[qt];
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* op = p.out + (((int64_t)b * dp.N + head) * S + row_s[qt]) * RS + 4 * g;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      u32x2 w;
      w[0] = pack_bf16x2(st.o[qt][j][0] * inv, st.o[qt][j][1] * inv);
      w[1] = pack_bf16x2(st.o[qt][j][2] * inv, st.o[qt][j][3] * inv);
      if (!PADDED || 16 * j + 4 * g < dp.H) *reinterpret_cast<u32x2*>(op + 16 * j) = w;
    }
  }
}

// ---------------------------------------------------------------------------------
// Many query rows per head (prefill): the four waves of a workgroup own 16*NQT query rows each
// and walk the whole L axis together.  Every 32-token unit of K and V is brought into LDS once
// per workgroup (coalesced 16-byte chunks, the next unit travelling through registers while
// the current one is consumed) and read back by every wave in operand order: K rows directly,
// V token-minor through the LDS transpose read.  No merge: a row's softmax state never leaves
// its wave.  Mask values of the next unit are fetched along with it.
// MASK: 0 none, 1 fp32 mask (element-wise loads), 2 bf16 mask: one 16-byte load per row and unit
// (unaligned where the row length makes it so).
// ---------------------------------------------------------------------------------
constexpr int kCoopWaves = 4;

// One turn of the walk that keeps its units in LDS by direct loads (dense_attn_coop_kernel, plain mask lines): send
// this wave's share of a coming unit into stage `nxt` and take the operands of the unit at hand out of stage `cur`
// (both row-major as in memory, so that every load is 1 KiB of contiguous rows; K with its 16-byte chunks swizzled by
// row for the operand reads, V with swizzled 32-byte pieces for the transposing read), with the score products
// between the K and the V reads.
// The LDS reads are written as instructions, with their own wait: before an LDS read the compiler sees, it waits for
// every outstanding direct-to-LDS load (it cannot tell that the read does not touch what they write) -- the full
// memory latency of the unit just sent, every turn (measured: more than half of the wave cycles).  The reads here
// are of a stage whose loads the caller has waited for (vmcnt, barrier), the loads in flight write other stages.
struct CoopSend {
  const uint16_t* kp;   // this lane's K piece of the coming unit (second load: four rows on, or kp2 where rows are clamped)
  const uint16_t* kp2;
  const uint16_t* vp;   // this lane's V piece (likewise)
  const uint16_t* vp2;
  bool on, whole;       // wave-uniform
};
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
template <int D, int NQT>
__device__ __forceinline__ void coop_stage_turn(const u32x4* cur, u32x4* nxt, const CoopSend& sd, int k_first, int k_at, int v_at,
                                                const u32x4 (&qreg)[NQT][D / 32], f32x4 (&sc)[NQT][2], u32x4 (&vop)[D / 16]) {
  constexpr int KK = D / 32, MT = D / 16, PER = MT / kCoopWaves, ROW_BYTES = D * 2;
  typedef const __attribute__((address_space(1))) void* gptr;
  typedef __attribute__((address_space(3))) void* lptr;
  static_assert(PER == 1 || PER == 2, "one or two loads per operand and wave");
  static_assert(KK == 2 || KK == 4, "head_dim 64 or 128");
  if (sd.on) {
    u32x4* const ks = nxt + k_first * 64;
    u32x4* const vs = nxt + (MT + k_first) * 64;
    __builtin_amdgcn_global_load_lds((gptr)sd.kp, (lptr)ks, 16, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr)sd.vp, (lptr)vs, 16, 0, 0);
    if (PER == 2) {
      if (sd.whole) {  // four rows on: 1024 bytes in memory and in the stage (the immediate offset moves both), the same swizzle
        __builtin_amdgcn_global_load_lds((gptr)sd.kp, (lptr)ks, 16, 4 * ROW_BYTES, 0);
        __builtin_amdgcn_global_load_lds((gptr)sd.vp, (lptr)vs, 16, 4 * ROW_BYTES, 0);
      } else {
        __builtin_amdgcn_global_load_lds((gptr)sd.kp2, (lptr)(ks + 64), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr)sd.vp2, (lptr)(vs + 64), 16, 0, 0);
      }
    }
  }
  // K: rows of token tile t lie four rows on (an immediate offset); the chunk of contraction step kk is one
  // exclusive-or away from that of step 0 (the swizzle key sits in the same bits)
  u32x4 kop[2][KK];
  const uint32_t k_base = lds_address(cur) + k_at;
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    const uint32_t at = k_base ^ (kk << 6);
#pragma unroll
    for (int t = 0; t < 2; ++t)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kop[t][kk]) : "v"(at), "n"(t * 4 * ROW_BYTES) : "memory");
  }
  if constexpr (KK == 4) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(kop[0][0]), "+v"(kop[0][1]), "+v"(kop[0][2]), "+v"(kop[0][3]), "+v"(kop[1][0]), "+v"(kop[1][1]), "+v"(kop[1][2]),
                   "+v"(kop[1][3]));
  } else {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kop[0][0]), "+v"(kop[0][1]), "+v"(kop[1][0]), "+v"(kop[1][1]));
  }
  score_products<D, NQT>(kop, qreg, sc);
  __builtin_amdgcn_sched_barrier(0);  // the products above are issued before any read below
  const uint32_t v_base = lds_address(cur) + v_at;
  u32x2 lo[MT], hi[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const uint32_t at = v_base ^ (j << 5);
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo[j]) : "v"(at) : "memory");
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi[j]) : "v"(at), "n"(4 * ROW_BYTES) : "memory");
  }
  if constexpr (MT == 8) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(lo[0]), "+v"(lo[1]), "+v"(lo[2]), "+v"(lo[3]), "+v"(lo[4]), "+v"(lo[5]), "+v"(lo[6]), "+v"(lo[7]), "+v"(hi[0]),
                   "+v"(hi[1]), "+v"(hi[2]), "+v"(hi[3]), "+v"(hi[4]), "+v"(hi[5]), "+v"(hi[6]), "+v"(hi[7]));
  } else {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[0]), "+v"(lo[1]), "+v"(lo[2]), "+v"(lo[3]), "+v"(hi[0]), "+v"(hi[1]), "+v"(hi[2]), "+v"(hi[3]));
  }
#pragma unroll
  for (int j = 0; j < MT; ++j) vop[j] = u32x4{lo[j][0], lo[j][1], hi[j][0], hi[j][1]};
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) asm volatile("" ::"v"(kop[t][kk]));  // K operands live up to here (see the kernel)
  __builtin_amdgcn_sched_barrier(0);
}

template <int D, int NQT, int MASK, bool PADDED = false>
__global__ __launch_bounds__(64 * kCoopWaves) __attribute__((amdgpu_waves_per_eu(2))) void dense_attn_coop_kernel(
    const DenseMfmaParams dp) {
  constexpr int KK = D / 32;
  constexpr int MT = D / 16;
  constexpr int KROW = D + 8;        // padded K row: the 16 rows of one operand read fall on different banks ...
  constexpr int KHALF = 32;          // ... together with this shift of rows 16..31
  constexpr int VROW = D + 24;       // padded V row for the transposed reads
  constexpr int KSTAGE = 32 * KROW + KHALF;
  constexpr int STAGE = KSTAGE + 32 * VROW;
  constexpr int CH = D / 8;          // 16-byte chunks per row
  constexpr int PER_THREAD = (32 * CH + 64 * kCoopWaves - 1) / (64 * kCoopWaves);
  constexpr bool WHOLE_ROUNDS = (32 * CH) % (64 * kCoopWaves) == 0;  // every thread has a chunk in every round
  constexpr bool HAS_MASK = MASK != 0;
  // (the walk over plain mask lines keeps three units of 2 * MT KiB in the same memory, see below)
  // (at head_dim 256 three such units would leave room for one workgroup per compute unit, and a unit of head_dim 96
  // does not divide into whole loads per wave: that walk is not built for them)
  constexpr bool DIRECT_WALK = D == 64 || D == 128;
  constexpr int STAGE_ELEMS = (!DIRECT_WALK || 2 * STAGE > 3 * MT * 1024) ? 2 * STAGE : 3 * MT * 1024;
  __shared__ __attribute__((aligned(256))) uint16_t stage_mem[STAGE_ELEMS];
  uint16_t(*stage)[STAGE] = reinterpret_cast<uint16_t(*)[STAGE]>(stage_mem);
  const PagedAttnParams& p = dp.base;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), n = lane & 15, g = lane >> 4;
  // Workgroups are dealt to the eight XCDs in turn: keep all row groups of one (batch, head) on
  // one XCD, so that its K / V enter a single L2.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  // Row groups from the last to the first: under a causal mask the later rows read more keys, and
  // the longest workgroups of a head should not be the last ones to start.
  const int pair = (slot / dp.n_qgroups) * 8 + xcd, rg = dp.n_qgroups - 1 - slot % dp.n_qgroups;
  if (pair >= dp.B * dp.N) return;  // uniform over the workgroup
  const int b = pair / dp.N, head = pair % dp.N;
  const int L = dp.L, S = dp.S;
  const int RS = PADDED ? dp.H : D;  // row stride of the tensors, in elements (PADDED: see dense_attn_mfma_kernel)
  const uint16_t* kbase = dp.k + (int64_t)pair * L * RS;
  const uint16_t* vbase = dp.v + (int64_t)pair * L * RS;
  const int row0 = (rg * kCoopWaves + wave) * (NQT * 16);
  const bool wave_has_rows = row0 < S;

  u32x4 qreg[NQT][KK];
  RowState<D, NQT> st;
  int row_s[NQT];
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int s = row0 + qt * 16 + n;
    const bool valid = s < S;
    row_s[qt] = s;
    st.limit[qt] = valid ? L - 1 : -1;
    if (HAS_MASK) {
      const int64_t mb = dp.mB == 1 ? 0 : b, mn = dp.mN == 1 ? 0 : head, ms = dp.mS == 1 ? 0 : (valid ? s : 0);
      st.mask_off[qt] = ((mb * dp.mN + mn) * dp.mS + ms) * (int64_t)L;
    } else {
      st.mask_off[qt] = 0;
    }
    st.m[qt] = kNegInf, st.m_top[qt] = kNegInf, st.m_neg[qt] = 0.f;
    st.l[qt] = 0.f;
    const uint16_t* qp = p.q + ((int64_t)pair * S + (valid ? s : 0)) * RS + 8 * g;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      qreg[qt][kk] = (valid && (!PADDED || 32 * kk + 8 * g < dp.H)) ? *reinterpret_cast<const u32x4*>(qp + kk * 32) : z;
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) st.o[qt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  u32x4 pre_k[PER_THREAD], pre_v[PER_THREAD];
  u32x4 pre_m[MASK == 2 ? NQT : 1], cur_m[MASK == 2 ? NQT : 1];  // raw bf16 mask values (MASK == 2)
  MaskRegs<NQT> mnext, mcur;                                      // fp32 values (MASK == 1)
  auto fetch = [&](int u, auto with_mask) {
    constexpr int MODE = decltype(with_mask)::value ? MASK : 0;
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = tid + i * 64 * kCoopWaves, r = c / CH, ch = c % CH;
      if (!WHOLE_ROUNDS && c >= 32 * CH) break;
      const int64_t off = (int64_t)min(L - 1, 32 * u + r) * RS + ch * 8;  // rows past the end are masked later
      pre_k[i] = pre_v[i] = u32x4{0u, 0u, 0u, 0u};
      if (!PADDED || ch * 8 < dp.H) {
        pre_k[i] = *reinterpret_cast<const u32x4*>(kbase + off);
        pre_v[i] = *reinterpret_cast<const u32x4*>(vbase + off);
      }
    }
    if (MODE == 2) {
      const int tok = 32 * u + 8 * g;
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) {
        const uint16_t* line = static_cast<const uint16_t*>(p.mask) + st.mask_off[qt];
        if (tok + 8 <= L) {
          pre_m[qt] = load16_unaligned(line + tok);
        } else {  // the end of a line whose length is no multiple of 8 (columns past it: any value, cut off later)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint32_t lo = tok + 2 * e < L ? line[tok + 2 * e] : 0u, hi = tok + 2 * e + 1 < L ? line[tok + 2 * e + 1] : 0u;
            pre_m[qt][e] = lo | (hi << 16);
          }
        }
      }
    } else if (MODE == 1) {
      const int tok = 32 * u + 8 * g;
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt)
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          float a = kNegInf;
          if (tok + c < L) {
            if (p.mask_is_f32)
              a = static_cast<const float*>(p.mask)[st.mask_off[qt] + tok + c];
            else
              a = bf16_bits_to_f32(static_cast<const uint16_t*>(p.mask)[st.mask_off[qt] + tok + c]);
          }
          mnext.a[qt][c] = fmaxf(a, kMaskFloor);
        }
    }
  };
  auto park = [&](int buf, auto with_mask) {
    constexpr int MODE = decltype(with_mask)::value ? MASK : 0;
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = tid + i * 64 * kCoopWaves, r = c / CH, ch = c % CH;
      if (!WHOLE_ROUNDS && c >= 32 * CH) break;
      *reinterpret_cast<u32x4*>(&stage[buf][r * KROW + (r >= 16 ? KHALF : 0) + ch * 8]) = pre_k[i];
      *reinterpret_cast<u32x4*>(&stage[buf][KSTAGE + r * VROW + ch * 8]) = pre_v[i];
    }
    if (MODE == 2) {
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) cur_m[qt] = pre_m[qt];
    } else if (MODE == 1) {
      mcur = mnext;
    }
  };

  typedef short tr_v4 __attribute__((ext_vector_type(4)));
  typedef tr_v4 __attribute__((address_space(3))) * tr_ptr;
  // One unit out of its stage: K rows in operand order for the scores, then V token-minor through the LDS
  // transpose read while the score products run.  K and V operands sit in registers of their own: the K
  // operands are kept alive (an empty asm statement that takes them as inputs, fenced by scheduling barriers)
  // until every V read has been issued, so no V read can be given a register the score products read from.
  // An LDS read that returns into a register which a matrix instruction issued earlier has yet to fetch (one
  // queued behind the accumulator of the instruction before it fetches its A / B operands late) is a
  // write-after-read hazard that neither the hardware nor the compiler's wait-state insertion covers; with
  // the two operand sets disjoint inside a unit, and a workgroup barrier between units, it cannot occur.
  // by_mask: the unit's mask values decide (all of [0, L) is walked); else the rows' own limits and `first` do
  // (plain mask lines, see below), and the mask values are not looked at.
  // before_weights(): called once the unit's operands are in their registers and the score products are issued (not
  // at all for a unit that is skipped) -- the place for loads whose registers should not be alive next to the K operands.
  auto unit = [&](int cur, int t0, auto full_tag, auto by_mask, int tok_end, int first, auto before_weights) {
    constexpr bool FULL = decltype(full_tag)::value;
    constexpr bool BY_MASK = decltype(by_mask)::value && HAS_MASK;
    if (BY_MASK && MASK == 2) {
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) mask_line_from_bf16x8(cur_m[qt], mcur.a[qt]);
    }
    if (BY_MASK && unit_is_masked_out<D, NQT>(mcur, st)) return;  // e.g. above the diagonal of a causal mask
    u32x4 kop[2][KK], vop[MT];
    // K: token 8*(n/4) + 4*tile + n%4 of the unit, dims 32*kk + 8g ..
    const int r0 = 8 * (n >> 2) + (n & 3);
    const uint16_t* ks = &stage[cur][r0 * KROW + (r0 >= 16 ? KHALF : 0) + 8 * g];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kop[t][kk] = *reinterpret_cast<const u32x4*>(ks + t * 4 * KROW + kk * 32);
    f32x4 sc[NQT][2];
    score_products<D, NQT>(kop, qreg, sc);
    __builtin_amdgcn_sched_barrier(0);  // the products above are issued before any read below
    // V: dim 16j + n of tokens 8g .. 8g+7 (see the transposed read in the kernel above)
    const uint16_t* tr_base = &stage[cur][KSTAGE + (8 * g + (n >> 2)) * VROW + 4 * (n & 3)];
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const tr_v4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(tr_base + 16 * j));
      const tr_v4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(tr_base + 4 * VROW + 16 * j));
      const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      vop[j] = u32x4{l2[0], l2[1], h2[0], h2[1]};
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) asm volatile("" ::"v"(kop[t][kk]));  // K operands live up to here
    __builtin_amdgcn_sched_barrier(0);
    before_weights();
    softmax_and_output<D, NQT, BY_MASK, FULL>(sc, vop, st, p, t0, tok_end, first, g, mcur);
  };
  // Units past the last one that matters to any row of the workgroup are not walked at all: with a
  // bf16 mask every wave first looks from the end of its rows' mask lines backwards for the last
  // value above the floor (several units per round trip), until each of its rows has shown one; a
  // row that shows none (masked everywhere: it ends as the average of V) keeps every unit.  What lies
  // past the workgroup's last such unit weighs exactly 0 for rows that have all met a real score by
  // then: the upper triangle of a causal mask, half of a prefill.
  // Summary of the mask (optional): per mask line the last column above the floor and, if the line is plain (0 from
  // a first column to that last one, at the floor elsewhere: a causal mask, padded or not), the first one.  When every
  // row of the workgroup has a plain line and all start at the same column, the rows are walked like rows without a
  // mask tensor -- that first column, their own last column -- and the mask is not read (`plain`).
  bool plain = false;
  int f_min = 0x7fffffff, f_max = -1, wg_last = -1, l_min = 0x7fffffff;
  const bool summarised = DIRECT_WALK && HAS_MASK && dp.line_last && dp.line_first;
  const int64_t line0 = ((dp.mB == 1 ? 0 : (int64_t)b) * dp.mN + (dp.mN == 1 ? 0 : head)) * dp.mS;
  if (summarised) {
#pragma unroll
    for (int i = 0; i < NQT; ++i) {
      const int r = rg * (kCoopWaves * NQT * 16) + i * 64 + lane;
      if (r < S) {
        const int64_t line = line0 + (dp.mS == 1 ? 0 : r);
        const int f = dp.line_first[line], l = dp.line_last[line];
        f_min = min(f_min, f), f_max = max(f_max, f), wg_last = max(wg_last, l), l_min = min(l_min, l);
      }
    }
#pragma unroll
    for (int o = 1; o < 64; o *= 2) {
      f_min = min(f_min, __shfl_xor(f_min, o, 64)), f_max = max(f_max, __shfl_xor(f_max, o, 64));
      wg_last = max(wg_last, __shfl_xor(wg_last, o, 64)), l_min = min(l_min, __shfl_xor(l_min, o, 64));
    }
    f_min = __builtin_amdgcn_readfirstlane(f_min), f_max = __builtin_amdgcn_readfirstlane(f_max);
    wg_last = __builtin_amdgcn_readfirstlane(wg_last), l_min = __builtin_amdgcn_readfirstlane(l_min);
    plain = f_min >= 0 && f_min == f_max;  // (-1 marks a line that is not plain)
  }
  int units = (L + 31) / 32;
  if (summarised) {
    if (l_min >= 0) units = min(units, wg_last / 32 + 1);  // every row has a real score: nothing past the last of them counts
  } else if (MASK == 2) {
    __shared__ int last_needed[kCoopWaves];
    constexpr int ROUND = 4;  // units looked at per round trip (16 measured slower: the volume counts, not the trips)
    int mine = -1;            // last unit in which this lane's columns of a (real) row hold a value above the floor
    bool shown[NQT];
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) shown[qt] = false;
    bool open_rows = wave_has_rows;
    for (int top = units - 1; top >= 0 && open_rows; top -= ROUND) {
      u32x4 raw[ROUND][NQT];
#pragma unroll
      for (int r = 0; r < ROUND; ++r) {
        const int tok = 32 * max(top - r, 0) + 8 * g;
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
          const uint16_t* line = static_cast<const uint16_t*>(p.mask) + st.mask_off[qt];
          if (tok + 8 <= L) {
            raw[r][qt] = load16_unaligned(line + tok);
          } else {  // columns that do not exist count as masked
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const uint32_t lo = tok + 2 * e < L ? line[tok + 2 * e] : 0xffffu, hi = tok + 2 * e + 1 < L ? line[tok + 2 * e + 1] : 0xffffu;
              raw[r][qt][e] = lo | (hi << 16);
            }
          }
        }
      }
      bool all_shown = true;
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) {
        int row_last = -1;
#pragma unroll
        for (int r = ROUND - 1; r >= 0; --r) {  // ascending unit index: the largest hit wins
          const uint32_t w = min_u16x2(min_u16x2(raw[r][qt][0], raw[r][qt][1]), min_u16x2(raw[r][qt][2], raw[r][qt][3]));
          const bool above = min(w & 0xffffu, w >> 16) < (kMaskFloorBf16x2 & 0xffffu);
          if (above && top - r >= 0 && st.limit[qt] >= 0) row_last = max(row_last, top - r);
        }
        mine = max(mine, row_last);
        // the row's four lanes (n, 0..3) look at different columns: it has shown a value if any of them has
        int any = row_last >= 0 || shown[qt];
        any |= __shfl_xor(any, 16, 64);
        any |= __shfl_xor(any, 32, 64);
        shown[qt] = any != 0;
        all_shown = all_shown && (st.limit[qt] < 0 || shown[qt]);
      }
      open_rows = !__all(all_shown);
    }
    int wave_last = open_rows ? units - 1 : mine;  // a row never showed a value: keep everything
#pragma unroll
    for (int off = 1; off < 64; off *= 2) wave_last = max(wave_last, __shfl_xor(wave_last, off, 64));
    if (!wave_has_rows) wave_last = -1;
    if (lane == 0) last_needed[wave] = wave_last;
    __syncthreads();
    int wg_last = last_needed[0];
#pragma unroll
    for (int w = 1; w < kCoopWaves; ++w) wg_last = max(wg_last, last_needed[w]);
    units = __builtin_amdgcn_readfirstlane(min(units, wg_last + 1));
  }
  // One loop per kind of unit -- masked before the rows' whole units, whole, masked after them, needed by other waves
  // only -- so that the accumulators have one path through each loop body.
  if constexpr (DIRECT_WALK) if (plain) {
    {
      int min_limit = 0x7fffffff, mine = -1;
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) {
        if (st.limit[qt] >= 0) {
          st.limit[qt] = dp.line_last[line0 + (dp.mS == 1 ? 0 : row_s[qt])];
          min_limit = min(min_limit, st.limit[qt]);
          mine = max(mine, st.limit[qt]);
        }
      }
#pragma unroll
      for (int o = 1; o < 64; o *= 2) min_limit = min(min_limit, __shfl_xor(min_limit, o, 64)), mine = max(mine, __shfl_xor(mine, o, 64));
      min_limit = __builtin_amdgcn_readfirstlane(min_limit);
      const int first = f_min;
      const int wave_end = wave_has_rows ? __builtin_amdgcn_readfirstlane(mine) + 1 : 0;
      const int u0 = first / 32;
      const int u_end = max(wg_last / 32 + 1, u0 + 1);  // (every line has a column: u_end > u0)
      const int u_mine = min(max((wave_end + 31) / 32, u0), u_end);
      const int u_whole_end = min(max((min(wave_end - 1, min_limit) + 1) / 32, u0), u_mine);
      const int u_whole_begin = min((first + 31) / 32, u_whole_end);
      // In this walk K / V go from memory straight into LDS (global_load_lds_dwordx4: lane l of a load lands at
      // base + 16 l), two units ahead of their use (three stages).  Both operands stay row-major, so that a load is 1 KiB of
      // contiguous rows, and are swizzled for the reads that follow (the padding the register-staged layout uses cannot
      // be had inside a 1 KiB load): K with the 16-byte chunks of row r at chunk index (chunk ^ kw(r)), V with the
      // 32-byte pieces of row r at piece index (piece ^ sw(r)), so that the sixteen rows one operand read or one
      // transposing read touches fall on different banks.  (K fetched in operand order instead -- lane (n, g) of load
      // (t, kk) the 16 bytes it reads back: sixteen 64-byte runs per load -- measured 2.6 % slower.)
      constexpr int UNIT_CHUNKS = 2 * MT * 64;  // 16-byte pieces of a unit: K, then V
      constexpr int PER = MT / kCoopWaves;      // K loads and V loads per wave and unit
      constexpr int ROWS_PER_LOAD = 64 / CH, ROW_BYTES = D * 2;
      static_assert(3 * UNIT_CHUNKS * 16 <= STAGE_ELEMS * 2, "the three stages of this walk fit the kernel's LDS");
      u32x4* const dstage = reinterpret_cast<u32x4*>(stage_mem);
      auto sw = [](int r) { return D == 128 ? 2 * (r >> 3) + ((r & 3) >> 1) : (r >> 3) & 3; };  // < 32-byte pieces per row
      const int k_first = wave * PER;
      // (the sixteen rows of one K operand read are 8a + b + 4t, a and b below 4: kw tells them apart and is the same
      // four rows on, so that a wave's second load is the first one's lane addresses plus an immediate offset)
      auto kw = [](int r) { return D == 128 ? ((r >> 3) << 2) | (r & 3) : 2 * (r >> 3) + ((r & 3) >> 1); };
      const int k_row = k_first * ROWS_PER_LOAD + lane / CH;
      const int k_col = 8 * ((lane % CH) ^ kw(k_row));
      const int v_row = k_first * ROWS_PER_LOAD + lane / CH;
      const int v_col = 8 * ((((lane % CH) >> 1) ^ sw(v_row)) * 2 + (lane & 1));
      auto sending = [&](int u, bool on) {  // the loads of unit u (rows past the end are clamped, and masked later)
        CoopSend sd;
        sd.on = on, sd.whole = 32 * (u + 1) <= L;
        sd.kp = kbase + (int64_t)min(32 * u + k_row, L - 1) * D + k_col;
        sd.kp2 = kbase + (int64_t)min(32 * u + k_row + ROWS_PER_LOAD, L - 1) * D + k_col;
        sd.vp = vbase + (int64_t)min(32 * u + v_row, L - 1) * D + v_col;
        sd.vp2 = vbase + (int64_t)min(32 * u + v_row + ROWS_PER_LOAD, L - 1) * D + v_col;
        return sd;
      };
      // byte offset (inside a stage) of this lane's first transposing read: row 8g + n/4, piece n%4 of 32-byte slot
      // (0 ^ sw); slot j is one exclusive-or away, the rows four on one immediate offset
      // byte offset of this lane's K read of token tile 0, contraction step 0: row 8 (n / 4) + n % 4, chunk g
      const int k_r0 = 8 * (n >> 2) + (n & 3);
      const int k_at = k_r0 * ROW_BYTES + ((g ^ kw(k_r0)) << 4);
      const int v_r0 = 8 * g + (n >> 2);
      const int v_at = (MT * 64 * 16 + v_r0 * ROW_BYTES + (n & 3) * 8) ^ (sw(v_r0) << 5);
      // Two units ahead: a unit's loads take longer than a unit's arithmetic here.  Unit u is complete in its stage
      // once every wave's loads of it are back -- all but the newest unit's, counted, then the barrier; the same
      // barrier says that every wave has taken unit u - 1 out of the stage the next loads reuse.  (Wait and barrier
      // are written out: the library barrier waits for every outstanding load.)
      auto send_only = [&](int u, int s) {  // prologue: nothing to read yet
        const CoopSend sd = sending(u, true);
        typedef const __attribute__((address_space(1))) void* gptr;
        typedef __attribute__((address_space(3))) void* lptr;
        u32x4* const nxt = dstage + s * UNIT_CHUNKS;
        u32x4* const ks = nxt + k_first * 64;
        __builtin_amdgcn_global_load_lds((gptr)sd.kp, (lptr)ks, 16, 0, 0);
        if (PER == 2) __builtin_amdgcn_global_load_lds((gptr)sd.kp2, (lptr)(ks + 64), 16, 0, 0);
        u32x4* const vs = nxt + (MT + k_first) * 64;
        __builtin_amdgcn_global_load_lds((gptr)sd.vp, (lptr)vs, 16, 0, 0);
        if (PER == 2) __builtin_amdgcn_global_load_lds((gptr)sd.vp2, (lptr)(vs + 64), 16, 0, 0);
      };
      // (a wait the compiler sees, for the query rows' loads: its own wait for them would otherwise land inside the
      // loop, at count 0, behind the direct-to-LDS loads of the coming units)
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      send_only(u0, 0);
      if (u0 + 1 < u_end) send_only(u0 + 1, 1);
      int cur = 0;  // stage of the unit at hand: (u - u0) % 3
      auto walk = [&](int from, int to, auto kind) {  // kind: 0 masked unit, 1 whole unit, 2 nothing to compute
        constexpr int KIND = decltype(kind)::value;
        for (int u = from; u < to; ++u) {
          if (u + 1 < u_end) {
            if (PER == 2) __builtin_amdgcn_s_waitcnt(0x0074);  // vmcnt(4) lgkmcnt(0)
            else __builtin_amdgcn_s_waitcnt(0x0072);           // vmcnt(2) lgkmcnt(0)
          } else {
            __builtin_amdgcn_s_waitcnt(0x0070);                // vmcnt(0) lgkmcnt(0)
          }
          asm volatile("s_barrier" ::: "memory");
          const int nxt = cur == 0 ? 2 : cur - 1;
          const CoopSend sd = sending(u + 2, u + 2 < u_end);
          if (KIND == 2) {
            if (sd.on) send_only(u + 2, nxt);
          } else {
            f32x4 sc[NQT][2];
            u32x4 vop[MT];
            coop_stage_turn<D, NQT>(dstage + cur * UNIT_CHUNKS, dstage + nxt * UNIT_CHUNKS, sd, k_first, k_at, v_at, qreg, sc, vop);
            if (KIND == 0) softmax_and_output<D, NQT, false, false>(sc, vop, st, p, 32 * u, wave_end, first, g);
            if (KIND == 1) softmax_and_output<D, NQT, false, true>(sc, vop, st, p, 32 * u, wave_end, first, g);
          }
          cur = cur == 2 ? 0 : cur + 1;
        }
      };
      walk(u0, u_whole_begin, std::integral_constant<int, 0>{});
      walk(u_whole_begin, u_whole_end, std::integral_constant<int, 1>{});
      walk(u_whole_end, u_mine, std::integral_constant<int, 0>{});
      walk(u_mine, u_end, std::integral_constant<int, 2>{});
    }
  }
  if (!plain) {
    // Whole units in the loop, the partial last one (if any) after it: the loop body has one shape.
    const int whole = min(L / 32, units);
    fetch(0, std::true_type{});
    park(0, std::true_type{});
    __syncthreads();
    for (int u = 0; u < whole; ++u) {
      const int cur = u & 1;
      if constexpr (D <= 128) {
        fetch(min(u + 1, units - 1), std::true_type{});  // unconditional: no branch between a load and the wait for it
        if (wave_has_rows) unit(cur, 32 * u, std::true_type{}, std::true_type{}, L, 0, [] {});
      } else {
        // head_dim 256: the next unit's loads are issued behind the score products, when the K operands' 64 registers
        // are free again -- with them issued first, about 90 registers spill
        bool sent = false;
        if (wave_has_rows) {
          unit(cur, 32 * u, std::true_type{}, std::true_type{}, L, 0, [&] {
            fetch(min(u + 1, units - 1), std::true_type{});
            sent = true;
          });
        }
        if (!sent) fetch(min(u + 1, units - 1), std::true_type{});
      }
      park(cur ^ 1, std::true_type{});
      __syncthreads();
    }
    if (whole < units && wave_has_rows) unit(whole & 1, 32 * whole, std::false_type{}, std::true_type{}, L, 0, [] {});
  }

#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    float l = st.l[qt];
    l += xor_lanes(l, 16);
    l += xor_lanes(l, 32);
    if (row_s[qt] >= S) continue;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* op = p.out + ((int64_t)pair * S + row_s[qt]) * RS + 4 * g;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      u32x2 w;
      w[0] = pack_bf16x2(st.o[qt][j][0] * inv, st.o[qt][j][1] * inv);
      w[1] = pack_bf16x2(st.o[qt][j][2] * inv, st.o[qt][j][3] * inv);
      if (!PADDED || 16 * j + 4 * g < dp.H) *reinterpret_cast<u32x2*>(op + 16 * j) = w;
    }
  }
}

// Launches the dense bf16 kernel; returns false when the shape is not one it handles.
// workspace (optional): room for the summary of the mask, two ints per mask line (dense_mfma_workspace_bytes).
bool launch_dense_mfma(const void* q, const void* k, const void* v, void* out, int B, int N, int S, int L, int H_real,
                       const void* mask, bool mask_is_f32, int mB, int mN, int mS, float scale, void* workspace,
                       size_t workspace_bytes, hipStream_t stream) {
  // Head sizes between 64 and 96 that are a multiple of 8 (OPT-2.7B's 80) run in the 96 build, their rows read as if
  // padded with zeros (PADDED); `scale` is the caller's, of the real head size.
  const bool padded = H_real > 64 && H_real < 96 && H_real % 8 == 0;
  const int H = padded ? 96 : H_real;
  if ((H != 64 && H != 96 && H != 128 && H != 256) || L < 1) return false;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || (reinterpret_cast<uintptr_t>(out) & 7u)) return false;
  DenseMfmaParams dp = {};
  dp.base.q = static_cast<const uint16_t*>(q);
  dp.base.out = static_cast<uint16_t*>(out);
  dp.base.mask = mask, dp.base.mask_is_f32 = mask_is_f32, dp.base.mask_len = L;
  dp.base.scale_log2 = scale * kLog2e;
  dp.base.scale = scale;
  dp.k = static_cast<const uint16_t*>(k), dp.v = static_cast<const uint16_t*>(v);
  dp.B = B, dp.N = N, dp.S = S, dp.L = L, dp.H = H_real, dp.mB = mB, dp.mN = mN, dp.mS = mS;
  const int tiles = (S + 15) / 16;
  const bool coop_built = H == 64 || H == 96 || H == 128 || H == 256;  // other head sizes: the split-L kernel, one launch of as many row groups as it takes
  if ((tiles > 4 || (H == 256 && tiles > 1)) && coop_built) {
    // prefill-sized: rows of a head share its K / V through LDS
    const int mode = !mask ? 0 : (mask_is_f32 ? 1 : 2);
    int cnqt = H == 256 ? 1 : 2;  // (two tiles of head_dim 256 do not fit the register file)
    dp.n_qgroups = (tiles + kCoopWaves * cnqt - 1) / (kCoopWaves * cnqt);
    // too few workgroups: halve their rows; so does the element-wise mask path at head_dim 128, whose
    // two-tile form does not fit the register file
    if ((long long)B * N * dp.n_qgroups < compute_units() || (mode == 1 && (H == 128 || H == 96))) {
      cnqt = 1;
      dp.n_qgroups = (tiles + kCoopWaves - 1) / kCoopWaves;
    }
    const long long pairs8 = ((long long)B * N + 7) / 8 * 8;
    const long long cblocks = pairs8 * dp.n_qgroups;
    if (cblocks >= (1ll << 31)) return false;
    const dim3 cgrid((unsigned)cblocks), cblock(64 * kCoopWaves);
    const size_t lines = mask ? (size_t)mB * mN * mS : 0;
    if (mask && workspace && (reinterpret_cast<uintptr_t>(workspace) & 3u) == 0 && lines < (1u << 31) &&
        workspace_bytes >= 2 * lines * sizeof(int32_t)) {
      int32_t* last = static_cast<int32_t*>(workspace);
      hipLaunchKernelGGL(dense_mask_lines_kernel, dim3((unsigned)lines), dim3(64), 0, stream, mask, mask_is_f32 ? 1 : 0, L, last, last + lines);
      dp.line_last = last, dp.line_first = last + lines;
    }
#define PACE_COOP(D_, Q_, M_) hipLaunchKernelGGL((dense_attn_coop_kernel<D_, Q_, M_>), cgrid, cblock, 0, stream, dp)
#define PACE_COOP_M(D_, Q_) \
  do { if (mode == 0) PACE_COOP(D_, Q_, 0); else if (mode == 1) PACE_COOP(D_, Q_, 1); else PACE_COOP(D_, Q_, 2); } while (0)
    if (H == 256) PACE_COOP_M(256, 1);
    else if (padded) {
#define PACE_COOP_P(Q_, M_) hipLaunchKernelGGL((dense_attn_coop_kernel<96, Q_, M_, true>), cgrid, cblock, 0, stream, dp)
      if (cnqt == 2) { if (mode == 0) PACE_COOP_P(2, 0); else if (mode == 1) PACE_COOP_P(2, 1); else PACE_COOP_P(2, 2); }
      else { if (mode == 0) PACE_COOP_P(1, 0); else if (mode == 1) PACE_COOP_P(1, 1); else PACE_COOP_P(1, 2); }
#undef PACE_COOP_P
    }
    else if (H == 96) { if (cnqt == 2) PACE_COOP_M(96, 2); else PACE_COOP_M(96, 1); }
    else if (H == 128) { if (cnqt == 2) PACE_COOP_M(128, 2); else PACE_COOP_M(128, 1); }
    else { if (cnqt == 2) PACE_COOP_M(64, 2); else PACE_COOP_M(64, 1); }
#undef PACE_COOP_M
#undef PACE_COOP
    return true;
  }
  const int nqt = (tiles >= 2 && H != 256) ? 2 : 1;  // two tiles of head_dim 256 do not fit the register file
  dp.n_qgroups = (tiles + nqt - 1) / nqt;
  const long long blocks = (long long)B * N * dp.n_qgroups;
  if (blocks >= (1ll << 31)) return false;
  const dim3 grid((unsigned)blocks), block(H > 128 ? 128 : 256);
  const bool m = mask != nullptr;
  const bool once = dp.n_qgroups == 1;
  // (head_dim 256: two waves per SIMD once there are more workgroups than compute units hold at one wave per SIMD)
  const bool packed = H == 256 && blocks > 2ll * compute_units();
#define PACE_DENSE1(D_, Q_, M_, O_)                                                                              \
  do {                                                                                                          \
    if (D_ == 256 && packed) hipLaunchKernelGGL((dense_attn_mfma_kernel<D_, Q_, M_, O_, 2>), grid, block, 0, stream, dp); \
    else hipLaunchKernelGGL((dense_attn_mfma_kernel<D_, Q_, M_, O_>), grid, block, 0, stream, dp);                \
  } while (0)
#define PACE_DENSE(D_, Q_, M_) do { if (once) PACE_DENSE1(D_, Q_, M_, true); else PACE_DENSE1(D_, Q_, M_, false); } while (0)
  if (padded) {
#define PACE_DENSE_P(Q_, M_)                                                                                              \
  do {                                                                                                                    \
    if (once) hipLaunchKernelGGL((dense_attn_mfma_kernel<96, Q_, M_, true, 2, true>), grid, block, 0, stream, dp);         \
    else hipLaunchKernelGGL((dense_attn_mfma_kernel<96, Q_, M_, false, 2, true>), grid, block, 0, stream, dp);             \
  } while (0)
    if (nqt == 2) { if (m) PACE_DENSE_P(2, true); else PACE_DENSE_P(2, false); }
    else { if (m) PACE_DENSE_P(1, true); else PACE_DENSE_P(1, false); }
#undef PACE_DENSE_P
    return true;
  }
  for_head_dim(H, [&](auto d) {
    constexpr int DIM = decltype(d)::value;
    if constexpr (DIM != 256) {
      if (nqt == 2) {
        if (m) PACE_DENSE(DIM, 2, true); else PACE_DENSE(DIM, 2, false);
        return;
      }
    }
    if (m) PACE_DENSE(DIM, 1, true); else PACE_DENSE(DIM, 1, false);
  });
#undef PACE_DENSE1
#undef PACE_DENSE
  return true;
}

// Scratch the dense bf16 path can use for these sizes (0: none): the summary of an explicit mask on prefill-sized
// launches.
size_t dense_mfma_workspace_bytes(int S, int H, int mB, int mN, int mS, bool has_mask) {
  const int tiles = (S + 15) / 16;
  if (!has_mask || tiles <= 4 || (H != 64 && H != 128)) return 0;
  return 2 * (size_t)mB * mN * mS * sizeof(int32_t);
}

}  // namespace pace_kv

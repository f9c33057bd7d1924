// Dense scaled-dot-product attention for gfx950: the body of the torch op
// pace::attention for arbitrary head_dim, fp32 or bf16 tensors and an arbitrary
// additive mask broadcast from [mB][mN][mS][L].
//
// General kernel (fp32 tensors, head sizes the bf16 kernels are not built for): fp32 arithmetic on
// the matrix cores (v_mfma_f32_16x16x4_f32), online softmax, the [S][L] score matrix never
// materialised.  A wave owns 16 query rows of one (batch, head) and walks its share of the keys in
// 16-token tiles; with lane = (n, g), n = lane % 16, g = lane / 16:
//   S^T tile = K[16 tokens x HP dims] * Q^T[HP dims x 16 rows], HP/4 steps of 4 dims: in step s lane
//       (n, g) supplies dim g*HP/4 + s of K row n (A operand) and of Q row n (B operand) -- any
//       assignment of dims to steps gives the same sum, this one lets a lane read its dims of a row
//       as one contiguous run; the result leaves lane (n, g) with tokens 4g..4g+3 of query row n;
//   O^T tile = V^T[16 dims x 16 tokens] * P^T[16 tokens x 16 rows], 4 steps: in step i lane (n, g)
//       supplies V[token 4g+i][dim 16j+n] and its own probability of token 4g+i,
// so probabilities never leave their lane and the state of query row n lives in lanes (n, 0..3).
// The four waves of a workgroup take four row groups, or split the keys of fewer row groups among
// themselves (few query rows: decode) and merge through LDS.  Four row groups of fp32 rows share
// the tiles they walk: the workgroup fetches each once and hands it round through LDS (COOP below);
// elsewhere every wave takes its operands straight from global memory.  The same body walks a pool of
// fp32 rows through its block table (PAGED).
#include "attn_core.h"

namespace pace_kv {

template <typename T>
__device__ __forceinline__ float load_f32(const T* p);
template <>
__device__ __forceinline__ float load_f32<float>(const float* p) {
  return *p;
}
template <>
__device__ __forceinline__ float load_f32<uint16_t>(const uint16_t* p) {
  return bf16_bits_to_f32(*p);
}

// e^x for x <= 0 as the hardware's 2^(x log2 e): the product's rounding costs |x| 2^-24 relative in the result
// (3e-6 at x = -50, where the weight is 2e-22), two instructions against the library routine's ten.
__device__ __forceinline__ float exp_of(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }

// Four consecutive elements as fp32 (p 16- resp. 8-byte aligned).
__device__ __forceinline__ f32x4 load4_f32(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load4_f32(const uint16_t* p) {
  const u32x2 w = *reinterpret_cast<const u32x2*>(p);
  return f32x4{bf16_bits_to_f32(w[0] & 0xffffu), __uint_as_float(w[0] & 0xffff0000u), bf16_bits_to_f32(w[1] & 0xffffu),
               __uint_as_float(w[1] & 0xffff0000u)};
}
// Four elements of a K / V row.  ONCE: the row is read by one row group and nobody after it (few query rows: decode);
// fetched non-temporally, which lifts a stream on this GPU from 6.0 - 6.25 to 7.0 - 7.25 TB/s -- provided every
// cache line is consumed by few instructions (past the L1 each instruction fetches its lines again; see ONCE below).
template <bool ONCE>
__device__ __forceinline__ f32x4 load4_kv(const float* p) {
  if constexpr (ONCE) return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
  else return load4_f32(p);
}
template <bool ONCE>
__device__ __forceinline__ f32x4 load4_kv(const uint16_t* p) { return load4_f32(p); }
// Two consecutive elements (p 8- resp. 4-byte aligned).
__device__ __forceinline__ f32x2 load2_f32(const float* p) { return *reinterpret_cast<const f32x2*>(p); }
__device__ __forceinline__ f32x2 load2_f32(const uint16_t* p) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
  return f32x2{bf16_bits_to_f32(w & 0xffffu), __uint_as_float(w & 0xffff0000u)};
}
__device__ __forceinline__ void store2_out(float* p, f32x2 v) { *reinterpret_cast<f32x2*>(p) = v; }
__device__ __forceinline__ void store2_out(uint16_t* p, f32x2 v) { *reinterpret_cast<uint32_t*>(p) = pack_bf16x2(v[0], v[1]); }
__device__ __forceinline__ void store4_out(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4_out(uint16_t* p, f32x4 v) {
  *reinterpret_cast<u32x2*>(p) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
}
__device__ __forceinline__ void store_out(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_out(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }

struct DenseParams {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  const void* mask;
  int32_t B, N, S, L, H;
  int32_t mB, mN, mS;
  int32_t l_split;  // waves of a workgroup that share one row group and split its keys: 1, 2 or 4
  float scale;
  // PAGED (attn_paged_f32_kernel): K / V rows come out of a pool of fp32 rows through a block table (one 16-token
  // tile is one block), N counts KV heads, the query rows of a KV head are those of its n_rep query heads one
  // after the other (row r: head r / S of the group, token r % S), q / out / mask are addressed by strides, the
  // length is the sequence's own and L is unused.
  const int32_t* table;
  const int32_t* seq_lens;
  const int32_t* len_bias_dev;
  const int32_t* kv_start;
  int64_t k_bs, k_hs, v_bs, v_hs, q_sb, q_sh, q_ss, o_sb, o_sh, o_ss, m_sb, m_ss;
  int32_t table_stride, len_bias, num_blocks, n_rep, causal, mask_len;
  // n_split > 1: the keys of a row group are cut over n_split workgroups (a batch that does not fill the GPU alone);
  // each leaves (o unnormalised, m, l) per row in `part` ([row][n_split][H + 4] floats), attn_paged_f32_merge_kernel ends.
  int32_t n_split;
  float* part;
  // PAGED with a fused append (FUSED): the last n_new tokens of every sequence are read from k_new / v_new
  // ([batch][KV heads][n_new][H] floats, element strides n_sb / n_sh / n_st) instead of from the pool, and the first
  // workgroup of every (sequence, KV head) stores them into their pool rows.
  const float* k_new;
  const float* v_new;
  int64_t n_sb, n_sh, n_st;
  int32_t n_new;
};

// HP: head size rounded up to the next size built (dims >= H read as zero).  VEC: H is a multiple
// of 4, so a lane's run of a row can be read four elements at a time.
// AHEAD: the operands of the next tile are fetched while this one is computed (a second set of registers: one
// wave per SIMD at head size 128).  It pays where the launch is bound by memory (few query rows: +8 % on an fp32
// decode step) and costs 10 % where it is bound by the matrix cores, so the launcher picks.
// EXACT: H == HP (and VEC): no bound on a dim is checked anywhere, which is a third of the vector instructions of a tile.
// COOP (row groups that do not share their keys with other waves, fp32 rows): the four waves of a workgroup walk the
// same keys, so the workgroup fetches every tile once -- 16 bytes per thread and load, a tile ahead, in registers
// over the tile's arithmetic -- and hands it round through LDS (two stages, one barrier per tile); rows keep their
// order there with their 16-byte chunks rotated by the row number, which keeps the operand reads of sixteen rows
// (the first product) and of sixteen chunks of a row (the second) off each other's banks; a head size below the built
// one is padded with zeros on the way in.  Each wave fetching its
// own operands from memory held the launch at 65 % of what the arithmetic alone takes.
template <typename T, typename MT, int HP, bool VEC, bool AHEAD, bool EXACT, bool PAGED, bool COOP = false, bool FUSED = false>
__device__ __forceinline__ void attn_dense_body(const DenseParams& p) {
  static_assert(!FUSED || (PAGED && !COOP), "the fused append belongs to the pool's launches of few query rows");
  static_assert(!COOP || (VEC && !AHEAD && sizeof(T) == 4), "the cooperative walk: fp32 rows of a multiple of four dims");
  static_assert(!EXACT || VEC, "a head size that is one of the built ones is a multiple of 4");
  static_assert(!PAGED || (VEC && sizeof(T) == 4), "pools of rows hold fp32 with head sizes that are multiples of 4");
  constexpr int KS = HP / 4;   // contraction steps of the first product = dims per lane
  constexpr int MTL = HP / 16;  // 16-dim output tiles
  constexpr int VG = MTL % 4 == 0 ? 4 : 2;  // output tiles whose dims of a lane are neighbours (see the V loads)
  static_assert(MTL % VG == 0, "head sizes built: multiples of 32");
  constexpr int ROW_F = HP + 2;
  constexpr int CPR = HP / 4;            // 16-byte chunks of a row
  constexpr int STAGE_F = 2 * 16 * HP;   // floats of one stage: the K tile, then the V tile
  __shared__ __attribute__((aligned(16))) float lds_f[COOP ? 2 * STAGE_F : 2 * 16 * ROW_F];
  float* const merge_buf = lds_f;
  const int H = EXACT ? HP : p.H, S = p.S;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, g = lane >> 4;
  const int split = p.l_split;
  const int head = blockIdx.y, b = blockIdx.z;  // PAGED: the KV head
  const int n_split = PAGED ? p.n_split : 1;
  const int ks = PAGED ? blockIdx.x % n_split : 0, wg_x = PAGED ? blockIdx.x / n_split : blockIdx.x;
  const int rowgroup = wg_x * (4 / split) + wave / split, ls = wave % split;
  const int row = rowgroup * 16 + n;
  // L: keys of this (batch, head); R: its query rows; [start, L) can be read, by this lane's row up to `limit`;
  // mcols: columns of a mask line.  Without PAGED these are the launch's constants.
  int L = p.L, R = S, start = 0, mcols = p.L;
  int pool_end = 0x7fffffff, n_new = 0;  // FUSED: tokens [pool_end, pool_end + n_new) are this step's new ones
  if constexpr (PAGED) {
    L = max(0, p.seq_lens[b] + p.len_bias + (p.len_bias_dev ? *p.len_bias_dev : 0));
    if constexpr (FUSED) n_new = min(p.n_new, L), pool_end = L - n_new;
    if (p.mask) L = min(L, p.mask_len);  // columns the mask does not have are masked
    start = p.kv_start ? min(max(p.kv_start[b], 0), L) : 0;
    R = S * p.n_rep, mcols = p.mask_len;
  }
  const bool valid = row < R;
  const int vrow = valid ? row : 0;
  const int row_s = PAGED ? vrow % S : vrow;                         // token of the row
  const int qhead = PAGED ? head * p.n_rep + vrow / S : head;        // its query head
  const int64_t pair = (int64_t)b * p.N + head;
  const T* qrow = PAGED ? static_cast<const T*>(p.q) + b * p.q_sb + qhead * p.q_sh + row_s * p.q_ss
                        : static_cast<const T*>(p.q) + (pair * S + vrow) * H;
  const T* kbase = PAGED ? static_cast<const T*>(p.k) + head * p.k_hs : static_cast<const T*>(p.k) + pair * (int64_t)L * H;
  const T* vbase = PAGED ? static_cast<const T*>(p.v) + head * p.v_hs : static_cast<const T*>(p.v) + pair * (int64_t)L * H;
  const MT* mrow = nullptr;
  if (p.mask) {
    if constexpr (PAGED) {
      mrow = static_cast<const MT*>(p.mask) + b * p.m_sb + row_s * p.m_ss;  // (strides of broadcast dims are 0)
    } else {
      const int64_t mb = p.mB == 1 ? 0 : b, mn = p.mN == 1 ? 0 : head, ms = p.mS == 1 ? 0 : vrow;
      mrow = static_cast<const MT*>(p.mask) + ((mb * p.mN + mn) * p.mS + ms) * (int64_t)L;
    }
  }
  // causal: query token s reads keys <= L - S + s
  const int limit = (PAGED && p.causal) ? min(L, L - S + row_s + 1) : L;
  int limit_lo = limit;  // the smallest limit of the wave's rows (wave-uniform)
  if constexpr (PAGED) {
#pragma unroll
    for (int o = 1; o < 64; o *= 2) limit_lo = min(limit_lo, __shfl_xor(limit_lo, o, 64));
    limit_lo = __builtin_amdgcn_readfirstlane(limit_lo);
  }
  // This lane's dims of a row for the first product: d0 .. d0 + KS - 1.
  const int d0 = g * KS;
  // Launches whose K / V are read by one row group (the dense kernel's key-splitting variants, the pool's small-row
  // launches): non-temporal loads, and the first product's dims dealt out so that the four lanes of a row read 64
  // contiguous bytes per load -- a 128-byte line is then consumed by two instructions instead of eight (fetched
  // non-temporally with a lane's dims as one run, the fp32 pool's decode launch took 638 us instead of 370; with both
  // changes 357, the dense op's fp32 decode 1.29 ms instead of 1.39).  Any assignment of dims to steps gives the same
  // sum as long as Q and K share it.
  constexpr bool ONCE = AHEAD || (PAGED && !COOP);
  auto load_run = [&](const T* r, float (&x)[KS], auto once_c) {
    constexpr bool kOnce = decltype(once_c)::value;
#pragma unroll
    for (int s4 = 0; s4 < KS; s4 += 4) {
      const int d = ONCE ? 4 * s4 + 4 * g : d0 + s4;
      if (VEC) {  // H is a multiple of 4: the four dims exist together or not at all
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
        if (d + 4 <= H) t = load4_kv<kOnce>(r + d);
        x[s4] = t[0], x[s4 + 1] = t[1], x[s4 + 2] = t[2], x[s4 + 3] = t[3];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) x[s4 + e] = (d + e < H) ? load_f32<T>(r + d + e) : 0.f;
      }
    }
  };
  float qf[KS];
  load_run(qrow, qf, std::false_type{});
  if (!valid) {
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = 0.f;
  }
  f32x4 o[MTL];
#pragma unroll
  for (int j = 0; j < MTL; ++j) o[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = kNegInf, l_run = 0.f;

  // This wave's share of the 16-token tiles that some row of its group reads.
  int key_end = L, tile_first = 0;  // wave-uniform
  if constexpr (PAGED) {
    if (p.causal) {  // the group's last token: its rows lie in one query head, or some row is a head's last token
      const int s0 = (rowgroup * 16) % S;
      key_end = max(0, min(L, L - S + (s0 + 15 < S ? s0 + 15 : S - 1) + 1));
    }
    tile_first = start / 16;
  }
  const int tiles = max(tile_first, (key_end + 15) / 16);
  const int per_wg = (tiles - tile_first + n_split - 1) / n_split;  // (n_split 1: the whole range)
  const int wg_lo = min(tiles, tile_first + ks * per_wg), wg_hi = min(tiles, wg_lo + per_wg);
  const int per = (wg_hi - wg_lo + split - 1) / split;
  const int tile_lo = min(wg_hi, wg_lo + ls * per), tile_hi = min(wg_hi, tile_lo + per);
  const bool has_rows = rowgroup * 16 < R;  // wave-uniform
  if constexpr (FUSED) {
    // The first workgroup of this (sequence, KV head) stores the step's new rows into the pool; no workgroup of the
    // launch reads those pool rows (they all take them from the caller's buffers).
    if (blockIdx.x == 0 && n_new > 0) {
      const int chunks = H / 4;  // (H is a multiple of 4)
      for (int item = threadIdx.x; item < n_new * chunks; item += 256) {
        const int idx = item / chunks, c = item % chunks, pos = pool_end + idx, jb = pos / PACE_KV_BLOCK_TOKENS;
        if (jb >= p.table_stride) continue;
        const int64_t blk = p.table[(int64_t)b * p.table_stride + jb];
        if (blk < 0 || blk >= p.num_blocks) continue;  // never write outside the pool
        const int64_t src = b * p.n_sb + head * p.n_sh + (int64_t)idx * p.n_st + 4 * c;
        const int64_t dst = (int64_t)(pos % PACE_KV_BLOCK_TOKENS) * H + 4 * c;
        float* kdst = const_cast<float*>(static_cast<const float*>(p.k)) + blk * p.k_bs + head * p.k_hs + dst;
        float* vdst = const_cast<float*>(static_cast<const float*>(p.v)) + blk * p.v_bs + head * p.v_hs + dst;
        *reinterpret_cast<u32x4*>(kdst) = *reinterpret_cast<const u32x4*>(p.k_new + src);
        *reinterpret_cast<u32x4*>(vdst) = *reinterpret_cast<const u32x4*>(p.v_new + src);
      }
    }
  }
  float kf[KS], vf[MTL][4], mv[4];
  auto fetch_mask = [&](int tile, float (&mx4)[4]) {
    // the lane's four mask values: one load where the four columns exist (mask lines start wherever L puts them;
    // the hardware takes unaligned multi-dword loads), element by element at the end of a line
    const int t = tile * 16 + 4 * g;
    if (!mrow) {
#pragma unroll
      for (int i = 0; i < 4; ++i) mx4[i] = 0.f;
    } else if (t + 4 <= mcols) {
      if constexpr (sizeof(MT) == 4) {
        u32x4 raw;
        __builtin_memcpy(&raw, mrow + t, 16);
#pragma unroll
        for (int i = 0; i < 4; ++i) mx4[i] = __uint_as_float(raw[i]);
      } else {
        u32x2 raw;
        __builtin_memcpy(&raw, mrow + t, 8);
        mx4[0] = __uint_as_float(raw[0] << 16), mx4[1] = __uint_as_float(raw[0] & 0xffff0000u);
        mx4[2] = __uint_as_float(raw[1] << 16), mx4[3] = __uint_as_float(raw[1] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) mx4[i] = (t + i < mcols) ? load_f32<MT>(mrow + t + i) : 0.f;
    }
  };
  auto fetch = [&](int tile, float (&kx)[KS], float (&vx)[MTL][4], float (&mx4)[4]) {
    const int t0 = tile * 16;
    const T* kblock = kbase;
    const T* vblock = vbase;
    if constexpr (PAGED) {  // one tile is one block: a scalar look-up; ids are clamped, nothing outside the pool is read
      const int64_t blk = min(max(p.table[(int64_t)b * p.table_stride + min(tile, p.table_stride - 1)], 0), p.num_blocks - 1);
      kblock = kbase + blk * p.k_bs - (int64_t)t0 * H, vblock = vbase + blk * p.v_bs - (int64_t)t0 * H;
    }
    // FUSED, a tile that holds new tokens: their rows are read from the caller's buffers (index held inside them:
    // rows past the end are masked below), the others from the pool as ever.  Wave-uniform.
    const bool with_new = FUSED && n_new > 0 && t0 + 16 > pool_end;
    const T* new_k = nullptr;
    const T* new_v = nullptr;
    if constexpr (FUSED) {
      new_k = reinterpret_cast<const T*>(p.k_new) + b * p.n_sb + head * p.n_sh;
      new_v = reinterpret_cast<const T*>(p.v_new) + b * p.n_sb + head * p.n_sh;
    }
    auto row_of = [&](const T* pool_rows, const T* new_rows, int pos) -> const T* {
      if (with_new && pos >= pool_end) return new_rows + (int64_t)min(pos - pool_end, n_new - 1) * p.n_st;
      return pool_rows + (int64_t)pos * H;
    };
    // rows past the end are masked below (PAGED: the block's 16 rows exist whatever the length is)
    if (FUSED) load_run(row_of(kblock, new_k, t0 + n), kx, std::integral_constant<bool, ONCE>{});
    else load_run(kblock + (int64_t)(PAGED ? t0 + n : min(L - 1, t0 + n)) * H, kx, std::integral_constant<bool, ONCE>{});
    // V: output tile j of lane n stands for dim v_dim(j, n) = 16 VG (j / VG) + VG n + j % VG, so that the VG values a
    // lane needs of one token for VG neighbouring tiles are one contiguous run: a quarter of the load instructions
    // that one value per load takes, and every load of a wave covers whole 256-byte stretches of four rows.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const T* vr = FUSED ? row_of(vblock, new_v, t0 + 4 * g + i) : vblock + (int64_t)(PAGED ? t0 + 4 * g + i : min(L - 1, t0 + 4 * g + i)) * H;
#pragma unroll
      for (int jj = 0; jj < MTL; jj += VG) {
        const int d = 16 * jj + VG * n;
        if (VEC && VG == 4) {
          f32x4 t = {0.f, 0.f, 0.f, 0.f};
          if (d + 4 <= H) t = load4_kv<ONCE>(vr + d);
#pragma unroll
          for (int e = 0; e < 4; ++e) vx[jj + (e % VG)][i] = t[e];
        } else if (VEC && VG == 2) {
          f32x2 t = {0.f, 0.f};
          if (d + 2 <= H) t = load2_f32(vr + d);
          vx[jj][i] = t[0], vx[jj + (1 % VG)][i] = t[1];
        } else {
#pragma unroll
          for (int e = 0; e < VG; ++e) vx[jj + e][i] = (d + e < H) ? load_f32<T>(vr + d + e) : 0.f;
        }
      }
    }
    fetch_mask(tile, mx4);
  };
  // One tile's arithmetic on the operands at hand.
  auto tile_math = [&](int t0, const float (&kf)[KS], const float (&vf)[MTL][4], const float (&mv)[4]) {
    f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[s], qf[s], sc, 0, 0, 0);
    // The softmax reference of a row moves lazily: only when a score lies more than kLazy above it (weights stay below
    // e^kLazy = 245, far inside fp32), which in a row of a few hundred keys happens a handful of times instead of in
    // most tiles -- and the accumulators are rescaled only then.  Whether any row of the wave moves is decided by
    // comparing the lane's own scores with the threshold; the row maximum is formed only when one does.
    constexpr float kLazy = 5.5f;
    const float top = m_run + kLazy;  // (-inf while the row has seen nothing)
    float val[4];
    bool above = false;
    if (t0 + 16 <= limit_lo && (!PAGED || t0 >= start)) {  // every row of the wave reads the whole tile: no bound to check
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        val[i] = fmaf(sc[i], p.scale, mv[i]);
        above = above || val[i] > top;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tk = t0 + 4 * g + i;
        val[i] = (tk < limit && (!PAGED || tk >= start)) ? fmaf(sc[i], p.scale, mv[i]) : kNegInf;
        above = above || val[i] > top;
      }
    }
    if (__any(above)) {
      const float mx = row_max4(fmaxf(fmaxf(val[0], val[1]), fmaxf(val[2], val[3])));
      const float m_new = mx > top ? mx : m_run;  // (the same in the four lanes of a row)
      const float alpha = exp_of(m_run - ((m_new == kNegInf) ? 0.f : m_new));  // 1 for a row that stays, 0 for a first score
      l_run *= alpha;
#pragma unroll
      for (int j = 0; j < MTL; ++j) o[j] *= alpha;
      m_run = m_new;
    }
    const float m_use = (m_run == kNegInf) ? 0.f : m_run;
    float pr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pr[i] = exp_of(val[i] - m_use);
      l_run += pr[i];
    }
    // token quarter by token quarter over all output tiles: neighbouring matrix instructions write different
    // accumulators (per tile the order of the four is unchanged)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < MTL; ++j) o[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[j][i], pr[i], o[j], 0, 0, 0);
  };
  if constexpr (COOP) {
    // Every wave of the workgroup passes every barrier: the walk covers the tiles any of its row groups reads, a wave
    // computes on those of its own range.
    int wg_end = L;
    if constexpr (PAGED) {
      if (p.causal) {  // the last token any row of the workgroup's four row groups reads (as key_end above, per group)
        wg_end = 0;
        for (int gi = wg_x * 4; gi < wg_x * 4 + 4 && gi * 16 < R; ++gi) {
          const int s0 = (gi * 16) % S;
          wg_end = max(wg_end, min(L, L - S + (s0 + 15 < S ? s0 + 15 : S - 1) + 1));
        }
      }
    }
    const int walk_lo = tile_first, walk_hi = max(tile_first, (wg_end + 15) / 16);
    constexpr int TILE_CHUNKS = 16 * CPR, PER_T = (TILE_CHUNKS + 255) / 256;
    auto rot = [](int x) { return (CPR & (CPR - 1)) == 0 ? (x & (CPR - 1)) : (x >= CPR ? x - CPR : x); };  // x < CPR + 16
    // Offsets that do not change from tile to tile, formed once (the stage and the K / V half are constants of the
    // instruction): where this thread's chunks of a tile come from and go to, where this lane's operands lie.
    int src_row[PER_T], src_col[PER_T], dst_at[PER_T], k_at[KS / 4], v_at[4][MTL / VG];
    uint32_t src_at[PER_T];
#pragma unroll
    for (int i = 0; i < PER_T; ++i) {
      const int id = min((int)threadIdx.x + 256 * i, TILE_CHUNKS - 1), r = id / CPR, c = id % CPR;
      src_row[i] = r, src_col[i] = 4 * c, dst_at[i] = 4 * (r * CPR + rot(c + r));
      src_at[i] = (uint32_t)(r * H + 4 * c) * (uint32_t)sizeof(T);
    }
#pragma unroll
    for (int k = 0; k < KS / 4; ++k) k_at[k] = 4 * (n * CPR + rot(d0 / 4 + k + n));
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int jv = 0; jv < MTL / VG; ++jv) {
        const int r = 4 * g + i, d = 16 * VG * jv + VG * n;
        v_at[i][jv] = 4 * (r * CPR + rot(d / 4 + r)) + d % 4;
      }
    u32x4 sk[PER_T], sv[PER_T];
    auto stage_load = [&](int tile) {
      const int t0 = tile * 16;
      const T* kblock = kbase + (int64_t)t0 * H;
      const T* vblock = vbase + (int64_t)t0 * H;
      if constexpr (PAGED) {
        const int64_t blk = min(max(p.table[(int64_t)b * p.table_stride + min(tile, p.table_stride - 1)], 0), p.num_blocks - 1);
        kblock = kbase + blk * p.k_bs, vblock = vbase + blk * p.v_bs;
      }
      // Rows past the end of a dense tensor are not read (zeros take their place; the arithmetic masks them.  PAGED:
      // a block's 16 rows exist whatever the length is).  The offsets were formed before the walk -- unsigned 32-bit
      // byte offsets from a pointer the whole wave shares, which is the load's own addressing: no vector arithmetic
      // per tile.
#pragma unroll
      for (int i = 0; i < PER_T; ++i) {
        if (TILE_CHUNKS % 256 == 0 || (int)threadIdx.x + 256 * i < TILE_CHUNKS) {
          sk[i] = sv[i] = u32x4{0u, 0u, 0u, 0u};
          if ((EXACT || src_col[i] < H) && (PAGED || src_row[i] < L - t0)) {  // (dims the rows do not have read as zero)
            sk[i] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(kblock) + src_at[i]);
            sv[i] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(vblock) + src_at[i]);
          }
        }
      }
    };
    auto stage_store = [&](auto stage_c) {
      constexpr int stage = decltype(stage_c)::value;
#pragma unroll
      for (int i = 0; i < PER_T; ++i) {
        if (TILE_CHUNKS % 256 == 0 || (int)threadIdx.x + 256 * i < TILE_CHUNKS) {
          *reinterpret_cast<u32x4*>(lds_f + stage * STAGE_F + dst_at[i]) = sk[i];
          *reinterpret_cast<u32x4*>(lds_f + stage * STAGE_F + 16 * HP + dst_at[i]) = sv[i];
        }
      }
    };
    auto operands = [&](auto stage_c, float (&kx)[KS], float (&vx)[MTL][4]) {
      constexpr int stage = decltype(stage_c)::value;
#pragma unroll
      for (int k = 0; k < KS / 4; ++k) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(lds_f + stage * STAGE_F + k_at[k]);
        kx[4 * k] = t[0], kx[4 * k + 1] = t[1], kx[4 * k + 2] = t[2], kx[4 * k + 3] = t[3];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int jv = 0; jv < MTL / VG; ++jv) {
          const float* at = lds_f + stage * STAGE_F + 16 * HP + v_at[i][jv];
          if (VG == 4) {
            const f32x4 t = *reinterpret_cast<const f32x4*>(at);
#pragma unroll
            for (int e = 0; e < 4; ++e) vx[VG * jv + (e % VG)][i] = t[e];
          } else {
            const f32x2 t = *reinterpret_cast<const f32x2*>(at);
            vx[VG * jv][i] = t[0], vx[VG * jv + (1 % VG)][i] = t[1];
          }
        }
      }
    };
    auto walk = [&](int tile, auto stage_c) {
      constexpr int stage = decltype(stage_c)::value;
      const bool more = tile + 1 < walk_hi;
      if (more) stage_load(tile + 1);  // in flight over this tile's arithmetic
      if (has_rows && tile >= tile_lo && tile < tile_hi) {
        fetch_mask(tile, mv);
        operands(stage_c, kf, vf);
        tile_math(tile * 16, kf, vf, mv);
      }
      // (the other stage was last read before the barrier that ended the tile before this one)
      if (more) stage_store(std::integral_constant<int, stage ^ 1>{});
      __syncthreads();
    };
    if (walk_lo < walk_hi) {
      stage_load(walk_lo);
      stage_store(std::integral_constant<int, 0>{});
    }
    __syncthreads();
    for (int tile = walk_lo; tile < walk_hi; tile += 2) {
      walk(tile, std::integral_constant<int, 0>{});
      if (tile + 1 < walk_hi) walk(tile + 1, std::integral_constant<int, 1>{});
    }
  } else {
    if (AHEAD && has_rows && tile_lo < tile_hi) fetch(tile_lo, kf, vf, mv);
    for (int tile = tile_lo; has_rows && tile < tile_hi; ++tile) {
      const int t0 = tile * 16;
      float kn[AHEAD ? KS : 1], vn[AHEAD ? MTL : 1][4], mn[4];
      const bool more = AHEAD && tile + 1 < tile_hi;
      if constexpr (AHEAD) {
        if (more) fetch(tile + 1, kn, vn, mn);
      } else {
        fetch(tile, kf, vf, mv);
      }
      tile_math(t0, kf, vf, mv);
    if constexpr (AHEAD) {
        if (more) {
#pragma unroll
          for (int s = 0; s < KS; ++s) kf[s] = kn[s];
#pragma unroll
          for (int j = 0; j < MTL; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) vf[j][i] = vn[j][i];
#pragma unroll
          for (int i = 0; i < 4; ++i) mv[i] = mn[i];
        }
      }
    }
  }
  // row sum over the four lanes of a row
  l_run += xor_lanes(l_run, 16);
  l_run += xor_lanes(l_run, 32);

  // Merge the key shares of a row group (fixed order: deterministic).  Every wave passes the same barriers.
  for (int stride = 1; stride < split; stride *= 2) {
    const bool sender = (ls & (2 * stride - 1)) == stride;
    const bool receiver = (ls & (2 * stride - 1)) == 0 && ls + stride < split;
    float* slot = merge_buf + (wave / (2 * stride)) * 16 * ROW_F + n * ROW_F;
    if (sender) {
#pragma unroll
      for (int j = 0; j < MTL; ++j)
#pragma unroll
        for (int c = 0; c < 4; ++c) slot[16 * j + 4 * g + c] = o[j][c];
      if (g == 0) slot[HP] = m_run, slot[HP + 1] = l_run;
    }
    __syncthreads();
    if (receiver) {
      const float m_b = slot[HP], l_b = slot[HP + 1];
      const float m_new = fmaxf(m_run, m_b);
      const float m_use = (m_new == kNegInf) ? 0.f : m_new;
      const float wa = exp_of(m_run - m_use), wb = exp_of(m_b - m_use);
#pragma unroll
      for (int j = 0; j < MTL; ++j)
#pragma unroll
        for (int c = 0; c < 4; ++c) o[j][c] = o[j][c] * wa + slot[16 * j + 4 * g + c] * wb;
      l_run = l_run * wa + l_b * wb;
      m_run = m_new;
    }
    __syncthreads();
  }
  if (ls != 0 || !valid) return;
  if constexpr (PAGED) {
    if (n_split > 1) {  // this workgroup's share of the row, left for the merge
      const int64_t grow = ((int64_t)b * p.N * p.n_rep + qhead) * S + row_s;
      float* slot = p.part + (grow * n_split + ks) * (H + 4);
#pragma unroll
      for (int jj = 0; jj < MTL; jj += VG) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int d = 16 * jj + VG * (4 * g + c);
          if (VG == 4) {
            if (d + 4 <= H) store4_out(slot + d, f32x4{o[jj][c], o[jj + (1 % VG)][c], o[jj + (2 % VG)][c], o[jj + (3 % VG)][c]});
          } else {
            if (d + 2 <= H) store2_out(slot + d, f32x2{o[jj][c], o[jj + (1 % VG)][c]});
          }
        }
      }
      if (g == 0) slot[H] = m_run, slot[H + 1] = l_run;
      return;
    }
  }
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
  T* orow = PAGED ? static_cast<T*>(p.out) + b * p.o_sb + qhead * p.o_sh + row_s * p.o_ss : static_cast<T*>(p.out) + (pair * S + row) * H;
  // o[j][c] of lane (row, g) is the output at dim v_dim(j, 4 g + c)
#pragma unroll
  for (int jj = 0; jj < MTL; jj += VG) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int d = 16 * jj + VG * (4 * g + c);
      if (VEC && VG == 4) {
        if (d + 4 <= H) store4_out(orow + d, f32x4{o[jj][c], o[jj + (1 % VG)][c], o[jj + (2 % VG)][c], o[jj + (3 % VG)][c]} * inv);
      } else if (VEC && VG == 2) {
        if (d + 2 <= H) store2_out(orow + d, f32x2{o[jj][c], o[jj + (1 % VG)][c]} * inv);
      } else {
#pragma unroll
        for (int e = 0; e < VG; ++e)
          if (d + e < H) store_out(orow + d + e, o[jj + e][c] * inv);
      }
    }
  }
}

template <typename T, typename MT, int HP, bool VEC, bool AHEAD, bool EXACT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, HP > 128 ? 1 : 2))) void attn_dense_kernel(
    const DenseParams p) {
  attn_dense_body<T, MT, HP, VEC, AHEAD, EXACT, false>(p);
}

// fp32 rows of a multiple of four dims, row groups with keys of their own (more than 32 query rows): the workgroup shares
// its tiles through LDS (COOP above).  PAGED: over a pool of fp32 rows.
template <typename MT, int HP, bool PAGED, bool EXACT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, HP > 128 ? 1 : 2))) void attn_f32_coop_kernel(
    const DenseParams p) {
  attn_dense_body<float, MT, HP, true, false, EXACT, PAGED, true>(p);
}

// The same walk over a pool of fp32 rows (pace_kv_pool_t with elem_bytes 4).  No fetch a tile ahead: here the second
// wave per SIMD hides more than the second set of registers did (decode, batch 64 x 8 KV heads x 4096 tokens of 128
// dims: 370 us against 460).
template <typename MT, int HP, bool EXACT, bool FUSED = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, HP > 128 ? 1 : 2))) void attn_paged_f32_kernel(
    const DenseParams p) {
  attn_dense_body<float, MT, HP, true, false, EXACT, true, false, FUSED>(p);
}

// Ends a launch whose sequences were cut over several workgroups: out = sum_i e^(m_i - M) o_i / sum_i e^(m_i - M) l_i
// per query row; lane t owns dims 4t .. 4t + 3.
__global__ __launch_bounds__(64) void attn_paged_f32_merge_kernel(const DenseParams p) {
  const int64_t grow = blockIdx.x;  // (b, query head, token)
  const int S = p.S, H = p.H, heads = p.N * p.n_rep;
  const int s = (int)(grow % S), hq = (int)((grow / S) % heads), b = (int)(grow / ((int64_t)S * heads));
  const float* slot = p.part + grow * p.n_split * (H + 4);
  float M = kNegInf;
  for (int i = 0; i < p.n_split; ++i) M = fmaxf(M, slot[i * (H + 4) + H]);
  const float m_use = (M == kNegInf) ? 0.f : M;
  const int d = 4 * threadIdx.x;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float L = 0.f;
  for (int i = 0; i < p.n_split; ++i) {
    const float* ps = slot + i * (H + 4);
    const float w = exp_of(ps[H] - m_use);
    L += w * ps[H + 1];
    if (d < H) acc += load4_f32(ps + d) * w;
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  if (d < H) store4_out(static_cast<float*>(p.out) + b * p.o_sb + hq * p.o_sh + s * p.o_ss + d, acc * inv);
}

int launch_paged_f32(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* a, const char* who, hipStream_t stream) {
  PACE_REQUIRE(a->batch <= 65535 && pool->num_kv_heads <= 65535, "%s: batch / heads exceed grid limits", who);
  DenseParams p = {};
  p.q = a->q, p.k = pool->k, p.v = pool->v, p.out = a->out, p.mask = a->mask;
  p.B = a->batch, p.N = pool->num_kv_heads, p.S = a->q_len, p.L = 0, p.H = pool->head_dim;
  p.scale = a->scale;
  p.table = a->block_table, p.seq_lens = a->seq_lens, p.len_bias_dev = a->seq_len_bias_ptr, p.kv_start = a->kv_start;
  p.k_bs = pool->k_block_stride, p.k_hs = pool->k_head_stride, p.v_bs = pool->v_block_stride, p.v_hs = pool->v_head_stride;
  p.q_sb = a->q_stride_b, p.q_sh = a->q_stride_h, p.q_ss = a->q_stride_s;
  p.o_sb = a->o_stride_b, p.o_sh = a->o_stride_h, p.o_ss = a->o_stride_s;
  p.m_sb = a->mask_stride_b, p.m_ss = a->mask_stride_s;
  p.table_stride = a->table_stride, p.len_bias = a->seq_len_bias, p.num_blocks = pool->num_blocks;
  p.n_rep = a->num_q_heads / pool->num_kv_heads, p.causal = a->causal ? 1 : 0, p.mask_len = a->mask_len;
  const int64_t rows = (int64_t)a->q_len * p.n_rep;
  PACE_REQUIRE(rows < (1 << 27), "%s: too many query rows per KV head", who);
  p.l_split = rows <= 16 ? 4 : (rows <= 32 ? 2 : 1);
  const int rowgroups = (int)((rows + 15) / 16), per_wg = 4 / p.l_split;
  const int H = pool->head_dim;
  // A batch that leaves compute units idle: cut the keys of every row group over several workgroups, as many as fill the
  // GPU twice, as leave a wave four tiles of the longest sequence, and as the caller's workspace has room for.
  const int64_t wgs = (int64_t)((rowgroups + per_wg - 1) / per_wg) * pool->num_kv_heads * a->batch;
  const int64_t rows_total = (int64_t)a->batch * a->num_q_heads * a->q_len;
  p.n_split = 1, p.part = nullptr;
  if (a->workspace && aligned16(a->workspace) && wgs < 2 * compute_units()) {
    const int64_t tiles = (a->max_seq_len + 15) / 16;
    int64_t n = (2 * compute_units() + wgs - 1) / wgs;
    n = n < tiles / (4 * p.l_split) ? n : tiles / (4 * p.l_split);
    const int64_t room = (int64_t)(a->workspace_bytes / ((size_t)rows_total * (H + 4) * sizeof(float)));
    n = n < room ? n : room;
    n = n < 64 ? n : 64;
    if (n > 1) p.n_split = (int)n, p.part = static_cast<float*>(a->workspace);
  }
  PACE_REQUIRE(rows_total < ((int64_t)1 << 31), "%s: too many query rows", who);
  const dim3 grid((unsigned)((rowgroups + per_wg - 1) / per_wg * p.n_split), pool->num_kv_heads, a->batch);
  const bool mf32 = a->mask_dtype == PACE_DTYPE_F32;
  const bool coop = p.l_split == 1 && p.n_split == 1;
  const bool fused = a->k_new != nullptr;
  if (fused) {
    PACE_REQUIRE(rows <= 32, "%s: over an fp32 pool the append rides in launches of up to 32 query rows per KV head (got %lld)", who,
                 (long long)rows);
    p.k_new = static_cast<const float*>(a->k_new), p.v_new = static_cast<const float*>(a->v_new);
    p.n_sb = a->new_stride_b, p.n_sh = a->new_stride_h, p.n_st = a->new_stride_t, p.n_new = a->n_new;
  }
#define PACE_PAGED_F32_GO(MT_, HP_) \
  do { \
    if (H == HP_ && coop) hipLaunchKernelGGL((attn_f32_coop_kernel<MT_, HP_, true, true>), grid, dim3(256), 0, stream, p); \
    else if (coop) hipLaunchKernelGGL((attn_f32_coop_kernel<MT_, HP_, true, false>), grid, dim3(256), 0, stream, p); \
    else if (H == HP_ && fused) hipLaunchKernelGGL((attn_paged_f32_kernel<MT_, HP_, true, true>), grid, dim3(256), 0, stream, p); \
    else if (fused) hipLaunchKernelGGL((attn_paged_f32_kernel<MT_, HP_, false, true>), grid, dim3(256), 0, stream, p); \
    else if (H == HP_) hipLaunchKernelGGL((attn_paged_f32_kernel<MT_, HP_, true>), grid, dim3(256), 0, stream, p); \
    else hipLaunchKernelGGL((attn_paged_f32_kernel<MT_, HP_, false>), grid, dim3(256), 0, stream, p); \
  } while (0)
#define PACE_PAGED_F32_HP(MT_) \
  do { \
    if (H <= 32) PACE_PAGED_F32_GO(MT_, 32); \
    else if (H <= 64) PACE_PAGED_F32_GO(MT_, 64); \
    else if (H <= 96) PACE_PAGED_F32_GO(MT_, 96); \
    else if (H <= 128) PACE_PAGED_F32_GO(MT_, 128); \
    else PACE_PAGED_F32_GO(MT_, 256); \
  } while (0)
  if (mf32) PACE_PAGED_F32_HP(float); else PACE_PAGED_F32_HP(uint16_t);
#undef PACE_PAGED_F32_HP
#undef PACE_PAGED_F32_GO
  PACE_HIP_CHECK(hipGetLastError());
  if (p.n_split > 1) {
    hipLaunchKernelGGL(attn_paged_f32_merge_kernel, dim3((unsigned)rows_total), dim3(64), 0, stream, p);
    PACE_HIP_CHECK(hipGetLastError());
  }
  return PACE_KV_OK;
}

}  // namespace pace_kv

using namespace pace_kv;

extern "C" size_t pace_attn_dense_workspace_bytes(int32_t qkv_dtype, int32_t S, int32_t H, int32_t has_mask, int32_t mB, int32_t mN,
                                                  int32_t mS) {
  if (qkv_dtype != PACE_DTYPE_BF16 || S <= 0 || H <= 0 || mB <= 0 || mN <= 0 || mS <= 0) return 0;
  return dense_mfma_workspace_bytes(S, H, mB, mN, mS, has_mask != 0);
}

extern "C" int pace_attn_dense(const void* q, const void* k, const void* v, void* out, int32_t qkv_dtype, int32_t B,
                               int32_t N, int32_t S, int32_t L, int32_t H, const void* mask, int32_t mask_dtype,
                               int32_t mB, int32_t mN, int32_t mS, void* stream) {
  return pace_attn_dense_ws(q, k, v, out, qkv_dtype, B, N, S, L, H, mask, mask_dtype, mB, mN, mS, nullptr, 0, stream);
}

extern "C" int pace_attn_dense_ws(const void* q, const void* k, const void* v, void* out, int32_t qkv_dtype, int32_t B,
                                  int32_t N, int32_t S, int32_t L, int32_t H, const void* mask, int32_t mask_dtype,
                                  int32_t mB, int32_t mN, int32_t mS, void* workspace, size_t workspace_bytes, void* stream) {
  PACE_REQUIRE(qkv_dtype == PACE_DTYPE_F32 || qkv_dtype == PACE_DTYPE_BF16, "pace_attn_dense*: bad qkv dtype %d", qkv_dtype);
  PACE_REQUIRE(B >= 0 && N >= 0 && S >= 0 && L >= 0 && H >= 1, "pace_attn_dense*: negative extent");
  if (B == 0 || N == 0 || S == 0) return PACE_KV_OK;
  PACE_REQUIRE(L >= 1, "pace_attn_dense*: empty key/value length");
  PACE_REQUIRE(H <= 256, "pace_attn_dense*: head_dim %d unsupported (max 256)", H);
  PACE_REQUIRE(q && k && v && out, "pace_attn_dense*: NULL tensor pointer");
  if (mask) {
    PACE_REQUIRE(mask_dtype == PACE_DTYPE_F32 || mask_dtype == PACE_DTYPE_BF16, "pace_attn_dense*: bad mask dtype %d",
                 mask_dtype);
    PACE_REQUIRE((mB == 1 || mB == B) && (mN == 1 || mN == N) && (mS == 1 || mS == S),
                 "pace_attn_dense*: mask dims [%d][%d][%d] not broadcastable to [%d][%d][%d]", mB, mN, mS, B, N, S);
  }
  PACE_REQUIRE(B <= 65535 && N <= 65535, "pace_attn_dense*: batch / heads exceed grid limits");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // bf16 with head_dim 64 / 96 / 128 / 256 runs on the bf16 matrix-core kernels; everything else (fp32,
  // other head sizes) takes the general kernel below.
  if (qkv_dtype == PACE_DTYPE_BF16 &&
      launch_dense_mfma(q, k, v, out, B, N, S, L, H, mask, mask_dtype == PACE_DTYPE_F32, mB, mN, mS,
                        1.0f / sqrtf((float)H), workspace, workspace_bytes, s)) {
    PACE_HIP_CHECK(hipGetLastError());
    return PACE_KV_OK;
  }
  DenseParams p = {};
  p.q = q, p.k = k, p.v = v, p.out = out, p.mask = mask;
  p.B = B, p.N = N, p.S = S, p.L = L, p.H = H;
  p.mB = mB, p.mN = mN, p.mS = mS;
  p.scale = 1.0f / sqrtf((float)H);
  // Few query rows: the four waves of a workgroup split the keys of one row group (or of two).
  p.l_split = S <= 16 ? 4 : (S <= 32 ? 2 : 1);
  const int rowgroups = (S + 15) / 16, per_wg = 4 / p.l_split;
  dim3 grid((rowgroups + per_wg - 1) / per_wg, N, B);
  const bool f32 = qkv_dtype == PACE_DTYPE_F32;
  const bool mf32 = mask_dtype == PACE_DTYPE_F32;
  // vector accesses need rows that start on a 16-byte (fp32) / 8-byte (bf16) boundary
  const size_t row_align = f32 ? 16 : 8;
  const bool ahead = p.l_split > 1;  // few query rows: bound by memory
  const bool vec = H % 4 == 0 && ((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % row_align == 0;
#define PACE_DENSE_GO(T_, MT_, HP_) \
  do { \
    constexpr bool kAheadBuilt = HP_ <= 128; /* at 256 the second set of registers does not fit */ \
    if constexpr (sizeof(T_) == 4) { \
      if (vec && p.l_split == 1) { \
        if (H == HP_) hipLaunchKernelGGL((attn_f32_coop_kernel<MT_, HP_, false, true>), grid, dim3(256), 0, s, p); \
        else hipLaunchKernelGGL((attn_f32_coop_kernel<MT_, HP_, false, false>), grid, dim3(256), 0, s, p); \
        break; \
      } \
    } \
    if (ahead && kAheadBuilt) { \
      if (vec && H == HP_) hipLaunchKernelGGL((attn_dense_kernel<T_, MT_, HP_, true, kAheadBuilt, true>), grid, dim3(256), 0, s, p); \
      else if (vec) hipLaunchKernelGGL((attn_dense_kernel<T_, MT_, HP_, true, kAheadBuilt, false>), grid, dim3(256), 0, s, p); \
      else hipLaunchKernelGGL((attn_dense_kernel<T_, MT_, HP_, false, kAheadBuilt, false>), grid, dim3(256), 0, s, p); \
    } else if (vec && H == HP_) hipLaunchKernelGGL((attn_dense_kernel<T_, MT_, HP_, true, false, true>), grid, dim3(256), 0, s, p); \
    else if (vec) hipLaunchKernelGGL((attn_dense_kernel<T_, MT_, HP_, true, false, false>), grid, dim3(256), 0, s, p); \
    else hipLaunchKernelGGL((attn_dense_kernel<T_, MT_, HP_, false, false, false>), grid, dim3(256), 0, s, p); \
  } while (0)
#define PACE_DENSE_HP(T_, MT_) \
  do { \
    if (H <= 32) PACE_DENSE_GO(T_, MT_, 32); \
    else if (H <= 64) PACE_DENSE_GO(T_, MT_, 64); \
    else if (H <= 96) PACE_DENSE_GO(T_, MT_, 96); \
    else if (H <= 128) PACE_DENSE_GO(T_, MT_, 128); \
    else PACE_DENSE_GO(T_, MT_, 256); \
  } while (0)
  if (f32 && mf32) PACE_DENSE_HP(float, float);
  else if (f32) PACE_DENSE_HP(float, uint16_t);
  else if (mf32) PACE_DENSE_HP(uint16_t, float);
  else PACE_DENSE_HP(uint16_t, uint16_t);
#undef PACE_DENSE_HP
#undef PACE_DENSE_GO
  PACE_HIP_CHECK(hipGetLastError());
  return PACE_KV_OK;
}

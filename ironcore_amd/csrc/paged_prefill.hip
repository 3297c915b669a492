// Chunked prefill against the block KV cache: the MFMA path.
//
// Each sequence brings a chunk of C new query tokens whose K/V rows are
// already in the pool; query row r sees keys j <= (L - C) + r (L = context
// length).  This is the reference's dense attention
// (ironcore/layers/attention.py:68-142) with sq = C, sk = L and the causal
// mask of ironcore/language_model.py:109-114 shifted by the cached prefix; with
// causal = 0 every row sees all L keys (the attention_mask=None case).  Query
// head h reads KV head h / G (attention.py:95-102).
//
// A dense contraction, so it runs on the matrix cores
// (v_mfma_f32_32x32x16 bf16/f16, fp32 accumulate), flash-attention style:
//
//  * One workgroup = a query tile of 256 rows of one query head; 8 waves, each
//    owning a 32-row query block for the whole K/V sweep (one workgroup per
//    CU, two waves per SIMD).  The wave's Q rows stay in registers as MFMA B
//    operands.  Workgroup ids are laid out so that all tiles and heads that
//    read the same K/V rows run on one XCD and share its L2.
//  * K/V are walked in tiles of 64 tokens (4 pool blocks).  Four waves stage
//    K and four stage V, each one 16-row group of every tile, fetched through
//    the block table (one table entry per wave and tile, a scalar load issued
//    before the step's softmax) STRAIGHT INTO LDS (global_load_lds: the data
//    never passes through registers, and no LDS write instruction competes
//    with the operand reads), two to three tiles ahead, into four LDS buffers
//    per pool, row-major ([token][dim]), unpadded, 16-byte chunks swizzled
//    within a row so that the operand reads stay free of bank conflicts.
//    Every load is unconditional (addresses are clamped into the sequence's
//    blocks; rows of a V tile past the context are overwritten with zeros
//    once they have landed), so the waits on the memory counter are exact and
//    a tile's latency hides behind two tiles of arithmetic.
//  * Two-sided schedule: the waves of a SIMD run half a tile apart, one in
//    its matrix step while the other is in its vector (softmax) step, with a
//    workgroup barrier between steps; see the loop at the end of the kernel.
//  * Scores are computed TRANSPOSED, S^T = K Q^T: in the MFMA result layout a
//    lane then holds one query column, so the softmax row maximum and row sum
//    are in-lane reductions plus one exchange between the two lane halves,
//    and the rescale of the output accumulator is a per-lane scalar.
//  * O^T += V^T P^T: the probabilities, rounded to the element type, are
//    already in B-operand order (with a fixed permutation of the token index
//    inside each 16-token step), and the matching V^T operand is read from
//    the row-major LDS tile with the transposing LDS read
//    (ds_read_b64_tr_b16), which hands each lane 4 consecutive tokens of one
//    head-dim column.  No transpose pass over V is needed.
//  * Tiles wholly above the causal diagonal are skipped; only tiles that touch
//    it pay for the mask.  Rows past the context length are zero-filled when
//    the tile is staged, so stale pool contents cannot leak.
//
// FLOPs per launch (what utilisation is quoted against): 4*hn*hd per visible
// (query, key) pair = 4*hn*hd * sum_i (C_i*P_i + C_i*(C_i+1)/2).
#include "prefill_common.h"
#include "../../include/ironcore_paged.h"

namespace ic {

using namespace prefill;

namespace {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;


// MFMA wrappers per element type: operands are 8 packed 16-bit values.
struct MmaBf16 {
  using T = __bf16;
  static __device__ __forceinline__ f32x16_t mma(const Vec16 &a, const Vec16 &b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    bf16x2_t v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
  }
};
struct MmaF16 {
  using T = _Float16;
  static __device__ __forceinline__ f32x16_t mma(const Vec16 &a, const Vec16 &b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f16x2_t v = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
  }
};

constexpr int kPrefillWaves = 8;
constexpr int kPrefillThreads = kPrefillWaves * kWave;
constexpr int kXcds = 8;
constexpr int kBN = 64;                   // tokens per K/V tile
constexpr int kBM = kPrefillWaves * 32;   // query rows per workgroup
constexpr int kStageBuffers = 4;          // LDS buffers per pool: a tile is fetched three tiles ahead

// SINGLE: every sequence is one pool block (a dense [b, sk, gn, hd] tensor
// viewed as a pool); otherwise blocks are a multiple of 16 tokens long.
// MASK: visibility comes from a byte mask instead of the causal rule; every
// query row walks all L keys and a chunk may be longer than its context.
template <class M, int HD, bool SINGLE, bool MASK>
__global__ __launch_bounds__(kPrefillThreads) void paged_prefill_kernel(const PrefillKP p) {
  using T = typename M::T;
  constexpr int KS = HD / 16;          // k-steps of the QK contraction
  constexpr int OB = HD / 32;          // 32-wide blocks of the output head dim
  constexpr int TB = kBN / 32;         // 32-token blocks per tile
  constexpr int CPR = HD / 8;          // 16-byte chunks per token row
  constexpr int WR = kWave / CPR;      // token rows one load instruction of a wave covers
  constexpr int NST = 16 / WR;         // loads (16-byte pieces) per lane and staged tile
  constexpr int ROWB = HD * 2;         // bytes of one token row; LDS tiles are unpadded [token][dim]
  constexpr int NB = kStageBuffers;    // LDS buffers per pool
  static_assert(kBN == 64 && 16 % WR == 0 && (CPR == 4 || CPR == 8 || CPR == 16), "tile staging shape");

  // A tile reaches LDS straight from memory (global_load_lds: no registers, no LDS write
  // instruction), 1 KiB per wave and load, lane l's 16 bytes at byte 16*l of that KiB.  Rows are
  // therefore unpadded, and what keeps the operand reads free of bank conflicts is a swizzle:
  // 16-byte chunk c of tile row r lives in slot c ^ swz(r) of its row (the lane that fills a slot
  // simply fetches the chunk that belongs there).  K (read as whole 16-byte chunks, 16 rows per
  // access): swz = r % 16 (head dim 128), (r / 2) % 8 (head dim 64), (r / 4) % 4 (head dim 32).
  // V (read by the transposing 8-byte reads, 4 rows x 64 bytes per access): swz = 4 * (r % 4),
  // resp. 4 * ((r / 2) % 2); none at head dim 32, where a row is one 64-byte group.
  __shared__ __attribute__((aligned(1024))) char s_k[NB][kBN * ROWB];
  __shared__ __attribute__((aligned(1024))) char s_v[NB][kBN * ROWB];
  auto swz_k = [](int r) { return CPR == 16 ? (r & 15) : CPR == 8 ? ((r >> 1) & 7) : ((r >> 2) & 3); };
  auto swz_v = [](int r) { return CPR == 16 ? ((r & 3) << 2) : CPR == 8 ? (((r >> 1) & 1) << 2) : 0; };

  // XCD-aware placement.  Workgroups are dealt to the 8 XCDs round-robin by
  // their linear id, and each XCD has its own L2.  All workgroups that read
  // the same K/V rows (one (sequence, KV head) unit: its G query heads x its
  // query tiles) get ids that differ by a multiple of 8, so they share an L2
  // and the rows come from HBM once.
  const int per_unit = p.group * p.n_qtiles;
  const int slice = blockIdx.x / (kXcds * per_unit);
  const int within = blockIdx.x - slice * (kXcds * per_unit);
  const int unit = slice * kXcds + (within % kXcds);  // (sequence, KV head)
  if (unit >= p.n_units) return;
  const int r = within / kXcds;
  // Longest first: workgroups are dispatched in id order and differ in length
  // by the spread of context lengths (and, under the causal mask, by their
  // query tile), so early ids take the longest sequences and the last query
  // tiles.  Sequences are ranked by context length on the fly (up to one per
  // lane).
  int seq = unit / p.gn;
  const int kvh = unit - seq * p.gn;
  const int n_seqs = p.n_units / p.gn;
  int q_lo, L, C;
  if (n_seqs <= kWave) {
    // (the chunk bounds travel with the context lengths, one sequence per lane: the chosen
    // sequence's come from its lane instead of a second round trip to memory)
    const int ln = threadIdx.x & (kWave - 1);
    const int mine = ln < n_seqs ? p.context_lens[ln] : -0x7fffffff;
    const int lo_mine = ln < n_seqs ? p.cu_seqlens_q[ln] : 0;
    const int hi_mine = ln < n_seqs ? p.cu_seqlens_q[ln + 1] : 0;
    int rank = 0;
    for (int j = 0; j < n_seqs; ++j) {
      const int other = __builtin_amdgcn_readlane(mine, j);
      rank += (other > mine || (other == mine && j < ln)) ? 1 : 0;
    }
    const uint64_t hit = __ballot(rank == seq && ln < n_seqs);
    seq = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(hit | (1ull << 63)));
    seq = seq < n_seqs ? seq : n_seqs - 1;
    q_lo = __builtin_amdgcn_readlane(lo_mine, seq);
    L = __builtin_amdgcn_readlane(mine, seq);
    C = __builtin_amdgcn_readlane(hi_mine, seq) - q_lo;
  } else {
    q_lo = p.cu_seqlens_q[seq];
    L = p.context_lens[seq];
    C = p.cu_seqlens_q[seq + 1] - q_lo;
  }
  const int h = kvh * p.group + r / p.n_qtiles;
  const int q0 = (p.n_qtiles - 1 - r % p.n_qtiles) * kBM;
  const bool causal = !MASK && p.causal;
  if (L < 0) L = 0;
  if (causal && C > L) C = L;  // under the causal rule a chunk cannot be longer than its context
  if (q0 >= C) return;
  if (L == 0) {  // query rows without any key (not under the causal rule): zero rows
    const int rows = C - q0 < kBM ? C - q0 : kBM;
    for (int idx = threadIdx.x; idx < rows * (HD / 8); idx += kPrefillThreads)
      store16(p.out + ((q_lo + q0 + idx / (HD / 8)) * p.out_stride_token + (int64_t)h * HD + (idx % (HD / 8)) * 8) * 2,
              Vec16{{0u, 0u, 0u, 0u}});
    return;
  }
  const int P = L - C;  // cached prefix (causal rule only)
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int side = wave >> 2;  // 0: waves 0-3, 1: waves 4-7 (one of each per SIMD)
  const int n = lane & 31;     // query column of this lane within the wave's 32-row block
  const int hh = lane >> 5;    // which half of each k-step this lane feeds

  // ---- query rows: registers for the whole sweep, as MFMA B operands ------------
  const int my_q = q0 + wave * 32 + n;
  const int qrow = my_q < C ? my_q : C - 1;
  const int limit = causal ? P + qrow : L - 1;  // last key this query row may see
  Vec16 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = load16(p.q + ((q_lo + qrow) * p.q_stride_token + (int64_t)h * HD + ks * 16 + hh * 8) * 2);

  f32x16_t o[OB];
  float m = kNegInf, l = 0.f;
#pragma unroll
  for (int ob = 0; ob < OB; ++ob)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[ob][i] = 0.f;

  int kv_end = causal ? P + q0 + kBM : L;  // keys any row of this workgroup can see
  kv_end = kv_end < L ? kv_end : L;
  const int n_tiles = (kv_end + kBN - 1) / kBN;
  // tiles this wave's rows reach (the causal diagonal cuts the later ones off;
  // a wave whose rows all lie past the end of the chunk has nothing to compute)
  int my_end = causal ? P + q0 + wave * 32 + 32 : L;
  my_end = my_end < kv_end ? my_end : kv_end;
  const int my_tiles = (my_end > 0 && q0 + wave * 32 < C) ? (my_end + kBN - 1) / kBN : 0;

  // ---- tile staging: memory -> LDS ---------------------------------------------------
  // A wave stages one 16-row group of every tile (group wave & 3) of ONE pool:
  // the waves of side 0 stage K, those of side 1 stage V.  Pool blocks are a
  // multiple of 16 rows long (or the sequence is a single block), so a
  // group lies inside one block: one table entry and one base address per wave
  // and tile, scalar work, and a lane only adds fixed offsets.  Nothing here is
  // conditional: a tile index past the sweep is clamped to the last tile, a
  // block index past the sequence to its last block (whose 16-row groups are
  // allocated whether filled or not), and in SINGLE mode a row past the context
  // to the last row; so every wave has the same number of loads in flight at the
  // same point of the program and the waits on the memory counter are exact.
  // The loads are written as inline assembly: to the compiler an LDS-writing
  // load is something every later LDS read must wait for, which would serialise
  // the prefetch; here the order is kept by hand (landed() before the workgroup
  // barrier that precedes a tile's first read).
  const int grp = wave & 3;
  const int cc = lane % CPR;    // LDS slot (16-byte chunk of the row) this lane fills
  const int rsub = lane / CPR;  // row within the rows one load covers
  // The address of a group is scalar work done once per tile in the vector step, whose length
  // the launch time follows: 32-bit factors (the host refuses pool blocks of 4 GiB and more),
  // one 32 x 32 -> 64-bit product per tile.
  const char *pool_head = (side == 0 ? p.k_pool : p.v_pool) + (int64_t)kvh * p.stride_head * 2;
  const uint32_t block_bytes = (uint32_t)(p.stride_block * 2);
  const uint32_t token_bytes = (uint32_t)(p.stride_token * 2);
  const int last_phys = (int)p.num_blocks - 1;
  // pool block of a row (wave-uniform: one multiplication on the scalar unit by the reciprocal
  // of the block size the host prepared, whatever multiple of 16 the block size is)
  auto block_of = [&](int row) { return (int)__umulhi((uint32_t)row, p.block_magic); };
  const int last_blk = SINGLE ? 0 : block_of(L - 1);
  typedef const __attribute__((address_space(4))) int32_t *TablePtr;  // scalar (SMEM) loads
  const TablePtr table_row = (TablePtr)(unsigned long long)(p.block_tables + (int64_t)seq * p.bt_stride);
  // byte offset, from the group's first row, of the chunk lane l fetches with load i: row
  // i*WR + rsub of the group, and the chunk whose place in that row is this lane's slot; less
  // the 1 KiB per load that the load's instruction offset adds (see fetch_rows; rows are at
  // least ROWB bytes apart, so this stays non-negative)
  uint32_t lane_src[NST];
#pragma unroll
  for (int i = 0; i < NST; ++i) {
    const int r = i * WR + rsub;  // (a group starts at a multiple of 16 rows: r stands for the tile row)
    const int chunk = cc ^ (side == 0 ? swz_k(r) : swz_v(r));
    lane_src[i] = (uint32_t)((int64_t)r * p.stride_token * 2 + chunk * 16) - i * WR * ROWB;
  }
  const uint32_t lds_pool = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)(side == 0 ? &s_k[0][0] : &s_v[0][0]);
  auto clamp_tile = [&](int tile) { return tile < n_tiles ? tile : n_tiles - 1; };
  // Table entry of this wave's group of `tile`, and the group's first row within its block.
  auto lookup = [&](int tile, int32_t &ent, int &rem) {
    const int first = clamp_tile(tile) * kBN + 16 * grp;  // this wave's first row of the tile
    int blk = SINGLE ? 0 : block_of(first);
    rem = first - blk * p.block_size;
    blk = blk < last_blk ? blk : last_blk;
    ent = table_row[blk];
  };
  // Issue the loads of this wave's group of `tile` into the tile's LDS buffer.
  auto fetch_rows = [&](int tile, int32_t ent, int rem) {
    int phys = ent;
    // A corrupt table entry must not become an out-of-pool address.
    phys = phys < 0 ? 0 : phys;
    phys = phys > last_phys ? last_phys : phys;
    const uint32_t dst = lds_pool + (uint32_t)((tile & (NB - 1)) * (kBN * ROWB) + 16 * grp * ROWB);
    if (SINGLE) {
      const int first = clamp_tile(tile) * kBN + 16 * grp;
      const char *base = pool_head + (uint64_t)(uint32_t)phys * block_bytes;
#pragma unroll
      for (int i = 0; i < NST; ++i) {
        int row = first + rsub + i * WR;
        row = row < L ? row : L - 1;
        const int chunk = cc ^ (side == 0 ? swz_k(i * WR + rsub) : swz_v(i * WR + rsub));
        const char *src = base + (int64_t)row * p.stride_token * 2 + chunk * 16;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                     :: "s"(dst + i * WR * ROWB), "v"(src) : "memory", "m0");
      }
    } else {
      const char *base = pool_head + ((uint64_t)(uint32_t)phys * block_bytes + (uint32_t)rem * token_bytes);
      // One LDS base for the group's loads: a load's instruction offset moves its LDS address
      // AND its memory address, here by the 1 KiB that one load fills (lane_src takes it off the
      // memory side again).
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" :: "s"(dst) : "memory", "m0");
#pragma unroll
      for (int i = 0; i < NST; ++i)
        asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2"
                     :: "v"(lane_src[i]), "s"(base), "n"(i * WR * ROWB) : "memory", "m0");
    }
  };
  // The loads of `tile` have arrived (everything but the `younger` loads issued after them); rows
  // of a V tile past the context become zeros (their probabilities are zeros, but 0 x NaN is not:
  // unused pool slots may hold anything).  The workgroup barrier that follows makes the tile
  // readable.
  auto landed = [&](int tile, int younger_tiles) {
    if (younger_tiles == 0)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (younger_tiles == 1)
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NST) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * NST) : "memory");
    if (tile == n_tiles - 1 && side == 1 && tile * kBN + 16 * grp + 16 > L) {  // (only a sweep's last tile can reach past L)
      char *buf = s_v[tile & (NB - 1)] + 16 * grp * ROWB + lane * 16;
      const int row = tile * kBN + 16 * grp + rsub;
#pragma unroll
      for (int i = 0; i < NST; ++i)
        if (row + i * WR >= L) store16(buf + i * WR * ROWB, Vec16{{0u, 0u, 0u, 0u}});
    }
  };

  // per-lane LDS offsets of the operand reads (the swizzles above, seen from the reading side)
  // K: row tb*32 + n, chunk 2*ks + hh  ->  (n*ROWB + 16*(hh ^ swz)) ^ 32*ks, + tb*32*ROWB
  const int k_lane = n * ROWB + ((hh ^ swz_k(n)) << 4);
  // V: rows kk*16 (+8) + 4*hh + q, bytes ob*64 + 32*bit4 + 8*(lane & 3)  ->  base ^ 64*ob
  const int vq = (lane & 15) >> 2;
  const int v_lane = (4 * hh + vq) * ROWB + ((swz_v(vq) >> 2) << 6) + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);

  // First tile that needs the mask: the one the causal diagonal of the wave's first row enters
  // (tile*64 + 63 > P + that row), or without the causal rule a last tile the context does not fill.
  const int mask_from = __builtin_amdgcn_readfirstlane(causal ? (P + q0 + wave * 32 + 1) / kBN : L / kBN);
  f32x16_t s[TB];        // S^T of the tile in flight: (token, query n)
  Vec16 pb[kBN / 16];    // its probabilities as MFMA B operands

  // ---- S^T = K Q^T ----------------------------------------------------------------
  auto scores = [&](int tile) {
    const char *sk = s_k[tile & (NB - 1)];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[tb][i] = 0.f;
    // (k-step outermost: consecutive MFMAs share their B operand, the query fragment, and go to
    // different accumulators; measured 1-2 % faster than token block outermost)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int tb = 0; tb < TB; ++tb) {
        const Vec16 a = load16(sk + (k_lane ^ (ks * 32)) + tb * 32 * ROWB);
        s[tb] = M::mma(a, qf[ks], s[tb]);
      }
    }
    // Operand reads run kAhead MFMAs ahead of their use: left to itself the
    // scheduler issues them two at a time, right before the MFMAs that need
    // them, and every pair waits out an LDS round trip (+2.5 % on the kernel;
    // the other product already gets its reads eight ahead).
    constexpr int kAhead = TB * KS < 6 ? TB * KS : 6;
    __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
    for (int i = 0; i < TB * KS - kAhead; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
  };
  // ---- softmax of the tile's scores: s -> pb, m, l (and o when the reference moves) ----
  auto softmax = [&](int tile) {
    // s[tb][i] is (token tile*64 + tb*32 + 4*hh + 8*(i/4) + i%4, query n)
    const int tok_base = tile * kBN + 4 * hh;
    const bool need_mask = tile >= mask_from;
    if (need_mask) {  // tiles that touch the causal diagonal (or the context end)
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int tok = tok_base + tb * 32 + 8 * (i / 4) + (i & 3);
          s[tb][i] = tok > limit ? kNegInf : s[tb][i];
        }
    }
    if constexpr (MASK) {  // keys the caller's mask hides from this lane's query row
      const uint8_t *mrow = p.mask + (int64_t)seq * p.mask_stride_seq + (int64_t)h * p.mask_stride_head +
                            (int64_t)qrow * p.mask_stride_row;
      // Every byte is fetched unconditionally, from an index clamped into the part of the row
      // that exists and counts (keys below both the context length and the mask's extent), so
      // the 32 loads of a tile are independent and in flight together; a key past the mask's
      // extent is hidden whatever the byte fetched in its place says.
      const int last = (limit < p.mask_keys - 1 ? limit : p.mask_keys - 1);
      uint8_t seen[TB][16];
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int tok = tok_base + tb * 32 + 8 * (i / 4) + (i & 3);
          seen[tb][i] = mrow[tok < last ? tok : last];
        }
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int tok = tok_base + tb * 32 + 8 * (i / 4) + (i & 3);
          const bool hidden = (tok <= limit) & ((tok >= p.mask_keys) | (seen[tb][i] == 0));
          s[tb][i] = hidden ? kHiddenScore : s[tb][i];
        }
    }
    // Row maximum on the raw scores (the scale is positive), one exchange
    // between the lane halves, then into log2 units.
    float mx = kNegInf;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[tb][i]);
    float mx_a, mx_b;
    both_halves(mx, mx_a, mx_b);
    mx = fmaxf(mx_a, mx_b) * p.scale_log2e;
    // Lazy reference maximum: it moves (and the accumulators are rescaled)
    // only when some row's maximum rises by more than 2^kLazySlack above
    // it.  Until then probabilities may exceed 1 (<= 2^kLazySlack), which
    // fp32 sums and the 16-bit P operand hold without loss of accuracy.
    if (__any(mx > m + kLazySlack)) {
      const float m_new = fmaxf(m, mx);
      const float alpha = (m == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
      m = m_new;
      l *= alpha;
#pragma unroll
      for (int ob = 0; ob < OB; ++ob)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[ob][i] *= alpha;
    }
    const float neg_ms = (m == kNegInf) ? 0.f : -m;
    float ps = 0.f;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[tb][i], p.scale_log2e, neg_ms));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[tb][i + 1], p.scale_log2e, neg_ms));
        ps += p0 + p1;
        pb[2 * tb + i / 8].w[(i & 7) / 2] = M::pack2(p0, p1);
      }
    }
    l += ps;
  };
  // ---- O^T += V^T P^T ---------------------------------------------------------------
  auto weighted_values = [&](int tile) {
    const char *sv = s_v[tile & (NB - 1)];
    // (token step outermost: the OB MFMAs of a step share their B operand, the probabilities)
#pragma unroll
    for (int kk = 0; kk < kBN / 16; ++kk) {
#pragma unroll
      for (int ob = 0; ob < OB; ++ob) {
        const char *at = sv + (v_lane ^ (ob * 64)) + kk * 16 * ROWB;
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t *)(at));
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t *)(at + 8 * ROWB));
        const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        o[ob] = M::mma(__builtin_bit_cast(Vec16, both), pb[kk], o[ob]);
      }
    }
    // the operand reads (two per MFMA) run four MFMAs ahead of their use, as in scores()
    constexpr int kAheadV = 4;
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAheadV, 0);
#pragma unroll
    for (int i = 0; i < OB * (kBN / 16) - kAheadV; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kAheadV, 0);
  };

  // ---- two-sided pipeline ---------------------------------------------------------------
  // A tile costs a wave about as many matrix-core cycles (K Q^T, V^T P^T) as
  // vector-ALU cycles (softmax).  Each SIMD holds one wave of either side, and
  // the sides run half a tile apart: in every phase one of them is in its
  // matrix step M(k) = { O += V(k-1) P(k-1) ; S = K(k) Q } while the other is in
  // its vector step V(k') = { P(k') = softmax(S) }, so the two pipes of a SIMD are
  // busy at the same time.  A workgroup barrier ends each phase.
  //   side 0:  M(0) V(0) M(1) V(1) ... M(n) V(n)  -
  //   side 1:   -   M(0) V(0) M(1) ... V(n-1) M(n) V(n)
  // LDS: four buffers per pool.  K(k) is read in phases 2k and 2k+1, V(k) in phases 2k+2 and
  // 2k+3.  In its vector step k a wave first makes sure its group of tile k+1 has arrived (the
  // barrier that ends the step publishes it: K(k+1) is first read in phase 2k+2, V(k+1) in phase
  // 2k+4), then issues the loads of tile k+3 into the buffer tile k-1 left (last read in phase
  // 2k-1 for K, 2k+1 for V: one barrier before the issue at the latest).  So a tile's loads are
  // in flight for four phases, and a wave always has two tiles of its pool on the way.
  int32_t ent;  // table entry of the tile the next vector step fetches
  int ent_rem;  // and the first row of this wave's group within that block
  auto matrix_step = [&](int k) {
    // the wave in its matrix step goes first when both waves of the SIMD have an instruction ready:
    // an MFMA or operand read issued late idles the matrix pipe, a softmax instruction issued late
    // costs nothing as long as the step ends in time (measured 1.5 %)
    __builtin_amdgcn_s_setprio(3);
    if (k >= 1 && k <= my_tiles) weighted_values(k - 1);
    if (k < my_tiles) {
      scores(k);
    } else {  // nothing to score: leave no stale value alive across the loop
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[tb][i] = 0.f;
    }
  };
  // Tile `tile` has arrived; fetch tile + 2; then the softmax of tile j.  The memory operations
  // go first and complete behind the softmax, which has no LDS or scalar-memory operation whose
  // wait would include them.
  auto vector_step = [&](int j, int tile) {
    __builtin_amdgcn_s_setprio(0);
    landed(tile, 1);
    fetch_rows(tile + 2, ent, ent_rem);
    lookup(tile + 3, ent, ent_rem);  // for the next vector step, which fetches tile + 3
    if (j >= 0 && j < my_tiles) {
      softmax(j);
    } else {
#pragma unroll
      for (int kk = 0; kk < kBN / 16; ++kk) pb[kk] = Vec16{{0u, 0u, 0u, 0u}};
    }
  };
  // prologue: side 0 issues K(0), K(1), K(2) and waits for K(0); side 1 issues V(0), V(1)
  // (all table entries first, then all tiles: one round trip each, not one per tile)
  if (side == 0) {
    int32_t e0, e1, e2;
    int r0, r1, r2;
    lookup(0, e0, r0);
    lookup(1, e1, r1);
    lookup(2, e2, r2);
    lookup(3, ent, ent_rem);  // the first vector step waits for K(1) and fetches K(3)
    fetch_rows(0, e0, r0);
    fetch_rows(1, e1, r1);
    fetch_rows(2, e2, r2);
    landed(0, 2);
  } else {
    int32_t e0, e1;
    int r0, r1;
    lookup(0, e0, r0);
    lookup(1, e1, r1);
    lookup(2, ent, ent_rem);  // the first vector step waits for V(0) and fetches V(2)
    fetch_rows(0, e0, r0);
    fetch_rows(1, e1, r1);
  }
  __syncthreads();
  // Both sides pass the same number of barriers.
  const int n_steps = (n_tiles + 2) & ~1;  // steps k = 0 .. n_steps-1 cover M(0..n_tiles), rounded up to even
  if (side == 0) {
    for (int k = 0; k < n_steps; ++k) {
      matrix_step(k);
      __syncthreads();
      vector_step(k, k + 1);  // publishes K(k+1)
      __syncthreads();
    }
    __syncthreads();
  } else {
    vector_step(-1, 0);  // publishes V(0)
    __syncthreads();
    for (int k = 0; k < n_steps; ++k) {
      matrix_step(k);
      __syncthreads();
      vector_step(k, k + 1);  // publishes V(k+1)
      __syncthreads();
    }
  }
  // every load this wave issued must have landed before its LDS is given up
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- normalise and store -------------------------------------------------------
  float l_a, l_b;
  both_halves(l, l_a, l_b);
  const float lt = l_a + l_b;
  const float inv = lt > 0.f ? 1.f / lt : 0.f;
  if (my_q < C) {
    T *orow = reinterpret_cast<T *>(p.out) + (q_lo + my_q) * p.out_stride_token + (int64_t)h * HD;
#pragma unroll
    for (int ob = 0; ob < OB; ++ob) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = ob * 32 + 4 * hh + 8 * j;
        uint2 w;
        w.x = M::pack2(o[ob][4 * j] * inv, o[ob][4 * j + 1] * inv);
        w.y = M::pack2(o[ob][4 * j + 2] * inv, o[ob][4 * j + 3] * inv);
        *reinterpret_cast<uint2 *>(orow + d) = w;
      }
    }
  }
}

template <class M, bool SINGLE, bool MASK>
int launch_hd(PrefillKP kp, const PrefillArgs &a, hipStream_t stream) {
  kp.n_qtiles = (a.max_chunk_len + kBM - 1) / kBM;
  const int64_t slices = (kp.n_units + kXcds - 1) / kXcds;
  const int64_t wgs = slices * kXcds * kp.group * kp.n_qtiles;
  if (wgs > 0x7fffffff) return IC_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)wgs);
  switch (a.hd) {
    case 32:
      hipLaunchKernelGGL((paged_prefill_kernel<M, 32, SINGLE, MASK>), grid, dim3(kPrefillThreads), 0, stream, kp);
      break;
    case 64:
      hipLaunchKernelGGL((paged_prefill_kernel<M, 64, SINGLE, MASK>), grid, dim3(kPrefillThreads), 0, stream, kp);
      break;
    case 128:
      hipLaunchKernelGGL((paged_prefill_kernel<M, 128, SINGLE, MASK>), grid, dim3(kPrefillThreads), 0, stream, kp);
      break;
    default:
      return IC_ERR_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? IC_OK : IC_ERR_LAUNCH;
}

template <class M>
int launch_mode(const PrefillKP &kp, const PrefillArgs &a, hipStream_t stream) {
  // A one-column block table means one block per sequence, of any length.
  const bool masked = a.mask != nullptr;
  if (a.block_table_stride == 1)
    return masked ? launch_hd<M, true, true>(kp, a, stream) : launch_hd<M, true, false>(kp, a, stream);
  if (kp.block_size < 16 || kp.block_size % 16 != 0) return IC_ERR_UNSUPPORTED;  // whole 16-token groups
  return masked ? launch_hd<M, false, true>(kp, a, stream) : launch_hd<M, false, false>(kp, a, stream);
}

}  // namespace

int launch_paged_prefill(const PrefillArgs &a, hipStream_t stream) {
  PrefillKP kp;
  kp.q = (const char *)a.q;
  kp.k_pool = (const char *)a.k_pool;
  kp.v_pool = (const char *)a.v_pool;
  kp.block_tables = a.block_tables;
  kp.context_lens = a.context_lens;
  kp.cu_seqlens_q = a.cu_seqlens_q;
  kp.out = (char *)a.out;
  kp.q_stride_token = a.q_stride_token;
  kp.out_stride_token = a.out_stride_token;
  kp.stride_block = a.pool.stride_block;
  kp.stride_head = a.pool.stride_head;
  kp.stride_token = a.pool.stride_token;
  kp.bt_stride = a.block_table_stride;
  kp.num_blocks = a.pool.num_blocks;
  kp.block_size = a.pool.block_size;
  kp.block_shift = -1;
  for (int s = 0; s < 31; ++s)
    if ((1 << s) == a.pool.block_size) kp.block_shift = s;
  kp.block_magic = 0;
  if (a.pool.block_size >= 2) {
    kp.block_magic = (uint32_t)((1ull << 32) / (uint32_t)a.pool.block_size) + (kp.block_shift < 0 ? 1u : 0u);
    // a block size that is no power of two: the reciprocal is exact for token rows below
    // 2^32 / block_size; tables that reach further are refused
    if (kp.block_shift < 0 && a.block_table_stride > 1 &&
        a.block_table_stride * (int64_t)a.pool.block_size >= ((int64_t)1 << 32) / a.pool.block_size)
      return IC_ERR_UNSUPPORTED;
  }
  kp.group = a.hn / a.gn;
  kp.gn = a.gn;
  kp.n_units = a.n_seqs * a.gn;
  kp.n_qtiles = 0;
  kp.causal = a.causal;
  kp.scale_log2e = a.scale * 1.4426950408889634f;
  kp.mask = a.mask;
  kp.mask_stride_seq = a.mask_stride_seq;
  kp.mask_stride_head = a.mask_stride_head;
  kp.mask_stride_row = a.mask_stride_row;
  kp.mask_keys = a.mask_keys > 0x7fffffff ? 0x7fffffff : (int)a.mask_keys;
  if ((int64_t)a.max_chunk_len >= (int64_t)65535 * 128 || a.hn > 65535 || a.n_seqs > 65535)
    return IC_ERR_UNSUPPORTED;
  // The 16-bit kernel addresses a block with 32-bit byte offsets (a block, and in a block table's
  // blocks the rows from a block's start to any of its 16-row groups, stay below 4 GiB; the 16
  // rows of a group below 4 GiB in any case) and numbers blocks with 32 bits, as the tables do.
  if (a.dtype != IC_DTYPE_F32) {
    const int64_t span_rows = a.block_table_stride > 1 && a.pool.block_size > 16 ? a.pool.block_size : 16;
    if (a.pool.stride_block >= ((int64_t)1 << 31) || a.pool.stride_token * span_rows >= ((int64_t)1 << 31) ||
        a.pool.num_blocks > 0x7fffffff)
      return IC_ERR_UNSUPPORTED;
  }
  switch (a.dtype) {
    case IC_DTYPE_BF16: return launch_mode<MmaBf16>(kp, a, stream);
    case IC_DTYPE_F16: return launch_mode<MmaF16>(kp, a, stream);
    case IC_DTYPE_F32: return launch_paged_prefill_f32(kp, a, stream);
    default: return IC_ERR_UNSUPPORTED;
  }
}

}  // namespace ic

// Causal grouped-query attention over the paged cache on the matrix cores (bfloat16 in,
// float32 accumulate), one kernel for prompt portions and decoded tokens alike.
//
// Work is cut into tiles of 16 *rows*; a row is a (token, query head) pair of one sequence and
// one key/value head: row f of the sequence stands for token f / G and head kvh * G + f % G,
// G being the number of query heads per key/value head.  All 16 rows of a tile read the same
// keys and values, so a decoded token's G heads (7 for 14 query heads over 2) fill one tile and
// the cache is read once for all of them; a prompt portion yields ceil(tokens * G / 16) tiles.
// Every wavefront owns one (tile, kv head, key split) and needs no shared memory:
//
//   S^T[key, row]  = K[key, :] . Q[row, :]        v_mfma_f32_16x16x32_bf16, A = K, B = Q^T
//   online softmax over keys in float32 (each lane holds 8 keys of one row)
//   O^T[dim, row] += V^T[dim, key] P^T[key, row]  A = V^T, B = P^T
//
// The 16x16 result of the first product leaves each lane with exactly the probabilities the
// second product wants from it as its B operand, and values are stored transposed within a
// page ([page, kv head, dim, slot]), so its A operand is a plain 8-byte load: the
// probabilities never leave registers.
//
// A long context is split along the keys over gridDim.z; each split writes an unnormalised
// partial result with its running maximum and sum, and a second kernel merges them in split
// order.  Formulas: reference mercury/model/attention.py:9-32, :61-74, :87-101.
#include "common.h"
#include "mercury_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

union Frag {
  bf16x8 v;
  uint4 u;
  uint2 u2[2];
  uint16_t h[8];
};

struct AttnParams {
  const bf16_t* q;
  int q_stride;
  bf16_t* out;
  int out_stride;
  float* part_o;   // [tile, kv head, split, tile_rows, D]
  float* part_ml;  // [tile, kv head, split, tile_rows, 2]
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  const int* tile_seq;
  const int* tile_row0;
  const int* cu_q;
  const int* kv_len;
  const int* block_table;
  int table_stride;
  int page_shift;
  int n_kv;
  int group;
  float scale;
  int window;
  int num_tiles;
  int num_splits;
  int split_blocks;  // key blocks per split; 0: each tile's range divided evenly
  int tile_rows;     // rows per tile: 16, 32 or 64
  int kv_fold;       // key/value heads per workgroup of the unstaged kernel: 1, 2 or 4
  int direct;        // no tile list: tile t is the one new token of sequence t
};

#define ATTN_WAVES 4
// Blocks of keys in flight beyond the one being used, per tile width (16, 32, 64 rows).
#ifndef ATTN_AHEAD_16
#define ATTN_AHEAD_16 1
#define ATTN_AHEAD_32 1
#define ATTN_AHEAD_64 0
#endif

// The keys and values of one block of 32 keys, as MFMA operands of this lane.
template <int D>
struct KeyBlock {
  Frag kf[2][D / 32];
  Frag vf[D / 16];
  bool live[2];
};

// The wavefront's view of its sequence's block table: 64 entries at a time, one per lane,
// handed out by lane index, so that finding a block's page costs no trip to memory.
struct TableWindow {
  const int* table;
  int width, base, mine;
  __device__ __forceinline__ int page(int index, int lane) {
    if (index >= base + 64) {  // uniform: every lane asks for the same index, never a lower one
      base = index;
      mine = index + lane < width ? table[index + lane] : 0;
      // Waited for here, once in 64 pages, so that no wait stands before the readlane below:
      // that one would also wait, every time, for the keys and values asked for ahead.
      __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
    }
    return __builtin_amdgcn_readlane(mine, index - base);
  }
};

// Loads are unconditional: a half that is not live (outside the keys the tile sees, or past
// the split's end while prefetching) reads page 0, which always exists, and its keys are
// masked in the scores.  Addresses are a wavefront-uniform base plus a 32-bit lane offset.
template <int D>
__device__ __forceinline__ void load_key_block(KeyBlock<D>& blk, const AttnParams& p,
                                               TableWindow& tw, int b, int b_end, int kmin,
                                               int kmax, int kvh, int lane) {
  const int r = lane & 15, g4 = lane >> 4;
  const int ps = 1 << p.page_shift;
  const uint32_t k_lane = (uint32_t)(r * D + g4 * 8) * 2u;   // bytes
  const uint32_t v_lane = (uint32_t)(r * ps + g4 * 4) * 2u;
  const char* kbase[2];
  const char* vbase[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int kh = (b << 5) + h * 16;
    blk.live[h] = b < b_end && kh <= kmax && kh + 15 >= kmin;  // wavefront-uniform
    const int page = blk.live[h] ? tw.page(kh >> p.page_shift, lane) : 0;
    const int off = kh & (ps - 1);
    const size_t head_bytes = ((size_t)page * p.n_kv + kvh) * ((size_t)ps * D * 2);
    kbase[h] = (const char*)p.k_cache + head_bytes + (size_t)off * D * 2;
    vbase[h] = (const char*)p.v_cache + head_bytes + (size_t)off * 2;
  }
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
      blk.kf[h][c].u = *(const uint4*)(kbase[h] + (k_lane + (uint32_t)c * 64u));
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt)
#pragma unroll
    for (int h = 0; h < 2; ++h)
      blk.vf[dt].u2[h] = *(const uint2*)(vbase[h] + (v_lane + (uint32_t)(dt * 32 * ps)));
}

// The same loads for a block whose two halves' pages are known (wavefront-uniform), live or
// not: addresses are valid either way, and what is not live is masked in the scores.
template <int D>
__device__ __forceinline__ void load_key_block_at(KeyBlock<D>& blk, const AttnParams& p, int b,
                                                  int page_lo, int page_hi, bool live, int kvh,
                                                  int lane) {
  const int r = lane & 15, g4 = lane >> 4;
  const int ps = 1 << p.page_shift;
  const uint32_t k_lane = (uint32_t)(r * D + g4 * 8) * 2u;   // bytes
  const uint32_t v_lane = (uint32_t)(r * ps + g4 * 4) * 2u;
  const char* kbase[2];
  const char* vbase[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int kh = (b << 5) + h * 16;
    blk.live[h] = live;
    const int page = h ? page_hi : page_lo;
    const int off = kh & (ps - 1);
    const size_t head_bytes = ((size_t)page * p.n_kv + kvh) * ((size_t)ps * D * 2);
    kbase[h] = (const char*)p.k_cache + head_bytes + (size_t)off * D * 2;
    vbase[h] = (const char*)p.v_cache + head_bytes + (size_t)off * 2;
  }
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
      blk.kf[h][c].u = *(const uint4*)(kbase[h] + (k_lane + (uint32_t)c * 64u));
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt)
#pragma unroll
    for (int h = 0; h < 2; ++h)
      blk.vf[dt].u2[h] = *(const uint2*)(vbase[h] + (v_lane + (uint32_t)(dt * 32 * ps)));
}

// A wavefront's view of the pages of every `stride`-th block of its sequence from `first` on:
// lane l holds the two pages of block first + (base + l) * stride (a block of 32 keys lies in
// one page or, with pages of 16, in two), 64 blocks at a time.
struct StridedPages {
  const int* table;
  int width, first, stride, base, lo, hi;
  __device__ __forceinline__ void fetch(int from, int page_shift, int lane) {
    base = from;
    const int key = (first + (from + lane) * stride) << 5;
    const int a = key >> page_shift, b = (key + 16) >> page_shift;
    // (entries past a sequence's pages are -1: page 0 stands in, its keys are masked)
    lo = a < width ? max(table[a], 0) : 0;
    hi = b < width ? max(table[b], 0) : 0;
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0), here and not before every readlane
  }
  // the pages of the wavefront's j-th block (j never decreases)
  __device__ __forceinline__ void pages(int j, int page_shift, int lane, int& page_lo, int& page_hi) {
    if (j >= base + 64) fetch(j, page_shift, lane);
    page_lo = __builtin_amdgcn_readlane(lo, j - base);
    page_hi = __builtin_amdgcn_readlane(hi, j - base);
  }
};

// The running state of RT tiles of 16 rows: this lane's row of each tile.
template <int D, int RT>
struct TileState {
  Frag qf[RT][D / 32];
  f32x4 acc[RT][D / 16];
  float m[RT], lsum[RT];
  int pos[RT], lo[RT];
  bool row_ok[RT];
};

// One block of 32 keys against the tiles: scores, online softmax, weighted values.  Scores
// are kept in the base-2 domain (`c` = scale * log2 e), so every exponential is one
// instruction.  MASKED is for blocks that some row of the tiles cannot see in full (the
// causal edge, the window's edge, the end of the sequence); inside, nothing is tested.
//
// PERM tells which keys of the block a lane's eight scores belong to.  Without it the two
// products of 16 keys take keys h * 16 + 0..15, and a lane holds keys h * 16 + g4 * 4 + i.
// With it product h takes keys q * 8 + h * 4 + m (q, m = 0..3), and a lane holds the eight
// consecutive keys g4 * 8 + 0..7: its operand of the second product is then one 16-byte
// piece of a row of values.
template <int D, int RT, bool MASKED, bool PERM>
__device__ __forceinline__ void attend_block(TileState<D, RT>& st, const KeyBlock<D>& blk,
                                             int key0, float c, int g4) {
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    float s[8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k = 0; k < D / 32; ++k)
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.kf[h][k].v, st.qf[t][k].v, sc, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = sc[i];
        if (MASKED) {
          const int key = key0 + (PERM ? g4 * 8 + h * 4 + i : h * 16 + g4 * 4 + i);
          const bool ok = blk.live[h] && st.row_ok[t] && key <= st.pos[t] && key >= st.lo[t];
          v = ok ? v : -INFINITY;
        }
        s[h * 4 + i] = v;
      }
    }
    // The largest raw score is also the largest scaled one (c > 0); the scale itself is
    // applied in the fused multiply-add that subtracts the running maximum.
    float bm = c * fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])),
                         fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    // The four lanes of a row exchange their maxima, and what is accumulated is rescaled,
    // only when some lane saw a score above its row's running maximum: rare once a row has
    // seen a few blocks.
    if (__builtin_amdgcn_ballot_w64(bm > st.m[t]) != 0) {
      bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
      bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
      const float m_new = fmaxf(st.m[t], bm);
      const float corr = __builtin_amdgcn_exp2f(st.m[t] - (m_new == -INFINITY ? 0.f : m_new));
      st.lsum[t] *= corr;
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) st.acc[t][dt] *= corr;
      st.m[t] = m_new;
    }
    const float m_use = (MASKED && st.m[t] == -INFINITY) ? 0.f : st.m[t];
    float e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j], c, -m_use));
    st.lsum[t] += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
    Frag pf;
    pf.u = make_uint4(pack_bf16x2(e[0], e[1]), pack_bf16x2(e[2], e[3]), pack_bf16x2(e[4], e[5]),
                      pack_bf16x2(e[6], e[7]));
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt)
      st.acc[t][dt] =
          __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.vf[dt].v, pf.v, st.acc[t][dt], 0, 0, 0);
  }
}

// Blocks wholly inside what every row of the tiles sees take the unmasked path.
template <int D, int RT, bool PERM = false>
__device__ __forceinline__ void attend(TileState<D, RT>& st, const KeyBlock<D>& blk, int key0,
                                       float c, int g4, int all_see_upto, int all_see_from) {
  if (key0 + 31 <= all_see_upto && key0 >= all_see_from)
    attend_block<D, RT, false, PERM>(st, blk, key0, c, g4);
  else
    attend_block<D, RT, true, PERM>(st, blk, key0, c, g4);
}

// RT: 16-row tiles per wavefront.  A decoded token's heads fill one tile (RT = 1, and the
// keys may be split); a prompt portion may give each wavefront RT consecutive tiles, which
// share every key and value fragment the wavefront loads.  AHEAD: how many blocks of keys
// are in flight beyond the one in the matrix cores (0, 1 or 2).
//
// GROUPED (one tile of 16 rows, keys split): the four wavefronts of a workgroup take four
// consecutive parts of one tile's keys for one kv head, and add their results up through LDS
// before anything is written: a quarter of the partial results for the merge, or none at all
// when the workgroup has the tile's whole range.  p.num_splits then counts workgroups per
// tile, each of ATTN_WAVES parts.
//
// DIRECT (decoding: every sequence brings one token, whose heads are one tile): tile t is
// sequence t, so nothing has to be looked up before the block table and the queries are asked
// for; and part s of S takes the blocks s, s + S, s + 2 S, ... of the keys, so a wavefront
// knows its first block, and where in the table its blocks' pages stand, without the
// sequence's length: table, queries and length travel together, the first block's keys and
// values follow, and the length is there when the scores are masked.  Two trips to memory
// before the first product instead of four, and parts that are equal for every sequence
// whatever its length.  (A first block past a sequence's end is read from whatever page the
// table names there, which exists, and masked.)
template <int D, int RT, int AHEAD, bool GROUPED = false, bool DIRECT = false>
__global__ __launch_bounds__(64 * ATTN_WAVES, (RT == 1 && D <= 128 ? 2 : 1)) void attn_mfma_kernel(AttnParams p) {
  static_assert(!GROUPED || (RT == 1 && D <= 128), "grouped parts: one tile, heads up to 128");
  static_assert(!DIRECT || (RT == 1 && AHEAD == 1), "direct: one tile, one block ahead");
  const int lane = threadIdx.x & 63;
  // Tiles are taken from the last: under a causal mask the later tiles of a prompt read the
  // most keys, and the longest work should start first.
  // The wavefronts of a workgroup take `kv_fold` key/value heads of the same tiles: a page
  // holds its heads' keys side by side, and wavefronts that read them at the same time read
  // a longer stretch of memory between them.
  const int wave = threadIdx.x >> 6, fold = GROUPED ? ATTN_WAVES : p.kv_fold;
  const int tile = p.num_tiles - 1 - (blockIdx.x * (ATTN_WAVES / fold) + wave / fold);
  if (tile < 0) return;   // never in a grouped launch: one tile per workgroup
  const int kvh = GROUPED ? blockIdx.y : blockIdx.y * fold + wave % fold;
  const int split = GROUPED ? blockIdx.z * ATTN_WAVES + wave : blockIdx.z;
  const int splits = GROUPED ? p.num_splits * ATTN_WAVES : p.num_splits;
  const int seq = DIRECT ? tile : p.tile_seq[tile], row0 = DIRECT ? 0 : p.tile_row0[tile];
  const int q0 = DIRECT ? seq : p.cu_q[seq], q_len = DIRECT ? 1 : p.cu_q[seq + 1] - q0;
  const int kv_len = p.kv_len[seq];      // (DIRECT: asked for here, first used after the loads below)
  const int G = p.group;
  const int rows_total = q_len * G;
  const int r = lane & 15, g4 = lane >> 4;

  // The rows this lane stands for as a column of S^T and O^T, one per tile.
  TileState<D, RT> st;
  int tok[RT], head[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int flat = row0 + t * 16 + r;
    st.row_ok[t] = flat < rows_total;
    tok[t] = st.row_ok[t] ? flat / G : 0;
    head[t] = kvh * G + (st.row_ok[t] ? flat % G : 0);
    st.m[t] = -INFINITY;
    st.lsum[t] = 0.f;
    const bf16_t* qrow = p.q + (size_t)(q0 + tok[t]) * p.q_stride + head[t] * D + g4 * 8;
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
      st.qf[t][c].u = st.row_ok[t] ? *(const uint4*)(qrow + c * 32) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) st.acc[t][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  TableWindow tw = {p.block_table + (size_t)seq * p.table_stride, p.table_stride, -64, 0};
  StridedPages sp = {tw.table, tw.width, split, splits, 0, 0, 0};
  KeyBlock<D> first_block;
  if constexpr (DIRECT) {
    sp.fetch(0, p.page_shift, lane);          // (the wait inside is for the queries too)
    int page_lo, page_hi;
    sp.pages(0, p.page_shift, lane, page_lo, page_hi);
    load_key_block_at<D>(first_block, p, split, page_lo, page_hi, true, kvh, lane);
  }

  const int pos0 = kv_len - q_len;  // position of the step's first token of the sequence
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    st.pos[t] = pos0 + tok[t];
    st.lo[t] = p.window > 0 ? max(0, st.pos[t] - p.window + 1) : 0;
  }

  // Keys any row of the tiles can see, in blocks of 32, and this split's share of them.
  const int last_flat = min(row0 + 16 * RT - 1, rows_total - 1);
  const int kmax = pos0 + last_flat / G;
  const int kmin = p.window > 0 ? max(0, pos0 + row0 / G - p.window + 1) : 0;
  const int blk_lo = kmin >> 5, blk_hi = (kmax >> 5) + 1;
  const int per = p.split_blocks > 0 ? p.split_blocks : (blk_hi - blk_lo + splits - 1) / splits;
  const int b0 = blk_lo + split * per, b1 = min(blk_hi, b0 + per);
  // Keys [see_from, see_upto] are visible to every valid row of the tiles.
  const int see_upto = pos0 + row0 / G;
  const int see_from = p.window > 0 ? max(0, kmax - p.window + 1) : 0;
  const float c = p.scale * 1.44269504088896340736f;

  if (AHEAD == 0) {
    KeyBlock<D> blk;
    for (int b = b0; b < b1; ++b) {
      load_key_block<D>(blk, p, tw, b, b1, kmin, kmax, kvh, lane);
      attend<D, RT>(st, blk, b << 5, c, g4, see_upto, see_from);
    }
  } else if (AHEAD == 1) {
    KeyBlock<D> x, y;
    if constexpr (DIRECT) {
      // blocks split, split + S, ...: the wavefront's j-th block is b
      x = first_block;
      int page_lo, page_hi;
      for (int b = split, j = 0; b < blk_hi; b += 2 * splits, j += 2) {
        const bool more = b + splits < blk_hi;
        sp.pages(more ? j + 1 : j, p.page_shift, lane, page_lo, page_hi);
        load_key_block_at<D>(y, p, b + splits, page_lo, page_hi, more, kvh, lane);
        attend<D, RT>(st, x, b << 5, c, g4, see_upto, see_from);
        if (more) {
          const bool further = b + 2 * splits < blk_hi;
          sp.pages(further ? j + 2 : j + 1, p.page_shift, lane, page_lo, page_hi);
          load_key_block_at<D>(x, p, b + 2 * splits, page_lo, page_hi, further, kvh, lane);
          attend<D, RT>(st, y, (b + splits) << 5, c, g4, see_upto, see_from);
        }
      }
    } else {
    load_key_block<D>(x, p, tw, b0, b1, kmin, kmax, kvh, lane);
    for (int b = b0; b < b1; b += 2) {
      load_key_block<D>(y, p, tw, b + 1, b1, kmin, kmax, kvh, lane);
      attend<D, RT>(st, x, b << 5, c, g4, see_upto, see_from);
      if (b + 1 < b1) {
        load_key_block<D>(x, p, tw, b + 2, b1, kmin, kmax, kvh, lane);
        attend<D, RT>(st, y, (b + 1) << 5, c, g4, see_upto, see_from);
      }
    }
    }
  } else {
    KeyBlock<D> x, y, z;
    load_key_block<D>(x, p, tw, b0, b1, kmin, kmax, kvh, lane);
    load_key_block<D>(y, p, tw, b0 + 1, b1, kmin, kmax, kvh, lane);
    for (int b = b0; b < b1; b += 3) {
      load_key_block<D>(z, p, tw, b + 2, b1, kmin, kmax, kvh, lane);
      attend<D, RT>(st, x, b << 5, c, g4, see_upto, see_from);
      if (b + 1 < b1) {
        load_key_block<D>(x, p, tw, b + 3, b1, kmin, kmax, kvh, lane);
        attend<D, RT>(st, y, (b + 1) << 5, c, g4, see_upto, see_from);
      }
      if (b + 2 < b1) {
        load_key_block<D>(y, p, tw, b + 4, b1, kmin, kmax, kvh, lane);
        attend<D, RT>(st, z, (b + 2) << 5, c, g4, see_upto, see_from);
      }
    }
  }

  if constexpr (GROUPED) {
    // Rows padded by four floats: the 16 rows a store instruction touches then start on
    // different banks.
    constexpr int PITCH = D + 4;
    __shared__ float part[ATTN_WAVES][16][PITCH];
    __shared__ float part_m[ATTN_WAVES][16], part_l[ATTN_WAVES][16];
    float l = st.lsum[0];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt)
      *(float4*)&part[wave][r][dt * 16 + g4 * 4] = make_float4(
          st.acc[0][dt][0], st.acc[0][dt][1], st.acc[0][dt][2], st.acc[0][dt][3]);
    if (g4 == 0) {
      part_m[wave][r] = st.m[0];
      part_l[wave][r] = l;
    }
    __syncthreads();
    // Each thread adds the four parts of four dims of a row, in the parts' order.
    constexpr int CHUNKS = D / 4;
    for (int e = threadIdx.x; e < 16 * CHUNKS; e += 64 * ATTN_WAVES) {
      const int row = e / CHUNKS, dim = (e % CHUNKS) * 4;
      const int flat = row0 + row;
      if (flat >= rows_total) continue;
      float mx = -INFINITY;
#pragma unroll
      for (int w = 0; w < ATTN_WAVES; ++w) mx = fmaxf(mx, part_m[w][row]);
      float total = 0.f;
      float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int w = 0; w < ATTN_WAVES; ++w) {
        const float mw = part_m[w][row];
        const float wt = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - mx);
        total += part_l[w][row] * wt;
        const float4 v = *(const float4*)&part[w][row][dim];
        o.x += v.x * wt;
        o.y += v.y * wt;
        o.z += v.z * wt;
        o.w += v.w * wt;
      }
      if (p.num_splits == 1) {
        const float inv = total > 0.f ? 1.f / total : 0.f;
        bf16_t* dst = p.out + (size_t)(q0 + flat / G) * p.out_stride + (kvh * G + flat % G) * D + dim;
        *(uint2*)dst = make_uint2(pack_bf16x2(o.x * inv, o.y * inv), pack_bf16x2(o.z * inv, o.w * inv));
      } else {
        const size_t slot = (((size_t)tile * p.n_kv + kvh) * p.num_splits + blockIdx.z) * 16 + row;
        *(float4*)(p.part_o + slot * D + dim) = o;
        if (dim == 0) {
          p.part_ml[slot * 2] = mx;
          p.part_ml[slot * 2 + 1] = total;
        }
      }
    }
    return;
  }

#pragma unroll
  for (int t = 0; t < RT; ++t) {
    float l = st.lsum[t];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    // acc[t][dt][i] is O^T[dim = dt*16 + g4*4 + i][row r of tile t].
    if (p.num_splits == 1) {
      if (!st.row_ok[t]) continue;
      const float inv = 1.f / l;
      bf16_t* dst = p.out + (size_t)(q0 + tok[t]) * p.out_stride + head[t] * D + g4 * 4;
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt) {
        ushort4 o;
        o.x = f32_to_bf16(st.acc[t][dt][0] * inv);
        o.y = f32_to_bf16(st.acc[t][dt][1] * inv);
        o.z = f32_to_bf16(st.acc[t][dt][2] * inv);
        o.w = f32_to_bf16(st.acc[t][dt][3] * inv);
        *(ushort4*)(dst + dt * 16) = o;
      }
    } else {
      const size_t slot =
          (((size_t)tile * p.n_kv + kvh) * p.num_splits + split) * (16 * RT) + t * 16 + r;
      // An empty split writes its zeros too, so that the merge never reads stale memory.
      float* po = p.part_o + slot * D + g4 * 4;
#pragma unroll
      for (int dt = 0; dt < D / 16; ++dt)
        *(float4*)(po + dt * 16) = make_float4(st.acc[t][dt][0], st.acc[t][dt][1],
                                               st.acc[t][dt][2], st.acc[t][dt][3]);
      if (g4 == 0) {
        p.part_ml[slot * 2] = st.m[t];
        p.part_ml[slot * 2 + 1] = l;
      }
    }
  }
}

// ---------------------------------------------------------------------- prompts through LDS
//
// With many rows per sequence (prompt portions), the four wavefronts of a workgroup take four
// consecutive stretches of 16 * RT rows of one sequence and one kv head and walk the same
// blocks of keys together: every block is fetched from the cache once per workgroup, each
// thread bringing 16 or 32 bytes of the keys and as much of the values, parked in registers
// for two iterations and then placed in one of two LDS buffers, from which every wavefront
// reads its operands.  Loads are so two blocks ahead of their use at a quarter of the
// registers a wavefront fetching for itself would need (deeper did not pay: the loop is bound
// by the instructions it issues, not by the loads), and the cache is read once, not four
// times.
//
// LDS layout of a block (32 keys): keys [32][D] and values [D][32], the 16-byte chunks of
// each row permuted so that the rows one operand read touches fall on different banks:
//   keys    with r the operand row that key k is (staged_key_row):
//           D = 64: rows of 128 bytes, chunk c of key k at c ^ ((r >> 1) & 7)
//           D a multiple of 128: chunk c of key k at (c & ~15) | ((c ^ r) & 15)
//           else: at (c & ~7) | ((c ^ r) & 7)
//   values  rows of 64 bytes (32 keys), 16-byte slot s of dim j at s ^ ((j >> 1) & 3)

// The row of a product's operand that key `key` of the block is (see PERM above).
__device__ __forceinline__ int staged_key_row(int key) { return ((key >> 3) << 2) | (key & 3); }

template <int D>
__device__ __forceinline__ int staged_key_offset(int key, int chunk) {  // in 16-byte units
  const int row = staged_key_row(key);
  if (D == 64) return key * 8 + ((chunk ^ (row >> 1)) & 7);
  if (D % 128 == 0) return key * (D / 8) + ((chunk & ~15) | ((chunk ^ row) & 15));
  return key * (D / 8) + ((chunk & ~7) | ((chunk ^ row) & 7));
}

__device__ __forceinline__ int staged_value_offset(int dim, int slot) {  // in 16-byte units
  return dim * 4 + ((slot ^ (dim >> 1)) & 3);
}

// What one thread carries of a block between its global loads and its LDS stores.
template <int D>
struct StagedRegs {
  uint4 k[D / 64], v[D / 64];
};

// Thread-slot u = tid + 256 i of a block's 4 D slots: half u / (2 D) of the block (16 keys,
// one page or a part of one), and 16 bytes t = u % (2 D) of that half's keys (a run of
// 32 D bytes in the cache) and of its values (dim t / 2, keys (t & 1) * 8 .. + 8).  All of a
// wavefront's slots of one i lie in one half, so a half's page is looked up once for the
// wavefront and each load is that page's address plus what the thread adds to it.
template <int D>
__device__ __forceinline__ StagedRegs<D> staged_fetch(const AttnParams& p, TableWindow& tw, int b,
                                                      int b_end, int kmin, int kmax, int kvh,
                                                      int lane) {
  StagedRegs<D> regs;
  const int ps = 1 << p.page_shift;
  const int tid = threadIdx.x & 255;   // within the four wavefronts that share the block
  // A page's address is one 64-bit product added to the cache's (a cache may hold more than
  // 4 GB); everything within the page, the head's and the thread's share, fits 32 bits.
  const uint32_t head_bytes = (uint32_t)ps * D * 2;
  const uint32_t page_bytes = head_bytes * (uint32_t)p.n_kv;
  const uint32_t head_at = (uint32_t)kvh * head_bytes;
#pragma unroll
  for (int i = 0; i < D / 64; ++i) {
    const int u = tid + i * 256, t = u % (2 * D);
    const int h = __builtin_amdgcn_readfirstlane(u / (2 * D));
    const int kh = (b << 5) + h * 16;
    const bool live = b < b_end && kh <= kmax && kh + 15 >= kmin;   // uniform
    const int page = live ? tw.page(kh >> p.page_shift, lane) : 0;
    const uint32_t off = kh & (ps - 1);
    const uint64_t page_at = (uint64_t)(uint32_t)page * page_bytes;
    const uint32_t k_at = head_at + off * (uint32_t)(D * 2) + (uint32_t)t * 16u;
    const uint32_t v_at = head_at + off * 2u + (uint32_t)((t >> 1) * ps * 2 + (t & 1) * 16);
    regs.k[i] = *(const uint4*)((const char*)p.k_cache + page_at + k_at);
    regs.v[i] = *(const uint4*)((const char*)p.v_cache + page_at + v_at);
  }
  return regs;
}

template <int D>
__device__ __forceinline__ void staged_store(const StagedRegs<D>& regs, uint4* lds_k, uint4* lds_v) {
  const int tid = threadIdx.x & 255;
#pragma unroll
  for (int i = 0; i < D / 64; ++i) {
    const int u = tid + i * 256, t = u % (2 * D), h = u / (2 * D);
    lds_k[staged_key_offset<D>(h * 16 + t / (D / 8), t % (D / 8))] = regs.k[i];
    lds_v[staged_value_offset(t >> 1, h * 2 + (t & 1))] = regs.v[i];
  }
}

// The block's operands of this lane, out of LDS, in the order PERM describes.
template <int D>
__device__ __forceinline__ void staged_operands(KeyBlock<D>& blk, const uint4* lds_k,
                                                const uint4* lds_v, int lane) {
  const int r = lane & 15, g4 = lane >> 4;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    blk.live[h] = true;   // keys outside what a row sees are masked one by one
    const int key = ((r >> 2) << 3) + h * 4 + (r & 3);
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
      blk.kf[h][c].u = lds_k[staged_key_offset<D>(key, c * 4 + g4)];
  }
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt)
    blk.vf[dt].u = lds_v[staged_value_offset(dt * 16 + r, g4)];
}

// KG groups of four wavefronts share a workgroup's 64 * RT rows: group g takes the key blocks
// b0 + g, b0 + g + KG, ... with LDS buffers of its own, and at the end the groups' running
// maxima, sums and weighted values are combined through LDS in group order.  A long prompt's
// last rows see thousands of keys; the groups cut that chain of dependent blocks into KG
// shorter ones that run side by side on the same compute unit.
template <int D, int RT, int KG>
__global__ __launch_bounds__(64 * ATTN_WAVES * KG, (RT == 1 ? (KG > 2 ? KG : 2) : 1)) void attn_staged_kernel(AttnParams p) {
  static_assert(D % 64 == 0, "256 threads bring whole 16-byte chunks of 32 keys");
  constexpr int BLOCK = 32 * D / 8;                       // 16-byte units of a block's keys (or values)
  constexpr int MERGE = RT * (D / 4 + 2);                 // floats a thread hands over
  static_assert(KG == 1 || (KG - 1) * MERGE * 4 <= KG * 4 * BLOCK * 4, "merge space fits the buffers");
  __shared__ uint4 lds[KG * 4 * BLOCK];                   // per group: keys[2], values[2]
  const int lane = threadIdx.x & 63;
  const int kgroup = (threadIdx.x >> 6) / ATTN_WAVES, wave = (threadIdx.x >> 6) % ATTN_WAVES;
  uint4* const lds_k = lds + kgroup * 4 * BLOCK;
  uint4* const lds_v = lds_k + 2 * BLOCK;
  const int tile = p.num_tiles - 1 - (int)blockIdx.x;   // the longest work first
  const int kvh = blockIdx.y;
  const int seq = p.tile_seq[tile];
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int pos0 = p.kv_len[seq] - q_len;
  const int G = p.group;
  const int rows_total = q_len * G;
  const int r = lane & 15, g4 = lane >> 4;
  constexpr int WAVE_ROWS = 16 * RT;
  const int wg_row0 = p.tile_row0[tile];
  const int row0 = wg_row0 + wave * WAVE_ROWS;          // this wavefront's rows
  const bool wave_has_rows = row0 < rows_total;

  TileState<D, RT> st;
  int tok[RT], head[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int flat = row0 + t * 16 + r;
    st.row_ok[t] = flat < rows_total;
    tok[t] = st.row_ok[t] ? flat / G : 0;
    head[t] = kvh * G + (st.row_ok[t] ? flat % G : 0);
    st.pos[t] = pos0 + tok[t];
    st.lo[t] = p.window > 0 ? max(0, st.pos[t] - p.window + 1) : 0;
    st.m[t] = -INFINITY;
    st.lsum[t] = 0.f;
    const bf16_t* qrow = p.q + (size_t)(q0 + tok[t]) * p.q_stride + head[t] * D + g4 * 8;
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
      st.qf[t][c].u = st.row_ok[t] ? *(const uint4*)(qrow + c * 32) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) st.acc[t][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  // Keys the workgroup's rows can see, and this wavefront's own share of them.
  const int wg_last = min(wg_row0 + ATTN_WAVES * WAVE_ROWS - 1, rows_total - 1);
  const int wg_kmax = pos0 + wg_last / G;
  const int wg_kmin = p.window > 0 ? max(0, pos0 + wg_row0 / G - p.window + 1) : 0;
  const int b0 = wg_kmin >> 5, b1 = (wg_kmax >> 5) + 1;
  const int last_flat = min(row0 + WAVE_ROWS - 1, rows_total - 1);
  // What steers the loop is the same in every lane of a wavefront, and is said to be so (a
  // wavefront's index comes out of threadIdx and counts as different from lane to lane):
  // the tests on it are then scalar compares and branches, and a block's pages and addresses
  // are worked out once for the wavefront, not in every lane.
  auto uniform = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  const int kmax = uniform(wave_has_rows ? pos0 + last_flat / G : -1);
  const int kmin = uniform(p.window > 0 ? max(0, pos0 + row0 / G - p.window + 1) : 0);
  const int see_upto = uniform(pos0 + row0 / G);
  const int see_from = p.window > 0 ? max(0, kmax - p.window + 1) : 0;
  const float c = p.scale * 1.44269504088896340736f;

  TableWindow tw = {p.block_table + (size_t)seq * p.table_stride, p.table_stride, -64, 0};
  const int first = b0 + uniform(kgroup);                        // this group's blocks: first, first + KG, ...
  StagedRegs<D> ra = staged_fetch<D>(p, tw, first, b1, wg_kmin, wg_kmax, kvh, lane);
  StagedRegs<D> rb = staged_fetch<D>(p, tw, first + KG, b1, wg_kmin, wg_kmax, kvh, lane);
  KeyBlock<D> blk;
  // One block: park what was fetched two iterations ago in LDS, ask for the block two ahead,
  // and, once every wavefront's share is in place, use the block.  Blocks past this
  // wavefront's last key or before its first are the others' business; blocks past the
  // workgroup's last (a group may have one fewer than another) fetch a page that exists and
  // are not used.
#define STAGED_ITERATION(regs, b, buf)                                                  \
  do {                                                                                  \
    staged_store<D>(regs, lds_k + (buf) * BLOCK, lds_v + (buf) * BLOCK);                \
    regs = staged_fetch<D>(p, tw, (b) + 2 * KG, b1, wg_kmin, wg_kmax, kvh, lane);       \
    __syncthreads();                                                                    \
    if (((b) << 5) <= kmax && ((b) << 5) + 31 >= kmin) {                                \
      staged_operands<D>(blk, lds_k + (buf) * BLOCK, lds_v + (buf) * BLOCK, lane);      \
      attend<D, RT, true>(st, blk, (b) << 5, c, g4, see_upto, see_from);                \
    }                                                                                   \
  } while (0)
  const int iterations = (b1 - b0 + KG - 1) / KG;       // the same for every group
  for (int i = 0; i < iterations; i += 2) {
    const int b = first + i * KG;
    STAGED_ITERATION(ra, b, 0);
    if (i + 1 < iterations) STAGED_ITERATION(rb, b + KG, 1);
  }
#undef STAGED_ITERATION

  if constexpr (KG > 1) {
    // Groups 1.. hand their state to group 0, element by element: the same lane of the same
    // wavefront-in-group holds the same rows and dims in every group.
    __syncthreads();                                    // the key and value buffers are free now
    float* const merge = (float*)lds;
    const int slot = threadIdx.x & 255;
    if (kgroup > 0) {
      float* mine = merge + (size_t)(kgroup - 1) * MERGE * 256 + slot;
      int e = 0;
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        mine[256 * e++] = st.m[t];
        mine[256 * e++] = st.lsum[t];
#pragma unroll
        for (int dt = 0; dt < D / 16; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) mine[256 * e++] = st.acc[t][dt][i];
      }
    }
    __syncthreads();
    if (kgroup > 0) return;
#pragma unroll
    for (int g = 1; g < KG; ++g) {
      const float* theirs = merge + (size_t)(g - 1) * MERGE * 256 + slot;
      int e = 0;
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const float m_g = theirs[256 * e++], l_g = theirs[256 * e++];
        const float m_new = fmaxf(st.m[t], m_g);
        const float c_own = m_new == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(st.m[t] - m_new);
        const float c_g = m_new == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_g - m_new);
        st.m[t] = m_new;
        st.lsum[t] = st.lsum[t] * c_own + l_g * c_g;
#pragma unroll
        for (int dt = 0; dt < D / 16; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            st.acc[t][dt][i] = st.acc[t][dt][i] * c_own + theirs[256 * e++] * c_g;
      }
    }
  }

#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (!st.row_ok[t]) continue;
    float l = st.lsum[t];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const float inv = 1.f / l;
    bf16_t* dst = p.out + (size_t)(q0 + tok[t]) * p.out_stride + head[t] * D + g4 * 4;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt)
      *(uint2*)(dst + dt * 16) =
          make_uint2(pack_bf16x2(st.acc[t][dt][0] * inv, st.acc[t][dt][1] * inv),
                     pack_bf16x2(st.acc[t][dt][2] * inv, st.acc[t][dt][3] * inv));
  }
}

// ------------------------------------------------------- prompts in tiles of 32 rows by 64 keys
//
// The same work as the kernel above with the products v_mfma_f32_32x32x16_bf16: a wavefront
// owns 32 rows, four wavefronts 128 consecutive rows of one sequence and one kv head, and a
// block is 64 keys.  With a query per lane (lane l: row l % 32; the two halves of the
// wavefront hold different keys of it) the maximum and the sum over a block's keys are
// sixteen values deep in a lane's own registers per sub-block of 32 keys, one exchange
// between the halves apart; per score there is the least left to do beside the products: one
// maximum, one fused multiply-add, one exponential, one addition, half a conversion.
//
//   S^T[key, row]  = K[key, :] . Q[row, :]     A = K (32 keys x 16 dims), B = Q^T (16 x 32 rows)
//   O^T[dim, row] += V^T[dim, key] P^T[key, row]   A = V^T (32 dims x 16 keys), B = P^T
//
// A lane's sixteen scores of a sub-block are keys 8 (i / 4) + 4 (l / 32) + i % 4; the second
// product's step s takes its registers 8 s .. 8 s + 7, which are keys 16 s + 4 (l / 32) +
// {0..3, 8..11}: the lane's operand of values is two 8-byte pieces of a dim's row of keys.
//
// Keys and values travel from the cache straight into LDS (global_load_lds_dwordx4: a
// wavefront's 64 x 16 bytes land side by side, no register in between), into a ring of
// buffers filled several blocks ahead of their use; a workgroup whose rows see few blocks has
// them all in flight at once, one whose rows see many never waits for the cache's latency.
// Per buffer: keys [64][D], the 16-byte chunks of a key's row permuted by the key's number
// against bank conflicts (by permuting which chunk each lane fetches); values [8 pieces of 8
// keys][D dims][8 keys], which the operand reads cover without conflicts as they lie.
//
// KG groups of four wavefronts may share a workgroup's rows, taking the key blocks in turn
// with rings of their own; their running maxima, sums and weighted values are combined
// through LDS in group order at the end (a short prompt's longest chain of blocks is cut
// into KG chains side by side).
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

// Where chunk `chunk` (16 bytes) of key `key` lies in a buffer, in 16-byte units: sixteen
// consecutive keys' rows of one chunk, which sixteen lanes read together, fall on all 64
// banks (rows of 128 bytes alternate between the banks' halves, so the key's bit 0 picks the
// half and bits 1-3 permute the chunk; rows of 256 bytes cover the banks, so bits 0-3 do).
template <int D>
__device__ __forceinline__ int wide_chunk_swizzle(int key, int chunk) {
  return D == 64 ? ((chunk ^ (key >> 1)) & 7) : ((chunk ^ key) & 15);
}

template <int D>
__device__ __forceinline__ int wide_key_offset(int key, int chunk) {   // in 16-byte units
  constexpr int CH = D / 8;
  return key * CH + wide_chunk_swizzle<D>(key, chunk);
}

// The loads of one block by one wavefront (D / 16 instructions), into the ring buffer at
// LDS byte address `dst`.  Instruction j < D / 32 brings keys: 1024 bytes are 1024 / (2 D)
// keys' rows; instruction j >= D / 32 brings values: 64 dims of one piece of 8 keys.  Keys
// outside what the workgroup's rows see (or past the group's last block) are fetched from
// page 0, which always exists, and masked in the scores.
// What a lane adds to the wavefront's address of a load, the same for every block.
struct WideLane {
  uint32_t k_at, v_at;   // bytes
};

template <int D>
__device__ __forceinline__ WideLane wide_lane(int page_size, int lane, int load) {
  constexpr int KEYS_PER_LOAD = 512 / D, CH = D / 8;
  const int key = load * KEYS_PER_LOAD + lane / CH;      // only key % 16 and load % (D / 64) count
  const int slot = lane % CH;
  const int chunk = wide_chunk_swizzle<D>(key, slot);    // the chunk that lies at the lane's slot
  const int dim = ((load % (D / 64)) * 64 + lane) % D;
  WideLane out;
  out.k_at = (uint32_t)(key & 15) * (uint32_t)(D * 2) + (uint32_t)chunk * 16u;
  out.v_at = (uint32_t)dim * (uint32_t)(page_size * 2);
  return out;
}

// The loads of one block by one of the GW wavefronts that share it, D / (8 GW) of keys and as
// many of values, into the ring buffer at LDS byte address `dst`.  Load number n of the keys
// brings 1024 bytes of rows (8 keys at D = 64, 4 at D = 128), load n of the values 64 dims of
// one piece of 8 keys; both lie in the same stretch of 16 keys of the block, so the page is
// looked up once for the pair, everything but the lane's own offset is the wavefront's
// (scalar) arithmetic, and the load takes that base and a 32-bit offset.  The wavefront's
// loads are numbers wave, wave + GW, ...: a lane's offset is the same for all of them where
// GW loads are a whole number of 16-key stretches, and alternates between two otherwise
// (`mine[j % 2]`).  Keys outside what the workgroup's rows see (or past the group's last
// block) are fetched from page 0, which always exists, and masked in the scores.
template <int D, int GW>
__device__ __forceinline__ void wide_fetch(const AttnParams& p, TableWindow& tw, int b, int b_end,
                                           int kmin, int kmax, int kvh, int lane, int wave,
                                           unsigned int dst, const WideLane (&mine)[2]) {
  constexpr int KEYS_PER_LOAD = 512 / D;
  const int ps = 1 << p.page_shift;
  const uint32_t head_bytes = (uint32_t)ps * D * 2;
  const uint32_t page_bytes = head_bytes * (uint32_t)p.n_kv;
  const uint32_t head_at = (uint32_t)kvh * head_bytes;
  auto uniform = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
#pragma unroll
  for (int j = 0; j < D / (8 * GW); ++j) {
    const int load = wave + GW * j;
    const WideLane& at = mine[(GW * KEYS_PER_LOAD) % 16 == 0 ? 0 : j % 2];
    const int stretch = (load * KEYS_PER_LOAD) >> 4;       // 16 keys, within one page
    const int piece = load / (D / 64);                      // the values' piece of 8 keys
    const int kh = uniform((b << 6) + stretch * 16);
    const int live = uniform(b < b_end && kh <= kmax && kh + 15 >= kmin);
    const int index = kh >> p.page_shift;
    if (live && uniform(index >= tw.base + 64)) {           // once in 64 pages
      tw.base = index;
      tw.mine = index + lane < tw.width ? tw.table[index + lane] : 0;
      __builtin_amdgcn_s_waitcnt(0x0F70);                    // vmcnt(0): before the readlane below
    }
    const int page = live ? __builtin_amdgcn_readlane(tw.mine, uniform(index - tw.base)) : 0;
    const uint64_t page_at = (uint64_t)(uint32_t)page * page_bytes + head_at;
    const uint32_t off = (uint32_t)(kh & (ps - 1));
    const char* k_from = (const char*)p.k_cache + page_at + off * (uint32_t)(D * 2);
    const char* v_from = (const char*)p.v_cache + page_at + (off + (uint32_t)(piece & 1) * 8u) * 2u;
    const unsigned int k_to = dst + (unsigned int)load * 1024u;
    const unsigned int v_to = dst + (unsigned int)(64 * D * 2) + (unsigned int)load * 1024u;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 : : "s"(k_to), "v"(at.k_at), "s"(k_from) : "memory", "m0");
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 : : "s"(v_to), "v"(at.v_at), "s"(v_from) : "memory", "m0");
  }
}

#define WIDE_SLACK 8.f

// NSUB sub-blocks of 32 keys (from `sub0` of the block in LDS) against a wavefront's 32
// rows: scores, one round of the online softmax over all of them, weighted values.
template <int D, int NSUB, bool MASKED>
__device__ __forceinline__ void wide_block(const Frag (&qf)[D / 16], f32x16 (&acc)[D / 32], float& m,
                                           f32x4 (&rowsum)[2], const Frag (&ones)[2],
                                           const uint4* lds_k, const uint2* lds_v,
                                           int key0, int sub0, float c, int n, int hh, bool row_ok,
                                           int pos, int lo) {
  // All of the keys' operands are asked for before the first product, and the values'
  // before the softmax, whose arithmetic then hides their way out of LDS.
  Frag kf[NSUB][D / 16];
#pragma unroll
  for (int u = 0; u < NSUB; ++u)
#pragma unroll
    for (int k = 0; k < D / 16; ++k)
      kf[u][k].u = lds_k[wide_key_offset<D>((sub0 + u) * 32 + n, k * 2 + hh)];
  f32x16 sc[NSUB];
#pragma unroll
  for (int u = 0; u < NSUB; ++u) {
#pragma unroll
    for (int i = 0; i < 16; ++i) sc[u][i] = 0.f;
#pragma unroll
    for (int k = 0; k < D / 16; ++k)
      sc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[u][k].v, qf[k].v, sc[u], 0, 0, 0);
  }
  // values [piece][dim][8 keys]: the lane's two pieces of four keys for step s of sub-block u
  // are bytes 8 hh .. + 8 of pieces 4 u + 2 s and 4 u + 2 s + 1 of its dim.
  Frag vf[D / 32][NSUB][2];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int u = 0; u < NSUB; ++u)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const int piece = (sub0 + u) * 4 + s2 * 2;
        vf[db][u][s2].u2[0] = lds_v[((piece * D) + db * 32 + n) * 2 + hh];
        vf[db][u][s2].u2[1] = lds_v[(((piece + 1) * D) + db * 32 + n) * 2 + hh];
      }
  if (MASKED) {
#pragma unroll
    for (int u = 0; u < NSUB; ++u)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = key0 + (sub0 + u) * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
        const bool ok = row_ok && key <= pos && key >= lo;
        sc[u][i] = ok ? sc[u][i] : -INFINITY;
      }
  }
  float bm = sc[0][0];
#pragma unroll
  for (int u = 0; u < NSUB; ++u)
#pragma unroll
    for (int i = (u == 0 ? 1 : 0); i < 16; ++i) bm = fmaxf(bm, sc[u][i]);
  bm *= c;     // the largest raw score is the largest scaled one (c > 0)
  // The row's reference maximum moves, and what is accumulated is rescaled, only when some
  // lane of the wavefront saw a score more than WIDE_SLACK (in powers of two) above its
  // row's: until then the exponentials may reach 2^WIDE_SLACK instead of 1, which float32
  // sums and bfloat16 weights hold as well, and the result is a quotient in which the
  // reference cancels.  The two lanes of a row exchange their maxima first, so that both
  // always hold the same reference.
  if (__builtin_expect(__builtin_amdgcn_ballot_w64(bm > m + WIDE_SLACK) != 0, 0)) {
    bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
    const float m_new = fmaxf(m, bm);
    const float corr = __builtin_amdgcn_exp2f(m - (m_new == -INFINITY ? 0.f : m_new));
    m = m_new;
    rowsum[0] *= corr;
    rowsum[1] *= corr;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[db][i] *= corr;
  }
  const float m_use = (MASKED && m == -INFINITY) ? 0.f : m;
  Frag pf[NSUB][2];
#pragma unroll
  for (int u = 0; u < NSUB; ++u) {
    float e[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) e[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[u][i], c, -m_use));
#pragma unroll
    for (int s = 0; s < 2; ++s)
      pf[u][s].u = make_uint4(pack_bf16x2(e[8 * s], e[8 * s + 1]), pack_bf16x2(e[8 * s + 2], e[8 * s + 3]),
                              pack_bf16x2(e[8 * s + 4], e[8 * s + 5]), pack_bf16x2(e[8 * s + 6], e[8 * s + 7]));
  }
  // The rows' sums of weights come out of the matrix cores as well, which have time to
  // spare while the vector unit does not: the weights against ones.  As the operand of a
  // 16 x 16 x 32 product a lane's eight weights are column lane % 16, keys' group lane / 16:
  // groups 0 and 2 are the two halves of row lane % 16, groups 1 and 3 those of row
  // 16 + lane % 16, and ones in the matching groups (`ones[0]`, `ones[1]`) pick each.
#pragma unroll
  for (int u = 0; u < NSUB; ++u)
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      rowsum[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones[0].v, pf[u][s].v, rowsum[0], 0, 0, 0);
      rowsum[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones[1].v, pf[u][s].v, rowsum[1], 0, 0, 0);
    }
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int u = 0; u < NSUB; ++u)
#pragma unroll
      for (int s = 0; s < 2; ++s)
        acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][u][s].v, pf[u][s].v, acc[db], 0, 0, 0);
}

// s_waitcnt immediate: at most `loads` vector-memory loads outstanding (vmcnt is split over
// bits 3:0 and 15:14; the other counters are left alone).
#define WIDE_WAIT(loads) (((loads) & 15) | (((loads) >> 4) << 14) | (7 << 4) | (15 << 8))

// GW wavefronts of 32 rows each make a key group, a tile of 32 GW rows: four, or two where
// tiles of 128 rows would be fewer than fill the chip.
template <int D, int KG, int NB, int GW = 4>
__global__ __launch_bounds__(64 * GW * KG, KG > 1 ? 1 : (NB * D <= 192 ? 3 : (NB * D <= 256 ? 2 : 1))) void attn_wide_kernel(AttnParams p) {
  constexpr int BUFFER = 2 * 64 * D * 2;                   // bytes of a block's keys and values
  constexpr int LOADS = D / (4 * GW);                      // load instructions per wavefront and block
  constexpr int MERGE = D / 2 + 2;                         // floats a thread hands over
  constexpr int GROUP_THREADS = 64 * GW, ROWS = 32 * GW;
  static_assert(GW == 2 || GW == 4, "two or four wavefronts a key group");
  static_assert(KG == 1 || (KG - 1) * MERGE * GROUP_THREADS * 4 <= KG * NB * BUFFER, "merge space fits the rings");
  static_assert((NB - 1) * LOADS < 64, "the loads in flight fit the counter");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[KG * NB * BUFFER];
  const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) % GW;
  const int kgroup = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / GROUP_THREADS));
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  unsigned char* const ring = lds + kgroup * (NB * BUFFER);
  const unsigned int ring_at = (unsigned int)(uintptr_t)(__attribute__((address_space(3))) void*)ring;
  const int n = lane & 31, hh = lane >> 5;
  const int G = p.group;
  const WideLane mine[2] = {wide_lane<D>(1 << p.page_shift, lane, wave_u),
                            wide_lane<D>(1 << p.page_shift, lane, wave_u + GW)};
  Frag ones[2];
  {
    const uint32_t pair = 0x3F803F80u;                    // two bfloat16 ones
    const uint32_t even = (lane & 16) ? 0u : pair, odd = (lane & 16) ? pair : 0u;
    ones[0].u = make_uint4(even, even, even, even);
    ones[1].u = make_uint4(odd, odd, odd, odd);
  }
  auto uniform = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  const float c = p.scale * 1.44269504088896340736f;

  // The order of work.  Workgroups are handed out in the order of their index, to the compute
  // units in turn, and stay until their chain of key blocks is done; the length of a chain
  // grows with the tile's number within its sequence.  So the index counts the (tile, kv
  // head) pairs from the longest down, kv heads side by side, and of the stretches of 256
  // that are resident from the start (as many as a unit holds workgroups) every second one
  // runs backwards: the unit that took the longest of one stretch takes the shortest of the
  // next, and what is resident on a unit adds up to about the same everywhere (8,192 tokens
  // of 14 heads of 64: 211 us against 227; 16,384: 641 against 683; 28 heads of 128: 610
  // against 634).  What follows the residents goes to whichever unit is free first, the
  // longest first.
  constexpr int RESIDENT = KG > 1 ? (GW == 2 && KG == 2 ? 2 : 1) : (NB * D <= 192 ? 3 : (NB * D <= 256 ? 2 : 1));
  int tile, kvh_x;
  {
    const int total = gridDim.x * gridDim.y, id = blockIdx.y * gridDim.x + blockIdx.x;
    const int stretch = id / 256, size = min(256, total - stretch * 256), at = id - stretch * 256;
    const bool backwards = (stretch & 1) && stretch < RESIDENT;
    const int rank = stretch * 256 + (backwards ? size - 1 - at : at);
    kvh_x = rank % (int)gridDim.y;
    tile = p.num_tiles - 1 - rank / (int)gridDim.y;
  }
  const int kvh = kvh_x;
  const int seq = p.tile_seq[tile];
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int pos0 = p.kv_len[seq] - q_len;
  const int rows_total = q_len * G;
  const int wg_row0 = p.tile_row0[tile];
  const int row0 = wg_row0 + wave * 32;
  const bool wave_has_rows = row0 < rows_total;

  const int flat = row0 + n;
  const bool row_ok = flat < rows_total;
  const int tok = row_ok ? flat / G : 0;
  const int head = kvh * G + (row_ok ? flat % G : 0);
  const int pos = pos0 + tok;
  const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;

  const int wg_last = min(wg_row0 + ROWS - 1, rows_total - 1);
  const int wg_kmax = pos0 + wg_last / G;
  const int wg_kmin = p.window > 0 ? max(0, pos0 + wg_row0 / G - p.window + 1) : 0;
  const int b0 = wg_kmin >> 6, b1 = (wg_kmax >> 6) + 1;
  const int first = __builtin_amdgcn_readfirstlane(b0 + kgroup);   // this group's blocks: first, first + KG, ...
  const int iterations = __builtin_amdgcn_readfirstlane((b1 - b0 + KG - 1) / KG);   // the same for every group

  // The ring starts to fill before anything else is asked of memory.
  TableWindow tw = {p.block_table + (size_t)seq * p.table_stride, p.table_stride, -64, 0};
#pragma unroll
  for (int i = 0; i < NB - 1; ++i)
    wide_fetch<D, GW>(p, tw, first + i * KG, b1, wg_kmin, wg_kmax, kvh, lane, wave_u,
                      ring_at + (unsigned int)(i * BUFFER), mine);

  Frag qf[D / 16];
  {
    const bf16_t* qrow = p.q + (size_t)(q0 + tok) * p.q_stride + head * D + hh * 8;
#pragma unroll
    for (int k = 0; k < D / 16; ++k)
      qf[k].u = row_ok ? *(const uint4*)(qrow + k * 16) : make_uint4(0, 0, 0, 0);
  }
  f32x16 acc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
  float m = -INFINITY;
  // Sums of weights per row, kept by the matrix cores (see wide_block): rowsum[h][.] on lane l
  // is the sum of row 16 h + l % 16, both halves' keys included.
  f32x4 rowsum[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};

  const int last_flat = min(row0 + 31, rows_total - 1);
  const int kmax = uniform(wave_has_rows ? pos0 + last_flat / G : -1);
  const int kmin = uniform(p.window > 0 ? max(0, pos0 + row0 / G - p.window + 1) : 0);
  const int see_upto = uniform(pos0 + row0 / G);       // every valid row of the wavefront sees up to here
  const int see_from = p.window > 0 ? max(0, kmax - p.window + 1) : 0;
  // the queries were asked for after the ring's first loads: all of them have to be there
  // before the counting below starts
  __builtin_amdgcn_s_waitcnt(WIDE_WAIT(0));

  // One block: block i's loads of this wavefront have landed once at most the NB - 2 later
  // blocks' are outstanding (in the first iteration the queries' loads were waited for
  // above, which covered everything); after the barrier every wavefront's have, and
  // everybody is done with block i - 1, whose buffer the block NB - 1 ahead now takes.
  // Heads of 64: one softmax round over the block's 64 keys; heads of 128 (twice the
  // accumulators): one per 32 keys, or the scores would not fit the registers.
  constexpr int NSUB = D <= 64 ? 2 : 1;
#define WIDE_ITERATION(MASKED)                                                                   \
  do {                                                                                           \
    const int b = first + i * KG;                                                                \
    __builtin_amdgcn_s_waitcnt(WIDE_WAIT((NB - 2) * LOADS));                                     \
    __syncthreads();                                                                             \
    wide_fetch<D, GW>(p, tw, b + (NB - 1) * KG, b1, wg_kmin, wg_kmax, kvh, lane, wave_u,         \
                      ring_at + (unsigned int)(((i + NB - 1) % NB) * BUFFER), mine);             \
    const uint4* lds_k = (const uint4*)(ring + (i % NB) * BUFFER);                               \
    const uint2* lds_v = (const uint2*)(ring + (i % NB) * BUFFER + 64 * D * 2);                  \
    const int key0 = b << 6;                                                                     \
    _Pragma("unroll") for (int sub0 = 0; sub0 < 2; sub0 += NSUB) {                               \
      const int lo_key = key0 + sub0 * 32, hi_key = lo_key + NSUB * 32 - 1;                      \
      if (MASKED && (b >= b1 || lo_key > kmax || hi_key < kmin)) continue;                       \
      wide_block<D, NSUB, MASKED>(qf, acc, m, rowsum, ones, lds_k, lds_v, key0, sub0, c, n, hh,  \
                                  row_ok, pos, lo);                                              \
    }                                                                                            \
  } while (0)
  // The blocks every valid row of the wavefront sees in full, [see_from, see_upto], take a
  // loop of their own in which nothing is tested; the blocks before (a window's edge) and
  // after (the causal edge, the sequence's end, blocks only other wavefronts see) are masked
  // key by key.  Every wavefront meets the same number of barriers, in whichever loop.
  const int full_from = uniform(max(0, ((see_from + 63) >> 6) - first + KG - 1) / KG);
  const int last_full = (see_upto - 63) >> 6;             // the last block seen in full, if any
  const int full_upto = uniform(see_upto >= 63 && last_full >= first
                                    ? min(iterations, (last_full - first) / KG + 1) : 0);
  int i = 0;
  for (; i < min(full_from, iterations); ++i) WIDE_ITERATION(true);
  for (; i < full_upto; ++i) WIDE_ITERATION(false);
  for (; i < iterations; ++i) WIDE_ITERATION(true);
#undef WIDE_ITERATION
  // nothing may still be on its way into LDS when the workgroup's memory is given up or reused
  __builtin_amdgcn_s_waitcnt(WIDE_WAIT(0));

  // this lane's row's sum of weights, both halves' keys included
  float lsum = (lane & 16) ? rowsum[1][0] : rowsum[0][0];
  if constexpr (KG > 1) {
    // Groups 1.. hand their state to group 0, element by element: the same lane of the same
    // wavefront-in-group holds the same rows and dims in every group.
    __syncthreads();                                    // the rings are free now
    float* const merge = (float*)lds;
    const int slot = threadIdx.x % GROUP_THREADS;
    if (kgroup > 0) {
      float* mine_out = merge + (size_t)(kgroup - 1) * MERGE * GROUP_THREADS + slot;
      int e = 0;
      mine_out[GROUP_THREADS * e++] = m;
      mine_out[GROUP_THREADS * e++] = lsum;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) mine_out[GROUP_THREADS * e++] = acc[db][i];
    }
    __syncthreads();
    if (kgroup == 0) {
#pragma unroll
      for (int g = 1; g < KG; ++g) {
        const float* theirs = merge + (size_t)(g - 1) * MERGE * GROUP_THREADS + slot;
        int e = 0;
        const float m_g = theirs[GROUP_THREADS * e++], l_g = theirs[GROUP_THREADS * e++];
        const float m_new = fmaxf(m, m_g);
        const float c_own = m_new == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
        const float c_g = m_new == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_g - m_new);
        m = m_new;
        lsum = lsum * c_own + l_g * c_g;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[db][i] = acc[db][i] * c_own + theirs[GROUP_THREADS * e++] * c_g;
      }
    }
  }

  if (row_ok && kgroup == 0) {
    const float inv = 1.f / lsum;
    // acc[db][i] is O^T[dim = db * 32 + 8 (i / 4) + 4 hh + i % 4][row n].
    bf16_t* dst = p.out + (size_t)(q0 + tok) * p.out_stride + head * D + 4 * hh;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *(uint2*)(dst + db * 32 + 8 * q4) =
            make_uint2(pack_bf16x2(acc[db][4 * q4] * inv, acc[db][4 * q4 + 1] * inv),
                       pack_bf16x2(acc[db][4 * q4 + 2] * inv, acc[db][4 * q4 + 3] * inv));
  }
}

// Merge the key splits of one (tile, kv head, row) per workgroup: the maximum of the running
// maxima, then the sums and the partial results rescaled to it.  Thread (g, dim) adds the
// splits g, g + 4, ... of its dim, four loads in flight at a time; the four groups are then
// added in order, so the result does not depend on timing.
template <int D>
__global__ __launch_bounds__(256) void attn_merge_kernel(AttnParams p) {
  __shared__ float weight[1024];
  __shared__ float group_sum[4][D];
  __shared__ float scratch[16];
  const int tile = blockIdx.x, kvh = blockIdx.y, r = blockIdx.z, R = p.tile_rows;
  // (no tile list: tile t is the one new token of sequence t)
  const int seq = p.direct ? tile : p.tile_seq[tile], row0 = p.direct ? 0 : p.tile_row0[tile];
  const int q0 = p.direct ? seq : p.cu_q[seq], q_len = p.direct ? 1 : p.cu_q[seq + 1] - q0;
  const int G = p.group;
  const int flat = row0 + r;
  if (flat >= q_len * G) return;
  const int S = p.num_splits;
  const size_t base = ((size_t)tile * p.n_kv + kvh) * S;

  float mx = -INFINITY;
  for (int s = threadIdx.x; s < S; s += blockDim.x)
    mx = fmaxf(mx, p.part_ml[((base + s) * R + r) * 2]);
  mx = block_max(mx, scratch);
  float part = 0.f;
  for (int s = threadIdx.x; s < S; s += blockDim.x) {
    const size_t slot = (base + s) * R + r;
    const float ms = p.part_ml[slot * 2];
    const float w = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - mx);  // base-2 maxima
    weight[s] = w;
    part += p.part_ml[slot * 2 + 1] * w;
  }
  const float total = block_sum(part, scratch);  // also orders the writes of weight[]

  const int g = threadIdx.x >> 6;
  for (int dim = threadIdx.x & 63; dim < D; dim += 64) {
    const float* src = p.part_o + ((base * R) + r) * D + dim;
    const size_t stride = (size_t)R * D;
    auto term = [&](int s) { return src[(size_t)s * stride] * weight[s]; };
    float o = 0.f;
    int s = g;
    for (; s + 12 < S; s += 16) {
      const float a = term(s), b = term(s + 4), c = term(s + 8), d = term(s + 12);
      o += (a + b) + (c + d);
    }
    for (; s < S; s += 4) o += term(s);
    group_sum[g][dim] = o;
  }
  __syncthreads();
  const int tok = flat / G, head = kvh * G + flat % G;
  for (int dim = threadIdx.x; dim < D; dim += blockDim.x) {
    const float o = (group_sum[0][dim] + group_sum[1][dim]) + (group_sum[2][dim] + group_sum[3][dim]);
    p.out[(size_t)(q0 + tok) * p.out_stride + head * D + dim] = f32_to_bf16(o / total);
  }
}

// The same merge for a handful of splits, where a workgroup per row would be thousands of
// workgroups with next to nothing to do (64 decoded tokens of 8 key/value heads in 2 splits:
// 8,192 of them, 9 us): one workgroup per (tile, kv head), 16 threads per row with D / 16 dims
// each, the splits added in split order.
template <int D>
__global__ __launch_bounds__(256) void attn_merge_rows_kernel(AttnParams p) {
  constexpr int PER = D / 16;
  const int tile = blockIdx.x, kvh = blockIdx.y, R = p.tile_rows, S = p.num_splits;
  // (no tile list: tile t is the one new token of sequence t)
  const int seq = p.direct ? tile : p.tile_seq[tile], row0 = p.direct ? 0 : p.tile_row0[tile];
  const int q0 = p.direct ? seq : p.cu_q[seq], q_len = p.direct ? 1 : p.cu_q[seq + 1] - q0;
  const int G = p.group;
  const size_t base = ((size_t)tile * p.n_kv + kvh) * S;
  const int sub = threadIdx.x & 15;
  for (int r = threadIdx.x >> 4; r < R; r += 16) {
    const int flat = row0 + r;
    if (flat >= q_len * G) continue;
    float mx = -INFINITY;
    for (int s2 = 0; s2 < S; ++s2) mx = fmaxf(mx, p.part_ml[((base + s2) * R + r) * 2]);
    float total = 0.f, o[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) o[i] = 0.f;
    for (int s2 = 0; s2 < S; ++s2) {
      const size_t slot = (base + s2) * R + r;
      const float ms = p.part_ml[slot * 2];
      const float w = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - mx);  // base-2 maxima
      total += p.part_ml[slot * 2 + 1] * w;
      const float2* src = (const float2*)(p.part_o + slot * D + sub * PER);
#pragma unroll
      for (int i = 0; i < PER / 2; ++i) {
        const float2 v = src[i];
        o[2 * i] += v.x * w;
        o[2 * i + 1] += v.y * w;
      }
    }
    const int tok = flat / G, head = kvh * G + flat % G;
    const float inv = 1.f / total;
    uint32_t* dst = (uint32_t*)(p.out + (size_t)(q0 + tok) * p.out_stride + head * D + sub * PER);
#pragma unroll
    for (int i = 0; i < PER / 2; ++i) dst[i] = pack_bf16x2(o[2 * i] * inv, o[2 * i + 1] * inv);
  }
}

#define ATTN_MERGE_ROWS_MAX_SPLITS 4

template <int D>
static void launch_staged(const AttnParams& p, int rows_per_tile, int key_groups, hipStream_t stream) {
  if constexpr (D == 64 || D == 128) {   // wider heads do not fit the register file
    dim3 grid(p.num_tiles, p.n_kv);
    if (rows_per_tile == 32)
      attn_staged_kernel<D, 2, 1><<<grid, 64 * ATTN_WAVES, 0, stream>>>(p);
    else if (key_groups == 1)
      attn_staged_kernel<D, 1, 1><<<grid, 64 * ATTN_WAVES, 0, stream>>>(p);
    else if (key_groups == 2)
      attn_staged_kernel<D, 1, 2><<<grid, 64 * ATTN_WAVES * 2, 0, stream>>>(p);
    else if constexpr (D == 64)   // 16 wavefronts of a wider head do not fit the register file
      attn_staged_kernel<D, 1, 4><<<grid, 64 * ATTN_WAVES * 4, 0, stream>>>(p);
  }
}

// Ring depths by measurement: 64-wide heads run three workgroups a compute unit with three
// buffers (2,048 x 4 tokens, 14 heads: 73 us against 83 with four buffers and two workgroups);
// 128-wide heads two workgroups with two buffers (8,192 tokens, 28 heads: 752 us against 1256
// with three buffers and one workgroup).  Key groups: as many as keep three (64) or two (128)
// wavefronts a SIMD in one workgroup, for launches of fewer workgroups than fill the chip.
// Tiles of 64 rows (64-wide heads): four key groups with two buffers each (128 KB, eight
// wavefronts, one workgroup a compute unit) or two (64 KB, two workgroups a unit).
template <int D>
static void launch_wide(const AttnParams& p, int staged, hipStream_t stream) {
  const dim3 grid(p.num_tiles, p.n_kv);
  const int chains = staged / 8;
  if constexpr (D == 64) {
    if (staged % 8) {   // tiles of 64 rows, two wavefronts a key group
      if (chains == 4) attn_wide_kernel<D, 4, 2, 2><<<grid, 512, 0, stream>>>(p);
      else attn_wide_kernel<D, 2, 2, 2><<<grid, 256, 0, stream>>>(p);
    } else if (chains == 3) {
      attn_wide_kernel<D, 3, 3><<<grid, 768, 0, stream>>>(p);
    } else {
      attn_wide_kernel<D, 1, 3><<<grid, 256, 0, stream>>>(p);
    }
  } else {
    if (chains == 2) attn_wide_kernel<D, 2, 2><<<grid, 512, 0, stream>>>(p);
    else attn_wide_kernel<D, 1, 2><<<grid, 256, 0, stream>>>(p);
  }
}

// Whether a split of one 16-row tile's keys goes to workgroups of ATTN_WAVES consecutive
// parts each (the GROUPED kernel).
static bool attn_grouped(int rows_per_tile, int num_splits) {
  return rows_per_tile == 16 && num_splits >= ATTN_WAVES && num_splits % ATTN_WAVES == 0;
}

template <int D>
static void launch_merge(const AttnParams& p, hipStream_t stream) {
  if (p.num_splits > 1 && p.num_splits <= ATTN_MERGE_ROWS_MAX_SPLITS) {
    attn_merge_rows_kernel<D><<<dim3(p.num_tiles, p.n_kv), 256, 0, stream>>>(p);
  } else if (p.num_splits > 1) {
    dim3 mgrid(p.num_tiles, p.n_kv, p.tile_rows);
    attn_merge_kernel<D><<<mgrid, 256, 0, stream>>>(p);
  }
}

template <int D>
static void launch_attn(const AttnParams& p, int rows_per_tile, bool merge, hipStream_t stream) {
  if constexpr (D <= 128) {
    if (attn_grouped(rows_per_tile, p.num_splits)) {
      AttnParams g = p;
      g.num_splits = p.num_splits / ATTN_WAVES;
      const dim3 grid(g.num_tiles, g.n_kv, g.num_splits);
      if (g.direct) attn_mfma_kernel<D, 1, ATTN_AHEAD_16, true, true><<<grid, 64 * ATTN_WAVES, 0, stream>>>(g);
      else attn_mfma_kernel<D, 1, ATTN_AHEAD_16, true><<<grid, 64 * ATTN_WAVES, 0, stream>>>(g);
      if (merge) launch_merge<D>(g, stream);
      return;
    }
  }
  const int per = ATTN_WAVES / p.kv_fold;   // tiles per workgroup
  dim3 grid((p.num_tiles + per - 1) / per, p.n_kv / p.kv_fold, p.num_splits);
  const int threads = 64 * ATTN_WAVES;
  if (rows_per_tile == 16) {
    if (p.direct) attn_mfma_kernel<D, 1, ATTN_AHEAD_16, false, true><<<grid, threads, 0, stream>>>(p);
    else attn_mfma_kernel<D, 1, ATTN_AHEAD_16><<<grid, threads, 0, stream>>>(p);
  } else if (rows_per_tile == 32) {
    if constexpr (D <= 128) attn_mfma_kernel<D, 2, ATTN_AHEAD_32><<<grid, threads, 0, stream>>>(p);
  } else {
    // 64 rows: only instantiated where the accumulators fit the register file
    if constexpr (D <= 64) attn_mfma_kernel<D, 4, ATTN_AHEAD_64><<<grid, threads, 0, stream>>>(p);
  }
  if (merge) launch_merge<D>(p, stream);
}

// The most rows (16, 32 or 64) one wavefront can take for this head size.
extern "C" int mk_attention_mfma_max_rows(int head_dim) {
  return head_dim <= 64 ? 64 : (head_dim <= 128 ? 32 : 16);
}

// Into how many groups (1, 2 or 4) the kernel that stages keys and values in LDS (workgroups
// of 4 * rows_per_tile rows of one sequence) can split a workgroup's keys at this head size
// and tile height; 0 if it does not take them at all.
extern "C" int mk_attention_mfma_staged(int head_dim, int rows_per_tile) {
  if (head_dim != 64 && head_dim != 128) return 0;
  return rows_per_tile == 16 ? (head_dim == 64 ? 4 : 2) : (rows_per_tile == 32 ? 1 : 0);
}

// Into how many chains the prompt kernel of 32-row wavefronts and 64-key blocks (`staged` =
// 8 times the number of chains; 32 rows per wavefront, tile list in steps of 128 rows) can cut
// a workgroup's keys at this head size: bit n - 1 is set when n chains exist (64: one or
// three, 128: one or two); 0 if it does not take the size.
extern "C" int mk_attention_mfma_wide(int head_dim) {
  return head_dim == 64 ? 0b101 : (head_dim == 128 ? 0b011 : 0);
}

// The same for its workgroups of 64 rows, two wavefronts a key group (`staged` = 8 times the
// number of chains, plus 4; tile list in steps of 64 rows): 64-wide heads in two or four chains.
extern "C" int mk_attention_mfma_wide_half(int head_dim) { return head_dim == 64 ? 0b1010 : 0; }

// Which instantiation of the kernel of 32-row wavefronts, as its `staged` code (0: none, the
// 16-row kernels are the faster ones), for a step of `wg128` workgroups of 128 rows or
// `wg64` of 64 (key/value heads counted) whose longest sequence is `blocks32` blocks of 32
// keys; `fresh`: most of the longest sequence's keys are this step's own (a prompt from its
// start rather than a portion over a long prefix).  The numbers belong to the instantiations,
// which is why they stand here and not with the planner.  Measured, us, against the best
// of the rest (each line: heads in groups, tokens (over a prefix), then the candidates):
//  64-wide heads (codes 8: one chain of key blocks, 24: three; tiles of 64 rows 36: four, 20: two)
//   14 in 2, 1,024: 16-row 15.7, 8 23.2, 24 19.5, 36 15.2    2,048: 29.5, 39.7, 29.0, 36 28.0
//   14 in 2, 3,072: 16-row 55.9, 8 57.2, 24 39.7, 36 50.9    6,144: 151, 8 117, 24 115
//   14 in 2, 512 over 3,584: 16-row 40.7, 24 48.2, 36 36.4   two of 1,024 over 1,024: 42.5, 8 40.3, 24 30.2, 36 35.8
//   28 in 4, 1,024: 16-row 23.8, 8 23.3, 24 19.8, 20 19.0    1,536: 36.5, 8 32.1, 24 25.9, 20 27.1
//   28 in 4, 2,048: 8 41.0, 24 35.8, 20 40.9    3,072: 8 62.6, 24 68.7    four of 512: 8 17.2, 24 24.4, 20 22.7
//   16 in 8, 1,536: 16-row 32.6, 24 24.1, 36 21.9    4,096: 8 76.0, 24 60.4    four of 512: 8 15.4, 20 14.0
//   32 in 8, 768: 16-row 20.5, 8 19.1, 20 15.8    2,048: 8 42.0, 24 38.7    3,072: 8 65.7, 24 74.8
//  128-wide heads (codes 8: one chain, 16: two)
//   28 in 4, 512: 16-row 15.9, 16 19.8    1,024: 37.5, 8 36.6, 16 30.6    2,048: 8 67.9, 16 58.3    3,072: 8 103, 16 116
//   28 in 4, 1,024 over 3,072: 16-row 137, 8 121, 16 91.7    four of 512: 8 28.0, 16 35.2    two of 1,024 over 1,024: 8 77.8, 16 81.5
//   40 in 8, 768: 16-row 30.2, 8 29.4, 16 25.9    1,536: 8 53.4, 16 49.8    2,048: 8 73.2, 16 84.9
//   16 in 8, 1,024: 16-row 25.3, 16 29.3    2,048: 8 62.8, 16 49.9    4,096: 8 127, 16 105    6,144: 8 207, 16 228
extern "C" int mk_attention_mfma_wide_choice(int head_dim, int wg128, int wg64, int blocks32,
                                             int fresh) {
  if (head_dim == 64) {
    if (wg128 >= 192 && wg128 <= 512 && blocks32 >= 48 && !(fresh && wg64 <= 512)) return 24;
    if (wg128 >= 512 || (wg128 >= 384 && blocks32 < 48)) return 8;
    if (wg64 >= 112 && wg64 <= 256 && blocks32 >= 24) return 36;
    if (wg64 > 256 && wg64 <= 512) return blocks32 >= 48 ? 36 : 20;
    return 0;
  }
  if (head_dim == 128) {
    if ((wg128 >= 160 && wg128 <= 384 && blocks32 >= 16) ||
        (wg128 > 384 && wg128 <= 512 && blocks32 >= 24 && fresh)) {
      return 16;
    }
    return wg128 >= 256 ? 8 : 0;
  }
  return 0;
}

extern "C" int mk_attention_mfma_supported(int head_dim, int page_size) {
  const bool d_ok = head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128 ||
                    head_dim == 192 || head_dim == 256;
  return d_ok && page_size >= 16 && mk_is_pow2(page_size);
}

extern "C" int mk_attention_mfma_check(int q_stride, int out_stride, int num_tiles, int page_size,
                                       int n_q, int n_kv, int d, float scale, int window,
                                       int rows_per_tile, int staged, int num_splits,
                                       int split_blocks, int has_workspace) {
  MK_REQUIRE(num_tiles >= 0 && n_q > 0 && n_kv > 0, "attention: bad sizes");
  MK_REQUIRE(n_q % n_kv == 0, "attention: %d query heads are not a multiple of %d kv heads",
             n_q, n_kv);
  MK_REQUIRE(mk_attention_mfma_supported(d, page_size),
             "attention (matrix cores): head size %d / page size %d not supported; head sizes "
             "32, 64, 96, 128, 192, 256 and pages of 16 or more are",
             d, page_size);
  MK_REQUIRE(num_splits >= 1 && num_splits <= 1024 && n_kv <= 65535, "attention: bad grid");
  MK_REQUIRE(num_splits == 1 || has_workspace, "attention: key splits need a workspace");
  MK_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0,
             "attention: row strides %d/%d break 16-byte alignment", q_stride, out_stride);
  MK_REQUIRE(window >= 0, "attention: negative window");
  MK_REQUIRE(scale > 0.f, "attention: the score scale %g is not positive", (double)scale);
  MK_REQUIRE(rows_per_tile == 16 || rows_per_tile == 32 || rows_per_tile == 64,
             "attention: %d rows per tile", rows_per_tile);
  MK_REQUIRE(rows_per_tile <= mk_attention_mfma_max_rows(d),
             "attention: %d rows per tile are too many for head size %d", rows_per_tile, d);
  MK_REQUIRE(split_blocks >= 0, "attention: negative split size");
  const int wide_chains = staged >= 8 ? staged / 8 : 0;
  MK_REQUIRE(staged == 0 || staged == 1 || staged == 2 || staged == 4 ||
                 (staged >= 8 && wide_chains <= 4 && (staged % 8 == 0 || staged % 8 == 4)),
             "attention: %d key groups (0, 1, 2 or 4; 8 times one to four for the kernel of "
             "32-row wavefronts, plus 4 for its tiles of 64 rows)", staged);
  MK_REQUIRE(staged < 8 || (num_splits == 1 && rows_per_tile == 32 &&
                            (((staged % 8 ? mk_attention_mfma_wide_half(d) : mk_attention_mfma_wide(d)) >>
                              (wide_chains - 1)) & 1)),
             "attention: the kernel of 32-row wavefronts takes unsplit keys, 32 rows per "
             "wavefront and head sizes 64 (one or three key groups, two or four with tiles of "
             "64 rows) and 128 (one or two)");
  MK_REQUIRE(!staged || staged >= 8 ||
                 (num_splits == 1 && staged <= mk_attention_mfma_staged(d, rows_per_tile)),
             "attention: staging in LDS takes unsplit keys, head sizes 64 and 128 and 16 or 32 "
             "rows per wavefront (one key group with 32)");
  return 0;
}

static int attention_mfma(const void* q, int q_stride, void* out, int out_stride,
                          const void* k_cache, const void* v_cache, const int* tile_seq,
                          const int* tile_row0, int num_tiles, const int* cu_q, const int* kv_len,
                          const int* block_table, int table_stride, int page_size, int n_q,
                          int n_kv, int d, float scale, int window, int rows_per_tile, int staged,
                          int num_splits, int split_blocks, float* part_o, float* part_ml,
                          bool merge, hipStream_t stream) {
  if (int code = mk_attention_mfma_check(q_stride, out_stride, num_tiles, page_size, n_q, n_kv, d,
                                         scale, window, rows_per_tile, staged, num_splits,
                                         split_blocks, part_o && part_ml)) {
    return code;
  }
  if (num_tiles == 0) return 0;
  // No tile list: tile t is the one new token of sequence t (see DIRECT).
  const bool direct = tile_seq == nullptr;
  MK_REQUIRE((tile_seq == nullptr) == (tile_row0 == nullptr), "attention: half a tile list");
  MK_REQUIRE(!direct || (rows_per_tile == 16 && staged == 0 && window == 0 && n_q / n_kv <= 16 &&
                         split_blocks == 0),
             "attention: without a tile list every sequence brings one token of at most 16 heads "
             "a group, in tiles of 16 rows, unwindowed (the parts of the keys are then every "
             "num_splits-th block, not stretches of split_blocks)");
  AttnParams p;
  p.q = (const bf16_t*)q;
  p.q_stride = q_stride;
  p.out = (bf16_t*)out;
  p.out_stride = out_stride;
  p.part_o = part_o;
  p.part_ml = part_ml;
  p.k_cache = (const bf16_t*)k_cache;
  p.v_cache = (const bf16_t*)v_cache;
  p.tile_seq = tile_seq;
  p.tile_row0 = tile_row0;
  p.cu_q = cu_q;
  p.kv_len = kv_len;
  p.block_table = block_table;
  p.table_stride = table_stride;
  p.page_shift = mk_log2(page_size);
  p.n_kv = n_kv;
  p.group = n_q / n_kv;
  p.scale = scale;
  p.window = window;
  p.num_tiles = num_tiles;
  p.num_splits = num_splits;
  p.split_blocks = split_blocks;
  p.tile_rows = rows_per_tile;
  // with few tiles the wavefronts are better spread over more workgroups (one decoded token
  // of 8 key/value heads: 10 us unfolded, 16 folded; 64 tokens: 194 and 186)
  p.kv_fold = num_tiles < 32 ? 1 : (n_kv % 4 == 0 ? 4 : (n_kv % 2 == 0 ? 2 : 1));
  p.direct = direct;
  if (staged >= 8) {
    if (d == 64) launch_wide<64>(p, staged, stream); else launch_wide<128>(p, staged, stream);
    MK_LAUNCH_CHECK("attention_mfma");
    return 0;
  }
  switch (d) {
    case 32: staged ? launch_staged<32>(p, rows_per_tile, staged, stream) : launch_attn<32>(p, rows_per_tile, merge, stream); break;
    case 64: staged ? launch_staged<64>(p, rows_per_tile, staged, stream) : launch_attn<64>(p, rows_per_tile, merge, stream); break;
    case 96: staged ? launch_staged<96>(p, rows_per_tile, staged, stream) : launch_attn<96>(p, rows_per_tile, merge, stream); break;
    case 128: staged ? launch_staged<128>(p, rows_per_tile, staged, stream) : launch_attn<128>(p, rows_per_tile, merge, stream); break;
    case 192: staged ? launch_staged<192>(p, rows_per_tile, staged, stream) : launch_attn<192>(p, rows_per_tile, merge, stream); break;
    case 256: staged ? launch_staged<256>(p, rows_per_tile, staged, stream) : launch_attn<256>(p, rows_per_tile, merge, stream); break;
  }
  MK_LAUNCH_CHECK("attention_mfma");
  return 0;
}

extern "C" int mk_attention_mfma(const void* q, int q_stride, void* out, int out_stride,
                                 const void* k_cache, const void* v_cache, const int* tile_seq,
                                 const int* tile_row0, int num_tiles, const int* cu_q,
                                 const int* kv_len, const int* block_table, int table_stride,
                                 int page_size, int n_q, int n_kv, int d, float scale, int window,
                                 int rows_per_tile, int staged, int num_splits, int split_blocks,
                                 float* part_o, float* part_ml, hipStream_t stream) {
  return attention_mfma(q, q_stride, out, out_stride, k_cache, v_cache, tile_seq, tile_row0,
                        num_tiles, cu_q, kv_len, block_table, table_stride, page_size, n_q, n_kv, d,
                        scale, window, rows_per_tile, staged, num_splits, split_blocks, part_o,
                        part_ml, true, stream);
}

extern "C" int mk_attention_mfma_parts_written(int rows_per_tile, int num_splits, int d) {
  return d <= 128 && attn_grouped(rows_per_tile, num_splits) ? num_splits / ATTN_WAVES : num_splits;
}

extern "C" int mk_attention_mfma_parts(const void* q, int q_stride, const void* k_cache,
                                       const void* v_cache, const int* tile_seq,
                                       const int* tile_row0, int num_tiles, const int* cu_q,
                                       const int* kv_len, const int* block_table,
                                       int table_stride, int page_size, int n_q, int n_kv, int d,
                                       float scale, int window, int rows_per_tile, int num_splits,
                                       int split_blocks, float* part_o, float* part_ml,
                                       hipStream_t stream) {
  // (four parts that one workgroup's wavefronts add up are one result, written to `out`)
  MK_REQUIRE(num_splits > 1 && mk_attention_mfma_parts_written(rows_per_tile, num_splits, d) > 1,
             "attention: partial results are left only where the keys are split over workgroups");
  return attention_mfma(q, q_stride, nullptr, n_q * d, k_cache, v_cache, tile_seq, tile_row0,
                        num_tiles, cu_q, kv_len, block_table, table_stride, page_size, n_q, n_kv, d,
                        scale, window, rows_per_tile, 0, num_splits, split_blocks, part_o, part_ml,
                        false, stream);
}

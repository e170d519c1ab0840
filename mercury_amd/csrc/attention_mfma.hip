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
  float* part_o;   // [tile, kv head, split, 16, D]
  float* part_ml;  // [tile, kv head, split, 16, 2]
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
};

#define ATTN_WAVES 4

template <int D>
__global__ __launch_bounds__(64 * ATTN_WAVES) void attn_mfma_kernel(AttnParams p) {
  const int lane = threadIdx.x & 63;
  const int tile = blockIdx.x * ATTN_WAVES + (threadIdx.x >> 6);
  if (tile >= p.num_tiles) return;
  const int kvh = blockIdx.y, split = blockIdx.z;
  const int seq = p.tile_seq[tile], row0 = p.tile_row0[tile];
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int pos0 = p.kv_len[seq] - q_len;  // position of the step's first token of the sequence
  const int G = p.group;
  const int rows_total = q_len * G;
  const int r = lane & 15, g4 = lane >> 4;

  // The row this lane stands for as a column of S^T and O^T.
  const int flat = row0 + r;
  const bool row_ok = flat < rows_total;
  const int tok = row_ok ? flat / G : 0;
  const int head = kvh * G + (row_ok ? flat % G : 0);
  const int pos = pos0 + tok;
  const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;

  // Keys any row of the tile can see, in blocks of 32, and this split's share of them.
  const int last_flat = min(row0 + 15, rows_total - 1);
  const int kmax = pos0 + last_flat / G;
  const int kmin = p.window > 0 ? max(0, pos0 + row0 / G - p.window + 1) : 0;
  const int blk_lo = kmin >> 5, blk_hi = (kmax >> 5) + 1;
  const int per = (blk_hi - blk_lo + p.num_splits - 1) / p.num_splits;
  const int b0 = blk_lo + split * per, b1 = min(blk_hi, b0 + per);

  Frag qf[D / 32];
  {
    const bf16_t* qrow = p.q + (size_t)(q0 + tok) * p.q_stride + head * D + g4 * 8;
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
      qf[c].u = row_ok ? *(const uint4*)(qrow + c * 32) : make_uint4(0, 0, 0, 0);
  }

  f32x4 acc[D / 16];
#pragma unroll
  for (int dt = 0; dt < D / 16; ++dt) acc[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;
  const int ps = 1 << p.page_shift;
  const int* table = p.block_table + (size_t)seq * p.table_stride;

  for (int b = b0; b < b1; ++b) {
    const int key0 = b << 5;
    // Addresses first, then every load of the block (keys and values) before any use, so
    // that one trip to memory covers them all.
    bool live[2];
    const bf16_t* krow[2];
    const bf16_t* vrow[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kh = key0 + h * 16;
      live[h] = kh <= kmax && kh + 15 >= kmin;  // the same for the whole wavefront
      const int page = live[h] ? table[kh >> p.page_shift] : 0;
      const int off = kh & (ps - 1);
      const size_t head_base = (size_t)page * p.n_kv + kvh;
      krow[h] = p.k_cache + (head_base * ps + off + r) * D + g4 * 8;
      vrow[h] = p.v_cache + head_base * ps * D + off + (size_t)r * ps + g4 * 4;
    }
    Frag kf[2][D / 32], vf[D / 16];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int c = 0; c < D / 32; ++c)
        kf[h][c].u = live[h] ? *(const uint4*)(krow[h] + c * 32) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt)
#pragma unroll
      for (int h = 0; h < 2; ++h)
        vf[dt].u2[h] = live[h] ? *(const uint2*)(vrow[h] + (size_t)dt * 16 * ps) : make_uint2(0, 0);

    float s[8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < D / 32; ++c)
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[h][c].v, qf[c].v, sc, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + h * 16 + g4 * 4 + i;
        const bool ok = live[h] && row_ok && key <= pos && key >= lo;
        s[h * 4 + i] = ok ? sc[i] * p.scale : -INFINITY;
      }
    }

    float bm = s[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) bm = fmaxf(bm, s[j]);
    bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
    bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
    const float m_new = fmaxf(m, bm);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __expf(m - m_use);
    Frag pf;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bf16_t e = f32_to_bf16(__expf(s[j] - m_use));
      pf.h[j] = e;
      psum += bf16_to_f32(e);
    }
    lsum = lsum * corr + psum;
    m = m_new;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) {
      acc[dt] *= corr;
      acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pf.v, acc[dt], 0, 0, 0);
    }
  }

  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);

  // acc[dt][i] is O^T[dim = dt*16 + g4*4 + i][row r].
  if (p.num_splits == 1) {
    if (!row_ok) return;
    const float inv = 1.f / lsum;
    bf16_t* dst = p.out + (size_t)(q0 + tok) * p.out_stride + head * D + g4 * 4;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) {
      ushort4 o;
      o.x = f32_to_bf16(acc[dt][0] * inv);
      o.y = f32_to_bf16(acc[dt][1] * inv);
      o.z = f32_to_bf16(acc[dt][2] * inv);
      o.w = f32_to_bf16(acc[dt][3] * inv);
      *(ushort4*)(dst + dt * 16) = o;
    }
  } else {
    const size_t slot = (((size_t)tile * p.n_kv + kvh) * p.num_splits + split) * 16 + r;
    float* po = p.part_o + slot * D + g4 * 4;
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt)
      *(float4*)(po + dt * 16) = make_float4(acc[dt][0], acc[dt][1], acc[dt][2], acc[dt][3]);
    if (g4 == 0) {
      p.part_ml[slot * 2] = m;
      p.part_ml[slot * 2 + 1] = lsum;
    }
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
  const int tile = blockIdx.x, kvh = blockIdx.y, r = blockIdx.z;
  const int seq = p.tile_seq[tile], row0 = p.tile_row0[tile];
  const int q0 = p.cu_q[seq], q_len = p.cu_q[seq + 1] - q0;
  const int G = p.group;
  const int flat = row0 + r;
  if (flat >= q_len * G) return;
  const int S = p.num_splits;
  const size_t base = ((size_t)tile * p.n_kv + kvh) * S;

  float mx = -INFINITY;
  for (int s = threadIdx.x; s < S; s += blockDim.x)
    mx = fmaxf(mx, p.part_ml[((base + s) * 16 + r) * 2]);
  mx = block_max(mx, scratch);
  float part = 0.f;
  for (int s = threadIdx.x; s < S; s += blockDim.x) {
    const size_t slot = (base + s) * 16 + r;
    const float ms = p.part_ml[slot * 2];
    const float w = ms == -INFINITY ? 0.f : __expf(ms - mx);
    weight[s] = w;
    part += p.part_ml[slot * 2 + 1] * w;
  }
  const float total = block_sum(part, scratch);  // also orders the writes of weight[]

  const int g = threadIdx.x >> 6;
  for (int dim = threadIdx.x & 63; dim < D; dim += 64) {
    const float* src = p.part_o + ((base * 16) + r) * D + dim;
    const size_t stride = (size_t)16 * D;
    float o = 0.f;
    int s = g;
    for (; s + 12 < S; s += 16) {
      const float a = src[(size_t)s * stride] * weight[s];
      const float b = src[(size_t)(s + 4) * stride] * weight[s + 4];
      const float c = src[(size_t)(s + 8) * stride] * weight[s + 8];
      const float d = src[(size_t)(s + 12) * stride] * weight[s + 12];
      o += (a + b) + (c + d);
    }
    for (; s < S; s += 4) o += src[(size_t)s * stride] * weight[s];
    group_sum[g][dim] = o;
  }
  __syncthreads();
  const int tok = flat / G, head = kvh * G + flat % G;
  for (int dim = threadIdx.x; dim < D; dim += blockDim.x) {
    const float o = (group_sum[0][dim] + group_sum[1][dim]) + (group_sum[2][dim] + group_sum[3][dim]);
    p.out[(size_t)(q0 + tok) * p.out_stride + head * D + dim] = f32_to_bf16(o / total);
  }
}

template <int D>
static void launch_attn(const AttnParams& p, hipStream_t stream) {
  dim3 grid((p.num_tiles + ATTN_WAVES - 1) / ATTN_WAVES, p.n_kv, p.num_splits);
  attn_mfma_kernel<D><<<grid, 64 * ATTN_WAVES, 0, stream>>>(p);
  if (p.num_splits > 1) {
    dim3 mgrid(p.num_tiles, p.n_kv, 16);
    attn_merge_kernel<D><<<mgrid, 256, 0, stream>>>(p);
  }
}

extern "C" int mk_attention_mfma_supported(int head_dim, int page_size) {
  const bool d_ok = head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128 ||
                    head_dim == 192 || head_dim == 256;
  return d_ok && page_size >= 16 && mk_is_pow2(page_size);
}

extern "C" int mk_attention_mfma(const void* q, int q_stride, void* out, int out_stride,
                                 const void* k_cache, const void* v_cache, const int* tile_seq,
                                 const int* tile_row0, int num_tiles, const int* cu_q,
                                 const int* kv_len, const int* block_table, int table_stride,
                                 int page_size, int n_q, int n_kv, int d, float scale, int window,
                                 int num_splits, float* part_o, float* part_ml,
                                 hipStream_t stream) {
  MK_REQUIRE(num_tiles >= 0 && n_q > 0 && n_kv > 0, "attention: bad sizes");
  MK_REQUIRE(n_q % n_kv == 0, "attention: %d query heads are not a multiple of %d kv heads",
             n_q, n_kv);
  MK_REQUIRE(mk_attention_mfma_supported(d, page_size),
             "attention (matrix cores): head size %d / page size %d not supported; head sizes "
             "32, 64, 96, 128, 192, 256 and pages of 16 or more are",
             d, page_size);
  MK_REQUIRE(num_splits >= 1 && num_splits <= 1024 && n_kv <= 65535, "attention: bad grid");
  MK_REQUIRE(num_splits == 1 || (part_o && part_ml), "attention: key splits need a workspace");
  MK_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0,
             "attention: row strides %d/%d break 16-byte alignment", q_stride, out_stride);
  MK_REQUIRE(window >= 0, "attention: negative window");
  if (num_tiles == 0) return 0;
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
  switch (d) {
    case 32: launch_attn<32>(p, stream); break;
    case 64: launch_attn<64>(p, stream); break;
    case 96: launch_attn<96>(p, stream); break;
    case 128: launch_attn<128>(p, stream); break;
    case 192: launch_attn<192>(p, stream); break;
    case 256: launch_attn<256>(p, stream); break;
  }
  MK_LAUNCH_CHECK("attention_mfma");
  return 0;
}

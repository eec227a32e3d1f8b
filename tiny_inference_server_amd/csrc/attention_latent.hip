// Attention over one shared latent per position on the matrix cores (gfx950, bfloat16): every query head of a row
// attends the same keys (KD channels: the latent and a rotated part) and takes the keys' first VD channels as values.
// Built once per (KD, VD): -DTIS_LATENT=KD*10000+VD.
//
// Pages of 16 slots hold the keys as [slot][KD] and then the values transposed, [VD][slot] (the layout of every
// attention kernel of this engine with one key/value head). One wave takes an item: 16 columns that share their keys,
// a column being a (row, query head) pair: with 16 heads or more a row's heads in blocks of 16, with fewer heads as many
// consecutive rows of one request as fit. Keys go by in steps of 32 (two pages):
//   S^T = K . Q^T    keys are the A operand straight from memory (16 bytes a lane), the queries stay in registers
//   O^T += V^T . P^T the transposed values are the A operand straight from memory, the weights never leave registers
// both on v_mfma_f32_16x16x32_bf16. The lane that holds a column's scores of the keys 4g .. 4g+3 of both pages feeds
// exactly those eight as its share of P^T, and takes the values of the same eight keys: the contraction's order is
// free as long as both operands agree. Softmax in 32-bit with a running maximum per column. Slots behind a row's
// position are read (their page is mapped) but their scores become -inf and their values zero before any arithmetic.
// A long key range is cut into `n_splits` parts (grid z) whose partial results a second kernel merges.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_attention_latent)

#ifndef TIS_LATENT
#define TIS_LATENT 5760512
#endif
static constexpr int KD = TIS_LATENT / 10000, VD = TIS_LATENT % 10000;
static_assert(KD % 8 == 0 && VD % 16 == 0 && VD <= KD && VD >= 16, "key channels in steps of 8, value channels in steps of 16");
static constexpr int DC = (KD + 31) / 32;      // 32-channel chunks of a key
static constexpr int DB = VD / 16;             // 16-channel blocks of a value
static constexpr int PAGE = 16;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ float quad_max(float v) {      // over the four lanes that share a column
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float quad_sum(float v) {
  v += __shfl_xor(v, 16, 64);
  return v + __shfl_xor(v, 32, 64);
}

__global__ __launch_bounds__(64) void latent_mfma_kernel(
    const bf16* __restrict__ q, long ldq, const bf16* __restrict__ plane, const int* __restrict__ block_tables, int bt_ld,
    const int* __restrict__ row_seq, const int* __restrict__ positions, const int2* __restrict__ items,
    bf16* __restrict__ out, long ldo, float* __restrict__ part_o, float2* __restrict__ part_ml, int H, float scale_log2,
    int n_splits) {
  const int item = blockIdx.x, hb = blockIdx.y, split = blockIdx.z;
  const int lane = threadIdx.x, c16 = lane & 15, g = lane >> 4;
  const int row0 = items ? items[item].x : item;
  const int n_rows = items ? items[item].y : 1;
  const int p_first = positions[row0];
  const int* bt = block_tables + (long)row_seq[row0] * bt_ld;
  const int p_last = p_first + n_rows - 1;
  // the lane's column
  const int ro = H >= 16 ? 0 : c16 / H;
  const int head = H >= 16 ? hb * 16 + c16 : c16 % H;
  const bool col_ok = ro < n_rows && head < H;
  const int col_row = row0 + (col_ok ? ro : 0);
  const int col_pos = col_ok ? p_first + ro : -1;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  bf16x8 qb[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) {
    const int d = dc * 32 + g * 8;
    qb[dc] = (col_ok && d < KD) ? *reinterpret_cast<const bf16x8*>(q + (long)col_row * ldq + (long)head * KD + d) : zero8;
  }

  const int n_steps = p_last / 32 + 1;
  const int per = (n_steps + n_splits - 1) / n_splits;
  const int s_begin = split * per, s_end = min(n_steps, s_begin + per);
  f32x4 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const long page_stride = (long)PAGE * (KD + VD);

  for (int s = s_begin; s < s_end; ++s) {
    const int kb = s * 32;
    const bool ok1 = kb + 16 <= p_last;                       // the step's second page holds keys some row sees
    const bf16* pg0 = plane + (long)bt[kb >> 4] * page_stride;
    const bf16* pg1 = plane + (long)(ok1 ? bt[(kb >> 4) + 1] : bt[kb >> 4]) * page_stride;
    f32x4 st0 = {0.f, 0.f, 0.f, 0.f}, st1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
      const int d = dc * 32 + g * 8;
      const bf16x8 k0 = d < KD ? *reinterpret_cast<const bf16x8*>(pg0 + (long)c16 * KD + d) : zero8;
      const bf16x8 k1 = (d < KD && ok1) ? *reinterpret_cast<const bf16x8*>(pg1 + (long)c16 * KD + d) : zero8;
      st0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qb[dc], st0, 0, 0, 0);
      st1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qb[dc], st1, 0, 0, 0);
    }
    // the lane holds, for its column, the scores of the keys kb + 4g + i (first page) and kb + 16 + 4g + i (second)
    float sv[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key0 = kb + 4 * g + i, key1 = key0 + 16;
      sv[i] = key0 <= col_pos ? st0[i] * scale_log2 : -INFINITY;
      sv[4 + i] = (ok1 && key1 <= col_pos) ? st1[i] * scale_log2 : -INFINITY;
      tmax = fmaxf(tmax, fmaxf(sv[i], sv[4 + i]));
    }
    tmax = quad_max(tmax);
    const float m_new = fmaxf(m, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;     // a column with no key yet: everything stays 0
    const float alpha = exp2f(m - m_use);
    float psum = 0.f;
    bf16x8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = exp2f(sv[e] - m_use);
      psum += p;
      pb[e] = static_cast<__bf16>(p);
    }
    l = l * alpha + psum;
    m = m_new;
    const bool last = kb + 31 > p_last;                        // some of the step's slots lie behind every row
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const long off = (long)PAGE * KD + (long)(db * 16 + c16) * PAGE + 4 * g;
      const bf16x4 lo = *reinterpret_cast<const bf16x4*>(pg0 + off);
      const bf16x4 hi = ok1 ? *reinterpret_cast<const bf16x4*>(pg1 + off) : (bf16x4){0, 0, 0, 0};
      bf16x8 va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      if (last) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (kb + 4 * g + i > p_last) va[i] = static_cast<__bf16>(0.f);
          if (kb + 16 + 4 * g + i > p_last) va[4 + i] = static_cast<__bf16>(0.f);
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) o[db][i] *= alpha;
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb, o[db], 0, 0, 0);
    }
  }

  // the lane holds, for its column, the channels db * 16 + 4g + i
  const float lt = quad_sum(l);
  if (!col_ok) return;
  if (n_splits == 1) {
    const float inv = 1.f / lt;
    bf16* dst = out + (long)col_row * ldo + (long)head * VD + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x4 w;
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = static_cast<__bf16>(o[db][i] * inv);
      *reinterpret_cast<bf16x4*>(dst + db * 16) = w;
    }
  } else {
    const long slot = ((long)col_row * H + head) * n_splits + split;
    float* dst = part_o + slot * VD + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; ++db) *reinterpret_cast<f32x4*>(dst + db * 16) = o[db];
    if (g == 0) part_ml[slot] = make_float2(m, lt);
  }
}

// Portions of prompts: a workgroup of four waves takes an item of 64 columns (with fewer than 64 heads, 64 / heads
// consecutive rows of one request; else a row's heads in blocks of 64), 16 columns a wave. A step's keys and transposed
// values are copied into LDS once per workgroup and are every wave's MFMA operands from there, so a key is fetched
// once per 64 columns instead of once per 16. Key rows lie 16 bytes further apart in LDS than in memory, so that the
// sixteen keys a group of lanes reads at one channel offset fall into different banks.
static constexpr int TK_STRIDE = KD + 8;                       // elements between two keys in LDS
static constexpr int TK_BYTES = 32 * TK_STRIDE * 2, TV_BYTES = 2 * VD * PAGE * 2;

__global__ __launch_bounds__(256) void latent_tile_kernel(
    const bf16* __restrict__ q, long ldq, const bf16* __restrict__ plane, const int* __restrict__ block_tables, int bt_ld,
    const int* __restrict__ row_seq, const int* __restrict__ positions, const int2* __restrict__ items,
    bf16* __restrict__ out, long ldo, int H, float scale_log2) {
  __shared__ __attribute__((aligned(16))) bf16 k_lds[32 * TK_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16 v_lds[2 * VD * PAGE];
  const int item = blockIdx.x, hb = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c16 = lane & 15, g = lane >> 4;
  const int row0 = items[item].x, n_rows = items[item].y;
  const int p_first = positions[row0];
  const int* bt = block_tables + (long)row_seq[row0] * bt_ld;
  const int p_last = p_first + n_rows - 1;
  const int c = wave * 16 + c16;                                // the lane's column among the item's 64
  const int ro = H >= 64 ? 0 : c / H;
  const int head = H >= 64 ? hb * 64 + c : c % H;
  const bool col_ok = ro < n_rows && head < H && (H >= 64 || c < (64 / H) * H);
  const int col_row = row0 + (col_ok ? ro : 0);
  const int col_pos = col_ok ? p_first + ro : -1;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  bf16x8 qb[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) {
    const int d = dc * 32 + g * 8;
    qb[dc] = (col_ok && d < KD) ? *reinterpret_cast<const bf16x8*>(q + (long)col_row * ldq + (long)head * KD + d) : zero8;
  }
  f32x4 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const long page_stride = (long)PAGE * (KD + VD);
  const int n_steps = p_last / 32 + 1;
  constexpr int KP = KD / 8;                                    // 16-byte pieces of a key
  constexpr int VP = VD * PAGE / 8;                             // ... of a page's values

  // A thread's pieces of a step's keys and values, fetched into registers a step ahead (all loads issued together,
  // in flight while the step before is computed) and put into LDS between two barriers.
  constexpr int KN = (32 * KP + 255) / 256, VN = (2 * VP + 255) / 256;
  bf16x8 kreg[KN], vreg[VN];
  auto fetch = [&](int s) {
    const int kb = s * 32;
    const bool ok1 = kb + 16 <= p_last;
    const bf16* pg0 = plane + (long)bt[kb >> 4] * page_stride;
    const bf16* pg1 = plane + (long)(ok1 ? bt[(kb >> 4) + 1] : bt[kb >> 4]) * page_stride;
#pragma unroll
    for (int j = 0; j < KN; ++j) {
      const int i = tid + j * 256, key = i / KP, piece = i % KP;
      if (i < 32 * KP) kreg[j] = *reinterpret_cast<const bf16x8*>((key < 16 ? pg0 : pg1) + (long)(key & 15) * KD + piece * 8);
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      const int i = tid + j * 256, pgi = i / VP, piece = i % VP;
      if (i < 2 * VP) vreg[j] = *reinterpret_cast<const bf16x8*>((pgi ? pg1 : pg0) + (long)PAGE * KD + piece * 8);
    }
  };
  fetch(0);
  for (int s = 0; s < n_steps; ++s) {
    const int kb = s * 32;
    const bool ok1 = kb + 16 <= p_last;
    __syncthreads();                                            // everyone has read the step before
#pragma unroll
    for (int j = 0; j < KN; ++j) {
      const int i = tid + j * 256, key = i / KP, piece = i % KP;
      if (i < 32 * KP) *reinterpret_cast<bf16x8*>(k_lds + key * TK_STRIDE + piece * 8) = kreg[j];
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      const int i = tid + j * 256;
      if (i < 2 * VP) *reinterpret_cast<bf16x8*>(v_lds + i * 8) = vreg[j];
    }
    __syncthreads();
    if (s + 1 < n_steps) fetch(s + 1);
    f32x4 st0 = {0.f, 0.f, 0.f, 0.f}, st1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
      const int d = dc * 32 + g * 8;
      const bf16x8 k0 = d < KD ? *reinterpret_cast<const bf16x8*>(k_lds + c16 * TK_STRIDE + d) : zero8;
      const bf16x8 k1 = d < KD ? *reinterpret_cast<const bf16x8*>(k_lds + (16 + c16) * TK_STRIDE + d) : zero8;
      st0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qb[dc], st0, 0, 0, 0);
      st1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qb[dc], st1, 0, 0, 0);
    }
    float sv[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key0 = kb + 4 * g + i, key1 = key0 + 16;
      sv[i] = key0 <= col_pos ? st0[i] * scale_log2 : -INFINITY;
      sv[4 + i] = (ok1 && key1 <= col_pos) ? st1[i] * scale_log2 : -INFINITY;
      tmax = fmaxf(tmax, fmaxf(sv[i], sv[4 + i]));
    }
    tmax = quad_max(tmax);
    const float m_new = fmaxf(m, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2f(m - m_use);
    float psum = 0.f;
    bf16x8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = exp2f(sv[e] - m_use);
      psum += p;
      pb[e] = static_cast<__bf16>(p);
    }
    l = l * alpha + psum;
    m = m_new;
    const bool last = kb + 31 > p_last;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int off = (db * 16 + c16) * PAGE + 4 * g;
      const bf16x4 lo = *reinterpret_cast<const bf16x4*>(v_lds + off);
      const bf16x4 hi = ok1 ? *reinterpret_cast<const bf16x4*>(v_lds + VD * PAGE + off) : (bf16x4){0, 0, 0, 0};
      bf16x8 va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      if (last) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (kb + 4 * g + i > p_last) va[i] = static_cast<__bf16>(0.f);
          if (kb + 16 + 4 * g + i > p_last) va[4 + i] = static_cast<__bf16>(0.f);
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) o[db][i] *= alpha;
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb, o[db], 0, 0, 0);
    }
  }
  const float lt = quad_sum(l);
  if (!col_ok) return;
  const float inv = 1.f / lt;
  bf16* dst = out + (long)col_row * ldo + (long)head * VD + 4 * g;
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    bf16x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = static_cast<__bf16>(o[db][i] * inv);
    *reinterpret_cast<bf16x4*>(dst + db * 16) = w;
  }
}

// out[row, head, :] = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s over a (row, head)'s splits, in a fixed order
__global__ __launch_bounds__(256) void latent_merge_kernel(const float* __restrict__ part_o, const float2* __restrict__ part_ml,
                                                           bf16* __restrict__ out, long ldo, int H, int n_splits) {
  __shared__ float w[256];                 // the weights of up to 256 splits at a time
  __shared__ float red[16];
  const long row = blockIdx.x;
  const int head = blockIdx.y, t = threadIdx.x;
  const long base = (row * H + head) * n_splits;
  float M = -INFINITY;
  for (int s = t; s < n_splits; s += 256) M = fmaxf(M, part_ml[base + s].x);
  M = block_max(M, red);
  float L = 0.f;
  float acc[(VD + 255) / 256];
#pragma unroll
  for (int j = 0; j < (VD + 255) / 256; ++j) acc[j] = 0.f;
  for (int s0 = 0; s0 < n_splits; s0 += 256) {
    const int cnt = min(256, n_splits - s0);
    float mine = 0.f, share = 0.f;
    if (t < cnt) {
      const float2 ml = part_ml[base + s0 + t];
      if (ml.x != -INFINITY) {             // else: a split that held no key of this row (its partial output is zero)
        mine = exp2f(ml.x - M);
        share = mine * ml.y;
      }
    }
    __syncthreads();
    w[t] = mine;
    L += block_sum(share, red);            // its barriers also publish w[]
    // (a split's partial outputs are independent loads: several are in flight at a time)
#pragma unroll
    for (int j = 0; j < (VD + 255) / 256; ++j) {
      const int c = j * 256 + t;
      if (c >= VD) continue;
      const float* src = part_o + (base + s0) * VD + c;
      float a = 0.f;
#pragma unroll 8
      for (int s = 0; s < cnt; ++s) a += w[s] * src[(long)s * VD];
      acc[j] += a;
    }
  }
#pragma unroll
  for (int j = 0; j < (VD + 255) / 256; ++j) {
    const int c = j * 256 + t;
    if (c < VD) out[row * ldo + (long)head * VD + c] = static_cast<__bf16>(acc[j] / L);
  }
}

TIS_EXPORT int tis_attention_latent_dims() { return TIS_LATENT; }

// items: (first row, rows) per item, or null where every item is the single row of its own index. part_o / part_ml:
// [rows][H][n_splits][VD] floats and [rows][H][n_splits] (maximum, sum) pairs, needed where n_splits > 1.
// n_splits 0: the items are those of the four-wave kernel (64 columns each: 64 / H rows, or a row's heads in blocks of
// 64), which takes every item's keys whole.
TIS_EXPORT int tis_attention_latent(const void* q, long ldq, const void* plane, const int* block_tables, int bt_ld,
                                    const int* row_seq, const int* positions, const int* items, int n_items, void* out,
                                    long ldo, float* part_o, float* part_ml, int rows, int H, int key_dim, int value_dim,
                                    int page_size, float scale, int n_splits, hipStream_t stream) {
  if (rows == 0 || n_items == 0) return 0;
  if (key_dim != KD || value_dim != VD) return tis_fail("attention_latent: built for keys of %d and values of %d, called with %d and %d", KD, VD, key_dim, value_dim);
  if (page_size != PAGE) return tis_fail("attention_latent: pages of %d slots (this kernel takes %d)", page_size, PAGE);
  if (rows < 0 || n_items < 0 || H < 1 || n_splits < 0 || n_splits > 65535 || (H + 15) / 16 > 65535)
    return tis_fail("attention_latent: bad size rows=%d items=%d heads=%d splits=%d", rows, n_items, H, n_splits);
  if (n_splits > 1 && (!part_o || !part_ml)) return tis_fail("attention_latent: %d splits need a workspace", n_splits);
  if ((ldq % 8) || (ldo % 4) || ((uintptr_t)q % 16) || ((uintptr_t)out % 8) || ((uintptr_t)plane % 16))
    return tis_fail("attention_latent: q, out and the cache plane must be 16-byte aligned with row strides in steps of 8");
  if (n_splits == 0) {
    if (!items) return tis_fail("attention_latent: the four-wave kernel needs its list of items");
    dim3 tgrid(n_items, (H + 63) / 64);
    latent_tile_kernel<<<tgrid, 256, 0, stream>>>((const bf16*)q, ldq, (const bf16*)plane, block_tables, bt_ld, row_seq,
                                                  positions, (const int2*)items, (bf16*)out, ldo, H,
                                                  scale * 1.4426950408889634f);
    return tis_launch_status("attention_latent tiles");
  }
  dim3 grid(n_items, (H + 15) / 16, n_splits);
  latent_mfma_kernel<<<grid, 64, 0, stream>>>((const bf16*)q, ldq, (const bf16*)plane, block_tables, bt_ld, row_seq, positions,
                                             (const int2*)items, (bf16*)out, ldo, part_o, (float2*)part_ml, H,
                                             scale * 1.4426950408889634f, n_splits);
  int rc = tis_launch_status("attention_latent");
  if (rc || n_splits == 1) return rc;
  dim3 mgrid(rows, H);
  latent_merge_kernel<<<mgrid, 256, 0, stream>>>(part_o, (const float2*)part_ml, (bf16*)out, ldo, H, n_splits);
  return tis_launch_status("attention_latent merge");
}

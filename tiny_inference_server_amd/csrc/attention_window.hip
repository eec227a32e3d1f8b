// Softmax attention whose keys and values differ in size, over a paged cache, with a sliding window: the step before
// it (per-head RMS norm of queries and keys, rotation of the first channels in interleaved pairs, a factor per query
// head, unit-RMS values, the write into the pages) and the attention itself.
//
// A page of `page_size` slots holds, for each key/value head, the keys as [slot][key size] and then, after the keys
// of all heads, the values transposed as [value size][slot]. With equal sizes that is the layout the other attention
// kernels read. The row at position p sees the keys at [max(0, p - window + 1), p] (window 0: all), found through the
// request's block table; keys outside are never read, so what a reused page holds cannot reach a result.
// Norms, angles, scores, the softmax and the weighted sum are 32-bit; `T` is the type of queries and pages.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_attention_window)

static constexpr int AW_THREADS = 256;
static constexpr int AW_CHUNK = 1024;
static constexpr int AW_MAX_DIM = 256;

// grid (rows, H + 2 G), one wave each: unit u < H is a query head, u < H + G a key head, else a value head.
// proj holds the projections of a row in 32-bit: queries at q_off, keys at k_off, values at v_off.
template <typename T>
__global__ __launch_bounds__(TIS_WAVE) void attention_prepare_kernel(
    const float* __restrict__ proj, long ldp, int q_off, int k_off, int v_off, const int* __restrict__ positions,
    const int* __restrict__ write_slots, T* __restrict__ plane, T* __restrict__ q_out, long ldq,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, const float* __restrict__ q_factor,
    const float* __restrict__ freqs, int rot_dims, float eps, int H, int G, int KD, int VD, int page_size) {
  const long r = blockIdx.x;
  const int u = blockIdx.y, lane = threadIdx.x;
  const long page_stride = (long)G * page_size * (KD + VD);
  if (u < H + G) {
    const bool is_q = u < H;
    const int h = is_q ? u : u - H;
    if (!is_q && !write_slots) return;
    const float* src = proj + r * ldp + (is_q ? q_off : k_off) + (long)h * KD;
    const float* gain = is_q ? q_gain : k_gain;
    float ss = 0.f;
    for (int e = lane; e < KD; e += TIS_WAVE) ss += src[e] * src[e];
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)KD + eps);
    const float factor = is_q ? q_factor[h] : 1.f;
    const float pos = (float)positions[r];
    T* dst;
    if (is_q) {
      dst = q_out + r * ldq + (long)h * KD;
    } else {
      const int ws = write_slots[r];
      dst = plane + (long)(ws / page_size) * page_stride + ((long)h * page_size + ws % page_size) * KD;
    }
    for (int p = lane; 2 * p < KD; p += TIS_WAVE) {
      const int e0 = 2 * p, e1 = e0 + 1;
      float a = src[e0] * inv * gain[e0];
      float b = e1 < KD ? src[e1] * inv * gain[e1] : 0.f;
      if (e1 < rot_dims) {
        float sn, cs;
        sincosf(pos * freqs[p], &sn, &cs);
        const float ra = a * cs - b * sn, rb = b * cs + a * sn;
        a = ra;
        b = rb;
      }
      dst[e0] = from_f<T>(a * factor);
      if (e1 < KD) dst[e1] = from_f<T>(b * factor);
    }
  } else {
    if (!write_slots) return;
    const int h = u - H - G;
    const float* src = proj + r * ldp + v_off + (long)h * VD;
    float ss = 0.f;
    for (int e = lane; e < VD; e += TIS_WAVE) ss += src[e] * src[e];
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)VD + eps);
    const int ws = write_slots[r];
    T* dst = plane + (long)(ws / page_size) * page_stride + (long)G * page_size * KD + (long)h * VD * page_size +
             ws % page_size;
    for (int e = lane; e < VD; e += TIS_WAVE) dst[(long)e * page_size] = from_f<T>(src[e] * inv);
  }
}

// One workgroup per (row, query head). Keys are walked in chunks of AW_CHUNK with a running maximum; the order of
// every sum depends on the row's own position and window only.
template <typename T>
__global__ __launch_bounds__(AW_THREADS) void attention_window_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ plane, const int* __restrict__ block_tables, int bt_ld,
    const int* __restrict__ row_seq, const int* __restrict__ positions, T* __restrict__ out, long ldo, int group_size,
    int G, int KD, int VD, int page_size, int window, float scale) {
  __shared__ float qs[AW_MAX_DIM];
  __shared__ float sc[AW_CHUNK];
  __shared__ float red[16];
  __shared__ float accm[AW_THREADS];
  const long r = blockIdx.x;
  const int h = blockIdx.y, g = h / group_size, t = threadIdx.x;
  const int pos = positions[r];
  const int* bt = block_tables + (long)row_seq[r] * bt_ld;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int end = pos + 1;
  for (int d = t; d < KD; d += AW_THREADS) qs[d] = to_f(q[r * ldq + (long)h * KD + d]) * scale;
  __syncthreads();
  const long page_stride = (long)G * page_size * (KD + VD);
  const long k_off = (long)g * page_size * KD;
  const long v_off = (long)G * page_size * KD + (long)g * VD * page_size;
  const int lanes_per_key = AW_THREADS / VD;      // threads that share a value channel, each taking every n-th key
  const int part = t / VD, d = t % VD;
  const bool pv = part < lanes_per_key;
  float m = -INFINITY, l = 0.f, acc = 0.f;
  for (int c0 = first; c0 < end; c0 += AW_CHUNK) {
    const int n = min(AW_CHUNK, end - c0);
    float cmax = -INFINITY;
    for (int i = t; i < n; i += AW_THREADS) {
      const int j = c0 + i;
      const T* kp = plane + (long)bt[j / page_size] * page_stride + k_off + (long)(j % page_size) * KD;
      float s = 0.f;
      for (int e = 0; e < KD; ++e) s += qs[e] * to_f(kp[e]);
      sc[i] = s;
      cmax = fmaxf(cmax, s);
    }
    cmax = block_max(cmax, red);
    const float m_new = fmaxf(m, cmax);
    float csum = 0.f;
    for (int i = t; i < n; i += AW_THREADS) {
      const float p = expf(sc[i] - m_new);
      sc[i] = p;
      csum += p;
    }
    csum = block_sum(csum, red);      // its barriers also publish sc[]
    const float rescale = expf(m - m_new);
    l = l * rescale + csum;
    acc *= rescale;
    m = m_new;
    if (pv) {
      for (int i = part; i < n; i += lanes_per_key) {
        const int j = c0 + i;
        const T* vp = plane + (long)bt[j / page_size] * page_stride + v_off + (j % page_size);
        acc += sc[i] * to_f(vp[(long)d * page_size]);
      }
    }
    __syncthreads();
  }
  accm[t] = pv ? acc : 0.f;
  __syncthreads();
  if (t < VD) {
    float o = 0.f;
    for (int p = 0; p < lanes_per_key; ++p) o += accm[p * VD + t];
    out[r * ldo + (long)h * VD + t] = from_f<T>(o / l);
  }
}

TIS_EXPORT int tis_attention_prepare(int dtype, const float* proj, long ldp, int q_off, int k_off, int v_off,
                                     const int* positions, const int* write_slots, void* plane, void* q_out, long ldq,
                                     const float* q_gain, const float* k_gain, const float* q_factor, const float* freqs,
                                     int rot_dims, float eps, int rows, int H, int G, int KD, int VD, int page_size,
                                     hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || G < 1 || KD < 1 || VD < 1 || page_size < 1 || H + 2 * G > 65535)
    return tis_fail("attention_prepare: bad size rows=%d heads=%d kv_heads=%d key=%d value=%d page=%d", rows, H, G, KD, VD,
                    page_size);
  if (rot_dims < 0 || rot_dims > KD || rot_dims % 2) return tis_fail("attention_prepare: %d rotated channels of %d", rot_dims, KD);
  if (write_slots && !plane) return tis_fail("attention_prepare: write slots without pages");
  dim3 grid(rows, H + 2 * G);
  if (dtype == TIS_F32)
    attention_prepare_kernel<float><<<grid, TIS_WAVE, 0, stream>>>(proj, ldp, q_off, k_off, v_off, positions, write_slots,
        (float*)plane, (float*)q_out, ldq, q_gain, k_gain, q_factor, freqs, rot_dims, eps, H, G, KD, VD, page_size);
  else if (dtype == TIS_BF16)
    attention_prepare_kernel<bf16><<<grid, TIS_WAVE, 0, stream>>>(proj, ldp, q_off, k_off, v_off, positions, write_slots,
        (bf16*)plane, (bf16*)q_out, ldq, q_gain, k_gain, q_factor, freqs, rot_dims, eps, H, G, KD, VD, page_size);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("attention_prepare");
}

TIS_EXPORT int tis_attention_window(int dtype, const void* q, long ldq, const void* plane, const int* block_tables,
                                    int bt_ld, const int* row_seq, const int* positions, void* out, long ldo, int rows,
                                    int H, int G, int KD, int VD, int page_size, int window, float scale,
                                    hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || G < 1 || H % G || page_size < 1 || window < 0 || H > 65535)
    return tis_fail("attention_window: bad size rows=%d heads=%d kv_heads=%d page=%d window=%d", rows, H, G, page_size, window);
  if (KD < 1 || KD > AW_MAX_DIM || VD < 1 || VD > AW_MAX_DIM)
    return tis_fail("attention_window: key size %d or value size %d is outside 1..%d", KD, VD, AW_MAX_DIM);
  dim3 grid(rows, H);
  if (dtype == TIS_F32)
    attention_window_kernel<float><<<grid, AW_THREADS, 0, stream>>>((const float*)q, ldq, (const float*)plane, block_tables,
        bt_ld, row_seq, positions, (float*)out, ldo, H / G, G, KD, VD, page_size, window, scale);
  else if (dtype == TIS_BF16)
    attention_window_kernel<bf16><<<grid, AW_THREADS, 0, stream>>>((const bf16*)q, ldq, (const bf16*)plane, block_tables,
        bt_ld, row_seq, positions, (bf16*)out, ldo, H / G, G, KD, VD, page_size, window, scale);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("attention_window");
}

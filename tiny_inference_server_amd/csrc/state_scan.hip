// Recurrent mixers whose state is a matrix per head, S [key channels D][value channels V], walked token by token:
//
//   kind 0, decay per key channel:   S_t = diag(a_t) S_(t-1) + k_t v_t^T,                 o_t = S_t^T q_t
//   kind 1, scalar gates (log input gate i, log forget gate f) with a running maximum m that starts at 0:
//           m_t = max(f_t + m_(t-1), i_t);   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T;
//           n_t the same with k_t alone;      o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),
//           with i = cap tanh((x_i + b_i) / cap), f = log sigmoid(cap tanh((x_f + b_f) / cap)).
//
// One workgroup per (request of the step, head, block of 16 value channels). Thread (s, j) owns the state's column j
// for the key channels s, s + 16, s + 32, ... in registers, from the request's state slot before the first token to
// the slot after the last. Tokens are taken in chunks: a chunk's q, k, v and gates go into LDS, the 16 threads of a
// column leave a partial o per token there, and one pass adds them up. Each state element sees its tokens strictly in
// order with nothing else mixed in, so the result of a token does not depend on how a prompt was cut into steps, on the
// chunk size or on what else is in the batch, bit for bit. State, gates and sums are 32-bit. Kind 1 keeps n and m once
// per block of value channels (every block needs them, none may read what another has already advanced).
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_state_scan)

static constexpr int SC_THREADS = 256;
static constexpr int SC_VB = 16;       // value channels of a workgroup
static constexpr int SC_R = 16;        // threads that share a column
static constexpr int SC_LDS_BYTES = 60 * 1024;

__device__ __forceinline__ float sc_log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <int KIND, int NS>
__global__ __launch_bounds__(SC_THREADS) void state_scan_kernel(
    const float* __restrict__ proj, long ldp, int q_off, int k_off, int v_off, float q_scale,
    const float* __restrict__ decay, long ldd, int i_off, int f_off, const float* __restrict__ bias_i,
    const float* __restrict__ bias_f, float cap, float* __restrict__ state, long state_ld,
    const int* __restrict__ cu_rows, const int* __restrict__ seq_slots, float* __restrict__ out, long ldo, int H, int D,
    int V, int n_vb, int chunk) {
  extern __shared__ float lds[];
  float* sq = lds;                                   // [chunk][D]
  float* sk = sq + chunk * D;                        // [chunk][D]
  float* sa = sk + chunk * D;                        // kind 0: [chunk][D] decays; kind 1: [chunk][3] gates i, f and m
  float* sv = sa + (KIND == 0 ? chunk * D : chunk * 3);   // [chunk][VB]
  float* part = sv + chunk * SC_VB;                  // [chunk][R][VB + 1]

  const int seq = blockIdx.x, h = blockIdx.y, vb = blockIdx.z, t = threadIdx.x;
  const int r0 = cu_rows[seq], r1 = cu_rows[seq + 1];
  if (r0 >= r1) return;
  float* st = state + (long)seq_slots[seq] * state_ld;
  float* S = st + (long)h * D * V;
  float* nm = st + (long)H * D * V + ((long)h * n_vb + vb) * (D + 1);     // kind 1: n [D], then m
  const int j = t % SC_VB, s = t / SC_VB;
  const int col = vb * SC_VB + j;
  const bool col_ok = col < V;

  float Sreg[NS], nreg[NS];
  float m = 0.f;
#pragma unroll
  for (int e = 0; e < NS; ++e) {
    const int i = s + SC_R * e;
    Sreg[e] = (i < D && col_ok) ? S[(long)i * V + col] : 0.f;
    nreg[e] = (KIND == 1 && i < D) ? nm[i] : 0.f;
  }
  if (KIND == 1) m = nm[D];

  for (int c0 = r0; c0 < r1; c0 += chunk) {
    const int nc = min(chunk, r1 - c0);
    __syncthreads();
    for (int idx = t; idx < nc * D; idx += SC_THREADS) {
      const int c = idx / D, i = idx - c * D;
      const float* row = proj + (long)(c0 + c) * ldp;
      sq[idx] = row[q_off + h * D + i] * q_scale;
      sk[idx] = row[k_off + h * D + i];
      if (KIND == 0) sa[idx] = decay[(long)(c0 + c) * ldd + h * D + i];
    }
    for (int idx = t; idx < nc * SC_VB; idx += SC_THREADS) {
      const int c = idx / SC_VB, jj = idx - c * SC_VB;
      sv[idx] = (vb * SC_VB + jj < V) ? proj[(long)(c0 + c) * ldp + v_off + h * V + vb * SC_VB + jj] : 0.f;
    }
    if (KIND == 1 && t < nc) {
      const float* row = proj + (long)(c0 + t) * ldp;
      const float xi = row[i_off + h] + bias_i[h], xf = row[f_off + h] + bias_f[h];
      sa[t * 3] = cap * tanhf(xi / cap);
      sa[t * 3 + 1] = sc_log_sigmoid(cap * tanhf(xf / cap));
    }
    __syncthreads();
    for (int c = 0; c < nc; ++c) {
      float keep = 1.f, take = 1.f;
      if (KIND == 1) {
        const float gi = sa[c * 3], gf = sa[c * 3 + 1];
        const float m_new = fmaxf(gf + m, gi);
        keep = expf(gf + m - m_new);
        take = expf(gi - m_new);
        m = m_new;
      }
      const float vj = sv[c * SC_VB + j];
      float acc = 0.f, nq = 0.f;
#pragma unroll
      for (int e = 0; e < NS; ++e) {
        const int i = s + SC_R * e;
        if (i < D) {
          const float kk = sk[c * D + i], qq = sq[c * D + i];
          if (KIND == 0) {
            Sreg[e] = sa[c * D + i] * Sreg[e] + kk * vj;
          } else {
            Sreg[e] = keep * Sreg[e] + take * (kk * vj);
            nreg[e] = keep * nreg[e] + take * kk;
            nq += nreg[e] * qq;
          }
          acc += Sreg[e] * qq;
        }
      }
      part[(c * SC_R + s) * (SC_VB + 1) + j] = acc;
      if (KIND == 1) {
        if (j == 0) part[(c * SC_R + s) * (SC_VB + 1) + SC_VB] = nq;
        if (t == 0) sa[c * 3 + 2] = m;
      }
    }
    __syncthreads();
    for (int idx = t; idx < nc * SC_VB; idx += SC_THREADS) {
      const int c = idx / SC_VB, jj = idx - c * SC_VB;
      float o = 0.f, nq = 0.f;
      for (int ss = 0; ss < SC_R; ++ss) {
        o += part[(c * SC_R + ss) * (SC_VB + 1) + jj];
        if (KIND == 1) nq += part[(c * SC_R + ss) * (SC_VB + 1) + SC_VB];
      }
      if (KIND == 1) o /= fmaxf(fabsf(nq), expf(-sa[c * 3 + 2])) + 1e-6f;
      if (vb * SC_VB + jj < V) out[(long)(c0 + c) * ldo + h * V + vb * SC_VB + jj] = o;
    }
  }
#pragma unroll
  for (int e = 0; e < NS; ++e) {
    const int i = s + SC_R * e;
    if (i < D && col_ok) S[(long)i * V + col] = Sreg[e];
    if (KIND == 1 && j == 0 && i < D) nm[i] = nreg[e];
  }
  if (KIND == 1 && t == 0) nm[D] = m;
}

template <int KIND>
static int launch_scan(int ns, dim3 grid, size_t lds, hipStream_t stream, const float* proj, long ldp, int q_off, int k_off,
                       int v_off, float q_scale, const float* decay, long ldd, int i_off, int f_off, const float* bias_i,
                       const float* bias_f, float cap, float* state, long state_ld, const int* cu_rows,
                       const int* seq_slots, float* out, long ldo, int H, int D, int V, int n_vb, int chunk) {
#define SC_LAUNCH(NS)                                                                                                   \
  state_scan_kernel<KIND, NS><<<grid, SC_THREADS, lds, stream>>>(proj, ldp, q_off, k_off, v_off, q_scale, decay, ldd,   \
                                                                 i_off, f_off, bias_i, bias_f, cap, state, state_ld,    \
                                                                 cu_rows, seq_slots, out, ldo, H, D, V, n_vb, chunk)
  if (ns <= 1) SC_LAUNCH(1);
  else if (ns <= 2) SC_LAUNCH(2);
  else if (ns <= 4) SC_LAUNCH(4);
  else if (ns <= 8) SC_LAUNCH(8);
  else SC_LAUNCH(16);
#undef SC_LAUNCH
  return tis_launch_status("state_scan");
}

// Floats of one request's state: S for every head, and for kind 1 also n and m per head and block of value channels.
TIS_EXPORT long tis_state_scan_floats(int kind, int H, int D, int V) {
  const long n_vb = (V + SC_VB - 1) / SC_VB;
  return (long)H * D * V + (kind == 1 ? (long)H * n_vb * (D + 1) : 0);
}

TIS_EXPORT int tis_state_scan(int kind, const float* proj, long ldp, int q_off, int k_off, int v_off, float q_scale,
                              const float* decay, long ldd, int i_off, int f_off, const float* bias_i,
                              const float* bias_f, float cap, float* state, long state_ld, const int* cu_rows,
                              const int* seq_slots, int n_seqs, float* out, long ldo, int H, int D, int V,
                              hipStream_t stream) {
  if (n_seqs == 0) return 0;
  if (n_seqs < 0 || H < 1 || H > 65535 || D < 1 || D > SC_R * 16 || V < 1)
    return tis_fail("state_scan: bad size requests=%d heads=%d key channels=%d (at most %d) value channels=%d", n_seqs, H,
                    D, SC_R * 16, V);
  if (kind != 0 && kind != 1) return tis_fail("state_scan: unknown kind %d", kind);
  if (kind == 0 && !decay) return tis_fail("state_scan: kind 0 needs the decays");
  if (kind == 1 && (!bias_i || !bias_f || !(cap > 0.f))) return tis_fail("state_scan: kind 1 needs gate biases and a cap");
  const int n_vb = (V + SC_VB - 1) / SC_VB;
  if (n_vb > 65535) return tis_fail("state_scan: %d value channels exceed the grid", V);
  if (state_ld < tis_state_scan_floats(kind, H, D, V))
    return tis_fail("state_scan: a state line of %ld floats is too short for %ld", state_ld, tis_state_scan_floats(kind, H, D, V));
  int chunk = 16;
  auto bytes = [&](int c) {
    return sizeof(float) * ((size_t)c * D * 2 + (kind == 0 ? (size_t)c * D : (size_t)c * 3) + (size_t)c * SC_VB +
                            (size_t)c * SC_R * (SC_VB + 1));
  };
  while (chunk > 1 && bytes(chunk) > SC_LDS_BYTES) chunk /= 2;
  if (bytes(chunk) > SC_LDS_BYTES) return tis_fail("state_scan: %d key channels do not fit the chunk buffers", D);
  dim3 grid(n_seqs, H, n_vb);
  const int ns = (D + SC_R - 1) / SC_R;
  if (kind == 0)
    return launch_scan<0>(ns, grid, bytes(chunk), stream, proj, ldp, q_off, k_off, v_off, q_scale, decay, ldd, i_off, f_off,
                          bias_i, bias_f, cap, state, state_ld, cu_rows, seq_slots, out, ldo, H, D, V, n_vb, chunk);
  return launch_scan<1>(ns, grid, bytes(chunk), stream, proj, ldp, q_off, k_off, v_off, q_scale, decay, ldd, i_off, f_off,
                        bias_i, bias_f, cap, state, state_ld, cu_rows, seq_slots, out, ldo, H, D, V, n_vb, chunk);
}

// Sequence mixers of the layered models, all sums in fp32.
//
//   lgs_retention        decayed linear attention: rotary (half layout) on q and k, k scaled, then per head
//                        S <- decay S + k v^T, o = S^T q, the state S (d x dv fp32) carried per cache slot
//   lgs_head_gate        per head: optional unit RMS of o, times act(g): the retention's output norm + silu gate and
//                        the latent attention's sigmoid gate
//   lgs_latent_prepare   latent attention, per token: RMS-normed latent c and the rotated shared key part go to the
//                        cache rows (slot, position); the queries' rotated parts are rotated in place (interleaved)
//   lgs_latent_attention softmax attention in the latent space: every head's query has been mapped through its key
//                        up-projection, so all heads read the same cached rows [c | k_rot]; scores, the sink's
//                        share of the denominator and the weighted sum of c are fp32; the value up-projection
//                        follows as a per-head product
#include "seq_common.h"

namespace lgs {

// ------------------------------------------------------------------------------------------------ retention
struct RetArgs {
  const float* q;  // row t, head h at q[t * ld + h * d]
  const float* k;
  const float* v;  // v[t * ld + h * dv]
  long ld;
  float* state;          // [slots][H][d][dv]
  const float* decay;    // [H]
  const float* inv_freq; // [rot_dims / 2]
  const int* seq_start;  // [B + 1] rows
  const int* seq_slot;   // [B]
  const int* seq_pos0;   // [B] position of the sequence's first row in this step
  float* out;            // [T][H * dv]
  int H, d, dv, rot_dims;
  float k_scale;
};

// grid (B, H, ceil(dv / 64)): a workgroup owns 64 columns of one head's state; wave w owns rows [w NR, (w + 1) NR)
template <int NR>
__global__ void __launch_bounds__(256) retention_scan_kernel(RetArgs p) {
  __shared__ float qs[256], ks[256];
  __shared__ float part[4][64];
  const int b = blockIdx.x, h = blockIdx.y, col = blockIdx.z * 64 + (threadIdx.x & 63);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, tid = threadIdx.x;
  const int d = p.d, dv = p.dv, half = p.rot_dims / 2;
  const int t0 = p.seq_start[b], t1 = p.seq_start[b + 1];
  const int pos0 = p.seq_pos0[b];
  const float lam = p.decay[h];
  const bool live = col < dv;
  float* sp = p.state + (((size_t)p.seq_slot[b] * p.H + h) * d) * dv + col;
  float S[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int row = wave * NR + i;
    S[i] = (pos0 > 0 && live && row < d) ? sp[(size_t)row * dv] : 0.0f;  // a sequence starts from the zero state
  }
  for (int t = t0; t < t1; ++t) {
    const float pos = (float)(pos0 + (t - t0));
    if (tid < d) {
      const float* qr = p.q + (size_t)t * p.ld + (size_t)h * d;
      const float* kr = p.k + (size_t)t * p.ld + (size_t)h * d;
      float qo = qr[tid], ko = kr[tid];
      if (tid < p.rot_dims) {
        const int j = tid < half ? tid : tid - half;
        float sn, cs;
        sincosf(pos * p.inv_freq[j], &sn, &cs);
        if (tid < half) {
          qo = qo * cs - qr[tid + half] * sn;
          ko = ko * cs - kr[tid + half] * sn;
        } else {
          qo = qo * cs + qr[tid - half] * sn;
          ko = ko * cs + kr[tid - half] * sn;
        }
      }
      qs[tid] = qo;
      ks[tid] = ko * p.k_scale;
    }
    __syncthreads();
    const float vt = live ? p.v[(size_t)t * p.ld + (size_t)h * dv + col] : 0.0f;
    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = wave * NR + i;
      if (row < d) {
        S[i] = fmaf(lam, S[i], ks[row] * vt);
        o = fmaf(S[i], qs[row], o);
      }
    }
    part[wave][lane] = o;
    __syncthreads();
    if (wave == 0 && live)
      p.out[(size_t)t * p.H * dv + (size_t)h * dv + col] = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = wave * NR + i;
      if (row < d) sp[(size_t)row * dv] = S[i];
    }
  }
}

// grid (T, H): o[t][h][:] <- (unit ? o / rms(o) : o) * act(g[t * ldg + h * dv + :])
__global__ void __launch_bounds__(256) head_gate_kernel(float* __restrict__ o, const float* __restrict__ g, long ldg,
                                                        int H, int dv, int unit, float eps, int act) {
  __shared__ float red[4];
  const int t = blockIdx.x, h = blockIdx.y;
  float* orow = o + ((size_t)t * H + h) * dv;
  const float* grow = g + (size_t)t * ldg + (size_t)h * dv;
  float rstd = 1.0f;
  if (unit) {
    float ss = 0.0f;
    for (int i = threadIdx.x; i < dv; i += 256) ss = fmaf(orow[i], orow[i], ss);
    ss = block_sum_256(ss, red);
    rstd = 1.0f / sqrtf(ss / (float)dv + eps);
  }
  for (int i = threadIdx.x; i < dv; i += 256) orow[i] = orow[i] * rstd * act_f(act, grow[i]);
}

// ------------------------------------------------------------------------------------------------ latent attention
struct LatPrepArgs {
  float* proj;  // row t: queries at q_off (head h at h * (d + dr): d unrotated, dr rotated), latent row at kv_off
  long ld;
  int q_off, kv_off;
  void* cache_c;    // [slots][S][r] bf16 or fp32
  float* cache_kr;  // [slots][S][dr]
  const float* norm_w;    // [r]
  const float* inv_freq;  // [rot_dims / 2]
  const int* slot;        // [T]
  const int* pos;         // [T]
  int H, d, dr, r, rot_dims, max_seq;
  float eps;
};

template <bool CF32>
__global__ void __launch_bounds__(256) latent_prepare_kernel(LatPrepArgs p) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int ps = p.pos[t];
  if (ps < 0 || ps >= p.max_seq) return;  // the host sizes the cache; never write out of bounds
  float* row = p.proj + (size_t)t * p.ld;
  const float* kv = row + p.kv_off;
  const size_t crow = (size_t)p.slot[t] * p.max_seq + ps;
  float ss = 0.0f;
  for (int i = tid; i < p.r; i += 256) ss = fmaf(kv[i], kv[i], ss);
  ss = block_sum_256(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)p.r + p.eps);
  for (int i = tid; i < p.r; i += 256) {
    const float c = kv[i] * rstd * p.norm_w[i];
    if (CF32) ((float*)p.cache_c)[crow * p.r + i] = c;
    else ((uint16_t*)p.cache_c)[crow * p.r + i] = f2bf(c);
  }
  const float fpos = (float)ps;
  const int half = p.rot_dims / 2;
  float* kro = p.cache_kr + crow * p.dr;
  for (int i = tid; i < p.dr; i += 256) {
    if (i >= p.rot_dims) kro[i] = kv[p.r + i];
    else if ((i & 1) == 0) {
      float sn, cs;
      sincosf(fpos * p.inv_freq[i >> 1], &sn, &cs);
      const float u = kv[p.r + i], v = kv[p.r + i + 1];
      kro[i] = u * cs - v * sn;
      kro[i + 1] = v * cs + u * sn;
    }
  }
  for (int it = tid; it < p.H * half; it += 256) {
    const int h = it / half, i = it % half;
    float* qr = row + p.q_off + (size_t)h * (p.d + p.dr) + p.d + 2 * i;
    float sn, cs;
    sincosf(fpos * p.inv_freq[i], &sn, &cs);
    const float u = qr[0], v = qr[1];
    qr[0] = u * cs - v * sn;
    qr[1] = v * cs + u * sn;
  }
}

struct LatAttArgs {
  const float* qc;    // [T][H][r] queries mapped into the latent space
  const float* proj;  // rotated query part of head h at proj[t * ld + q_off + h * (d + dr) + d]
  long ld;
  int q_off;
  const void* cache_c;
  const float* cache_kr;
  const float* sink;  // [H] or null
  const int* slot;
  const int* pos;
  float* out;  // [T][H][r]
  int H, d, dr, r, max_seq;
  float scale;
};

// grid (T, H): wave w walks keys w, w + 4, ... <= pos with an online softmax; lanes hold dims lane + 64 e
template <bool CF32, int NR>
__global__ void __launch_bounds__(256) latent_attention_kernel(LatAttArgs p) {
  __shared__ float sm[4], sl[4];
  extern __shared__ float sacc[];  // [4][r]
  const int t = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = p.r, dr = p.dr;
  const int last = min(p.pos[t], p.max_seq - 1);
  const size_t base = (size_t)p.slot[t] * p.max_seq;
  const float* qc = p.qc + ((size_t)t * p.H + h) * r;
  const float* qr = p.proj + (size_t)t * p.ld + p.q_off + (size_t)h * (p.d + dr) + p.d;
  float q[NR], qrot[2], acc[NR];
#pragma unroll
  for (int e = 0; e < NR; ++e) {
    q[e] = lane + 64 * e < r ? qc[lane + 64 * e] : 0.0f;
    acc[e] = 0.0f;
  }
#pragma unroll
  for (int e = 0; e < 2; ++e) qrot[e] = lane + 64 * e < dr ? qr[lane + 64 * e] : 0.0f;
  float m = -INFINITY, l = 0.0f;
  for (int j = wave; j <= last; j += 4) {
    float c[NR];
    float dot = 0.0f;
#pragma unroll
    for (int e = 0; e < NR; ++e) {
      const int i = lane + 64 * e;
      c[e] = i < r ? (CF32 ? ((const float*)p.cache_c)[(base + j) * r + i]
                           : bf2f(((const uint16_t*)p.cache_c)[(base + j) * r + i]))
                   : 0.0f;
      dot = fmaf(q[e], c[e], dot);
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int i = lane + 64 * e;
      if (i < dr) dot = fmaf(qrot[e], p.cache_kr[(base + j) * dr + i], dot);
    }
    const float s = wave_sum(dot) * p.scale;
    const float mn = fmaxf(m, s);
    const float corr = expf(m - mn), w = expf(s - mn);
    l = l * corr + w;
#pragma unroll
    for (int e = 0; e < NR; ++e) acc[e] = acc[e] * corr + w * c[e];
    m = mn;
  }
  if (lane == 0) {
    sm[wave] = m;
    sl[wave] = l;
  }
#pragma unroll
  for (int e = 0; e < NR; ++e)
    if (lane + 64 * e < r) sacc[wave * r + lane + 64 * e] = acc[e];
  __syncthreads();
  const float snk = p.sink ? p.sink[h] : -INFINITY;
  const float mx = fmaxf(fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3])), snk);
  float f[4], den = p.sink ? expf(snk - mx) : 0.0f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = sl[w] > 0.0f ? expf(sm[w] - mx) : 0.0f;
    den += sl[w] * f[w];
  }
  float* o = p.out + ((size_t)t * p.H + h) * r;
  for (int i = threadIdx.x; i < r; i += 256)
    o[i] = ((sacc[i] * f[0] + sacc[r + i] * f[1]) + (sacc[2 * r + i] * f[2] + sacc[3 * r + i] * f[3])) / den;
}

}  // namespace lgs

extern "C" int lgs_retention(const float* q, const float* k, const float* v, long ld, float* state, const float* decay,
                             const float* inv_freq, const int* seq_start, const int* seq_slot, const int* seq_pos0,
                             float* out, int B, int H, int d, int dv, int rot_dims, float k_scale,
                             hipStream_t stream) {
  LGA_CHECK_ARG(q && k && v && state && decay && seq_start && seq_slot && seq_pos0 && out, "lgs_retention: null pointer");
  LGA_CHECK_ARG(B > 0 && H > 0 && H <= 65535 && d > 0 && d <= 256 && dv > 0, "lgs_retention: head dim must be in [1, 256]");
  LGA_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= d && (rot_dims == 0 || inv_freq),
                "lgs_retention: bad rotary dims");
  lgs::RetArgs p{q, k, v, ld, state, decay, inv_freq, seq_start, seq_slot, seq_pos0, out, H, d, dv, rot_dims, k_scale};
  const dim3 grid(B, H, (dv + 63) / 64);
  if (d <= 64) lgs::retention_scan_kernel<16><<<grid, 256, 0, stream>>>(p);
  else if (d <= 128) lgs::retention_scan_kernel<32><<<grid, 256, 0, stream>>>(p);
  else lgs::retention_scan_kernel<64><<<grid, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_head_gate(float* o, const float* g, long ldg, int T, int H, int dv, int unit_norm, float eps,
                             int act, hipStream_t stream) {
  LGA_CHECK_ARG(o && g && T > 0 && H > 0 && H <= 65535 && dv > 0, "lgs_head_gate: bad arguments");
  lgs::head_gate_kernel<<<dim3(T, H), 256, 0, stream>>>(o, g, ldg, H, dv, unit_norm, eps, act);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_latent_prepare(float* proj, long ld, int q_off, int kv_off, void* cache_c, int cache_f32,
                                  float* cache_kr, const float* norm_w, const float* inv_freq, const int* slot,
                                  const int* pos, int T, int H, int d, int dr, int r, int rot_dims, int max_seq,
                                  float eps, hipStream_t stream) {
  LGA_CHECK_ARG(proj && cache_c && cache_kr && norm_w && slot && pos, "lgs_latent_prepare: null pointer");
  LGA_CHECK_ARG(T > 0 && H > 0 && d >= 0 && dr >= 0 && r > 0 && max_seq > 0, "lgs_latent_prepare: bad sizes");
  LGA_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dr && (rot_dims == 0 || inv_freq),
                "lgs_latent_prepare: bad rotary dims");
  lgs::LatPrepArgs p{proj, ld, q_off, kv_off, cache_c, cache_kr, norm_w, inv_freq, slot, pos,
                     H, d, dr, r, rot_dims, max_seq, eps};
  if (cache_f32) lgs::latent_prepare_kernel<true><<<T, 256, 0, stream>>>(p);
  else lgs::latent_prepare_kernel<false><<<T, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_latent_attention(const float* qc, const float* proj, long ld, int q_off, const void* cache_c,
                                    int cache_f32, const float* cache_kr, const float* sink, const int* slot,
                                    const int* pos, float* out, int T, int H, int d, int dr, int r, int max_seq,
                                    float scale, hipStream_t stream) {
  LGA_CHECK_ARG(qc && proj && cache_c && cache_kr && slot && pos && out, "lgs_latent_attention: null pointer");
  LGA_CHECK_ARG(T > 0 && H > 0 && H <= 65535 && r > 0 && r <= 512 && dr >= 0 && dr <= 128 && max_seq > 0,
                "lgs_latent_attention: latent rank must be <= 512 and the rotated part <= 128");
  lgs::LatAttArgs p{qc, proj, ld, q_off, cache_c, cache_kr, sink, slot, pos, out, H, d, dr, r, max_seq, scale};
  const dim3 grid(T, H);
  const size_t lds = (size_t)4 * r * sizeof(float);
#define LGS_LAT(NR)                                                                              \
  do {                                                                                           \
    if (cache_f32) lgs::latent_attention_kernel<true, NR><<<grid, 256, lds, stream>>>(p);        \
    else lgs::latent_attention_kernel<false, NR><<<grid, 256, lds, stream>>>(p);                 \
  } while (0)
  if (r <= 128) LGS_LAT(2);
  else if (r <= 256) LGS_LAT(4);
  else LGS_LAT(8);
#undef LGS_LAT
  LGA_LAUNCH_RETURN();
}

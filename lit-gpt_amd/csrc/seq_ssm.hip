// Selective state-space mixer (Mamba-2 form) of the layered models; everything that enters the recurrence is fp32.
//
//   lgs_conv_silu        per-channel causal convolution over a packed batch + bias + silu; the last taps - 1 inputs
//                        of every sequence are part of its state (a slot-indexed buffer) and are read at the start
//                        of a step that continues a sequence and rewritten at its end
//   lgs_ssm_scan         per head: dt = softplus(raw + bias), a = exp(-exp(A_log) dt),
//                        S <- a S + dt B x^T (S is N x dv, fp32, one per cache slot), y = S^T C + D x;
//                        heads share B and C in groups. Token by token (decode, short portions), or for prompts
//                        in chunks of 64 tokens as fp32 matrix products with the chunks side by side
//   lgs_gated_group_norm out = unit_rms_per_group(y * silu(z)) * w: gating first, the grouped norm on the gated values
#include "seq_common.h"

namespace lgs {

constexpr int kMaxTaps = 16;
constexpr int kConvTile = 16;  // tokens per workgroup (>= kMaxTaps - 1: only a sequence's first tile reads the state)

struct ConvArgs {
  const float* u;  // [T][ld] inputs (the channels start at u)
  long ld;
  const void* w;   // [C][taps]
  const void* b;   // [C]
  float* state;    // [slots][taps - 1][C]: the inputs at the last taps - 1 positions, oldest first
  const int *seq_start, *seq_slot, *seq_pos0;
  float* out;      // [T][C]
  int C, taps;
};

__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// grid (ceil(C / 256), tiles, B): thread = channel; tile = kConvTile consecutive tokens of sequence b. The first
// tile of a sequence reads the stored inputs (unless the sequence starts at position 0: then they count as zeros)
// and, after it, writes the inputs that the step leaves behind.
template <bool WF32>
__global__ void __launch_bounds__(256) conv_silu_kernel(ConvArgs p) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int b = blockIdx.z;
  const int r0 = p.seq_start[b], n = p.seq_start[b + 1] - r0;
  const int first = blockIdx.y * kConvTile;
  if (c >= p.C || first >= n) return;
  const int taps = p.taps, hist = taps - 1;
  const int pos0 = p.seq_pos0[b];
  float* st = p.state + (size_t)p.seq_slot[b] * hist * p.C + c;
  // the window's last entry is the current token; weights are aligned to it (zeros in front of the first tap)
  float w[kMaxTaps], win[kMaxTaps];
#pragma unroll
  for (int k = 0; k < kMaxTaps; ++k) {
    w[kMaxTaps - 1 - k] = k < taps ? wload<WF32>(p.w, (size_t)c * taps + (taps - 1 - k)) : 0.0f;
    float v = 0.0f;  // the input k tokens before the tile's first
    if (k >= 1 && k <= hist) {
      const int src = first - k;  // relative to the sequence's first row of this step
      if (src >= 0) v = p.u[(size_t)(r0 + src) * p.ld + c];
      else if (pos0 + src >= 0) v = st[(size_t)(hist + src) * p.C];  // (first == 0 here: the stored inputs)
    }
    win[kMaxTaps - 1 - k] = v;
  }
  const float bias = wload<WF32>(p.b, c);
  const int last = min(first + kConvTile, n);
  for (int i = first; i < last; ++i) {
    win[kMaxTaps - 1] = p.u[(size_t)(r0 + i) * p.ld + c];
    float acc = bias;
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) acc = fmaf(w[j], win[j], acc);
    p.out[(size_t)(r0 + i) * p.C + c] = acc / (1.0f + expf(-acc));
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j) win[j] = win[j + 1];
  }
  if (first == 0) {
    // what the step leaves behind: the inputs at positions pos0 + n - hist + j. A stored input is read at a higher
    // index than any written before it, so ascending order works in place.
    for (int j = 0; j < hist; ++j) {
      const int src = n - hist + j;
      float v = 0.0f;
      if (src >= 0) v = p.u[(size_t)(r0 + src) * p.ld + c];
      else if (pos0 + src >= 0) v = st[(size_t)(hist + src) * p.C];
      st[(size_t)j * p.C] = v;
    }
  }
}

struct ScanArgs {
  const float* xbc;  // [T][ldx]: x (heads * dv) | B (groups * N) | C (groups * N) after the convolution
  long ldx;
  const float* dt;   // [T][ldd] raw step sizes, one per head (at dt)
  long ldd;
  const float *dt_bias, *A_log, *D;  // [heads]
  float* state;      // [slots][heads][N][dv]
  const int *seq_start, *seq_slot, *seq_pos0;
  float* y;          // [T][heads * dv]
  int heads, groups, N, dv;
};

constexpr int kScanBatch = 8;  // tokens between two barriers

// grid (ceil(dv / 64), heads, B): a workgroup owns 64 columns of one head's state; wave w owns the state rows
// [w NR, (w + 1) NR), lane = column. Tokens are taken kScanBatch at a time: every wave advances its rows through the
// batch and leaves its share of each token's output in LDS; wave 0 sums the four shares in a fixed order.
template <int NR>
__global__ void __launch_bounds__(256) ssm_scan_kernel(ScanArgs p) {
  __shared__ float part[4][kScanBatch][64];
  __shared__ float sdt[kScanBatch], sa[kScanBatch];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int hd = blockIdx.y, b = blockIdx.z;
  const int col = blockIdx.x * 64 + lane;
  const bool live = col < p.dv;
  const int N = p.N, dv = p.dv, H = p.heads;
  const int g = hd / (H / p.groups);
  const int r0 = p.seq_start[b], n = p.seq_start[b + 1] - r0;
  const int inner = H * dv;
  float* st = p.state + (((size_t)p.seq_slot[b] * H + hd) * N) * dv;
  const int n0 = wave * NR;
  float S[NR];
  const bool fresh = p.seq_pos0[b] == 0;
#pragma unroll
  for (int i = 0; i < NR; ++i) S[i] = (!fresh && live && n0 + i < N) ? st[(size_t)(n0 + i) * dv + col] : 0.0f;
  const float bias = p.dt_bias[hd], rate = expf(p.A_log[hd]), Dh = p.D[hd];
  for (int t0 = 0; t0 < n; t0 += kScanBatch) {
    const int nb = min(kScanBatch, n - t0);
    if (threadIdx.x < nb) {
      const float d = softplus_f(p.dt[(size_t)(r0 + t0 + threadIdx.x) * p.ldd + hd] + bias);
      sdt[threadIdx.x] = d;
      sa[threadIdx.x] = expf(-rate * d);
    }
    __syncthreads();
    for (int t = 0; t < nb; ++t) {
      const float* row = p.xbc + (size_t)(r0 + t0 + t) * p.ldx;
      const float d = sdt[t], a = sa[t];
      const float dx = live ? d * row[hd * dv + col] : 0.0f;
      const float* Bt = row + inner + g * N + n0;
      const float* Ct = row + inner + p.groups * N + g * N + n0;
      float acc = 0.0f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        if (n0 + i < N) {
          S[i] = fmaf(a, S[i], Bt[i] * dx);
          acc = fmaf(S[i], Ct[i], acc);
        }
      }
      part[wave][t][lane] = acc;
    }
    __syncthreads();
    if (wave == 0 && live) {
      for (int t = 0; t < nb; ++t) {
        const size_t r = (size_t)(r0 + t0 + t);
        const float x = p.xbc[r * p.ldx + hd * dv + col];
        const float v = (part[0][t][lane] + part[1][t][lane]) + (part[2][t][lane] + part[3][t][lane]);
        p.y[r * inner + hd * dv + col] = fmaf(Dh, x, v);
      }
    }
    // (the next batch's writes to `part` come after its first barrier, which wave 0 reaches after these reads)
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (n0 + i < N) st[(size_t)(n0 + i) * dv + col] = S[i];
  }
}

// The prompt form of the scan: chunks of 64 tokens as fp32 matrix products (v_mfma_f32_16x16x4_f32), all chunks of
// all sequences side by side. With l_i the running sum of log a over the chunk's tokens up to i, S0 the state at the
// chunk's start and n its token count:
//   y_i = exp(l_i) C_i^T S0 + sum_{j <= i} exp(l_i - l_j) dt_j (C_i . B_j) x_j + D x_i
//   S'  = exp(l_{n-1}) S0 + sum_j exp(l_{n-1} - l_j) dt_j B_j x_j^T
// MODE 1, grid (B * max_chunks, heads, ceil(dv / 64)): the second term of S' of every chunk -> workspace, the chunk's
// whole decay -> wdec. ssd_carry_kernel turns these into the state at each chunk's start (an elementwise recurrence
// over the chunks, which also leaves the final state in the slot). MODE 2: the outputs of every chunk.
// LDS (floats): C, B [64][NP + 4], x [64][80], scores [64][66], l, dt, weights [64] each; N <= 128.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
constexpr int kSC = 64, kXS = 80, kGS = 66;

struct SsdArgs {
  const float* xbc;
  long ldx;
  const float* dt;
  long ldd;
  const float *dt_bias, *A_log, *D;
  float* state;
  const int *seq_start, *seq_slot, *seq_pos0;
  float* y;
  float* ws;    // [B * max_chunks][heads][N][dv]
  float* wdec;  // [B * max_chunks][heads]
  int heads, groups, N, dv, max_chunks;
};

template <int MODE>
__global__ void __launch_bounds__(256) ssd_chunk_kernel(SsdArgs p) {
  extern __shared__ float lds[];
  const int b = blockIdx.x / p.max_chunks, cidx = blockIdx.x % p.max_chunks;
  const int h = blockIdx.y, col0 = blockIdx.z * 64;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int t0 = p.seq_start[b], t1 = p.seq_start[b + 1];
  const int tc = t0 + cidx * kSC;
  if (tc >= t1) return;
  const int n = min(kSC, t1 - tc);
  const int N = p.N, dv = p.dv, H = p.heads, inner = H * dv;
  const int g = h / (H / p.groups);
  const int NP = (N + 15) / 16 * 16, NS = NP + 4;
  float* Cs = lds;
  float* Bs = Cs + kSC * NS;
  float* Xs = Bs + kSC * NS;
  float* Gs = Xs + kSC * kXS;
  float* la = Gs + kSC * kGS;
  float* dts = la + kSC;
  float* wgt = dts + kSC;
  const int fr = lane & 15, fk = lane >> 4;
  const size_t tile = ((size_t)blockIdx.x * H + h) * N * dv;
  // MODE 2: this lane's share of the state at the chunk's start (the B operand of C S0), fetched before anything
  // else so that its latency passes under the staging and the score product (one wave per SIMD: nothing else hides it)
  float sv[32][4];
  if (MODE == 2) {
#pragma unroll
    for (int kk = 0; kk < 32; ++kk)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int krow = kk * 4 + fk, col = col0 + c * 16 + fr;
        sv[kk][c] = (krow < N && col < dv) ? p.ws[tile + (size_t)krow * dv + col] : 0.0f;
      }
  }
  if (wave == 0) {
    float d = 0.0f, l = 0.0f;
    if (lane < n) {
      d = softplus_f(p.dt[(size_t)(tc + lane) * p.ldd + h] + p.dt_bias[h]);
      l = -expf(p.A_log[h]) * d;
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float v = __shfl_up(l, o);
      if (lane >= o) l += v;
    }
    la[lane] = l;
    dts[lane] = d;
  }
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  if (((N | dv | inner) & 3) == 0 && (p.ldx & 3) == 0) {  // 16-byte loads and LDS stores (NS is a multiple of 4)
    const int q = NP / 4;
    for (int i = tid; i < kSC * q; i += 256) {
      const int row = i / q, k = (i - row * q) * 4;
      const bool in = row < n && k < N;
      const float* at = p.xbc + (size_t)(tc + row) * p.ldx + inner + (size_t)g * N + k;
      *(float4*)(Bs + row * NS + k) = in ? *(const float4*)at : zero4;
      if (MODE == 2) *(float4*)(Cs + row * NS + k) = in ? *(const float4*)(at + (size_t)p.groups * N) : zero4;
    }
    for (int i = tid; i < kSC * 16; i += 256) {
      const int row = i >> 4, c = (i & 15) * 4;
      const bool in = row < n && col0 + c < dv;
      *(float4*)(Xs + row * kXS + c) =
          in ? *(const float4*)(p.xbc + (size_t)(tc + row) * p.ldx + (size_t)h * dv + col0 + c) : zero4;
    }
  } else {
    for (int i = tid; i < kSC * NP; i += 256) {
      const int row = i / NP, k = i - row * NP;
      const bool in = row < n && k < N;
      const size_t at = (size_t)(tc + row) * p.ldx + inner + (size_t)g * N + k;
      Bs[row * NS + k] = in ? p.xbc[at] : 0.0f;
      if (MODE == 2) Cs[row * NS + k] = in ? p.xbc[at + (size_t)p.groups * N] : 0.0f;
    }
    for (int i = tid; i < kSC * 64; i += 256) {
      const int row = i >> 6, c = i & 63;
      Xs[row * kXS + c] = (row < n && col0 + c < dv) ? p.xbc[(size_t)(tc + row) * p.ldx + (size_t)h * dv + col0 + c] : 0.0f;
    }
  }
  __syncthreads();
  if (MODE == 1) {
    const float lal = la[n - 1];
    if (tid < kSC) wgt[tid] = tid < n ? expf(lal - la[tid]) * dts[tid] : 0.0f;
    __syncthreads();
    for (int td = wave; td < NP / 16; td += 4) {
      f32x4_t s[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) s[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
      for (int k = 0; k < kSC; k += 4) {
        const int j = k + fk;
        const float a = Bs[j * NS + td * 16 + fr] * wgt[j];
#pragma unroll
        for (int c = 0; c < 4; ++c)
          s[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Xs[j * kXS + c * 16 + fr], s[c], 0, 0, 0);
      }
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = td * 16 + fk * 4 + r, col = col0 + c * 16 + fr;
          if (row < N && col < dv) p.ws[tile + (size_t)row * dv + col] = s[c][r];
        }
    }
    if (tid == 0 && blockIdx.z == 0) p.wdec[(size_t)blockIdx.x * H + h] = expf(lal);
    return;
  }
  // ---- MODE 2: wave w owns tokens 16 w .. 16 w + 15
  const int ti = wave;
  {
    f32x4_t acc[4];
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) acc[tj] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const float* qa = Cs + (ti * 16 + fr) * NS + fk;
    const float* kb = Bs + fr * NS + fk;
#pragma unroll 2
    for (int k = 0; k < NP; k += 4) {
      const float a = qa[k];
#pragma unroll
      for (int tj = 0; tj < 4; ++tj)
        if (tj <= ti) acc[tj] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, kb[tj * 16 * NS + k], acc[tj], 0, 0, 0);
    }
#pragma unroll
    for (int tj = 0; tj < 4; ++tj)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = ti * 16 + fk * 4 + r, j = tj * 16 + fr;
        Gs[i * kGS + j] = j <= i ? acc[tj][r] * expf(la[i] - la[j]) * dts[j] : 0.0f;
      }
  }
  f32x4_t o[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) o[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kk = 0; kk < 32; ++kk) {
    if (kk * 4 < NP) {
      const float a = Cs[(ti * 16 + fr) * NS + kk * 4 + fk];
#pragma unroll
      for (int c = 0; c < 4; ++c) o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, sv[kk][c], o[c], 0, 0, 0);
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r) o[c][r] *= expf(la[ti * 16 + fk * 4 + r]);
  __syncthreads();
#pragma unroll 4
  for (int k = 0; k < (ti + 1) * 16; k += 4) {
    const float a = Gs[(ti * 16 + fr) * kGS + k + fk];
#pragma unroll
    for (int c = 0; c < 4; ++c)
      o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Xs[(k + fk) * kXS + c * 16 + fr], o[c], 0, 0, 0);
  }
  const float Dh = p.D[h];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = ti * 16 + fk * 4 + r, col = col0 + c * 16 + fr;
      if (i < n && col < dv)
        p.y[(size_t)(tc + i) * inner + (size_t)h * dv + col] = fmaf(Dh, Xs[i * kXS + c * 16 + fr], o[c][r]);
    }
}

// grid (B, heads, ceil(N dv / 256)): one state element per thread walks its sequence's chunks: the workspace's local
// sums become the states at the chunks' starts, and the state after the last chunk goes back to the slot
__global__ void __launch_bounds__(256) ssd_carry_kernel(SsdArgs p) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  const int nd = p.N * p.dv;
  if (e >= nd) return;
  const int chunks = (p.seq_start[b + 1] - p.seq_start[b] + kSC - 1) / kSC;
  float* st = p.state + ((size_t)p.seq_slot[b] * p.heads + h) * nd + e;
  float s = p.seq_pos0[b] > 0 ? *st : 0.0f;
  for (int c = 0; c < chunks; ++c) {
    const size_t idx = ((size_t)b * p.max_chunks + c) * p.heads + h;
    const float local = p.ws[idx * nd + e];
    p.ws[idx * nd + e] = s;
    s = fmaf(p.wdec[idx], s, local);
  }
  *st = s;
}

static size_t ssd_lds(int N) {
  const int NP = (N + 15) / 16 * 16;
  return sizeof(float) * ((size_t)2 * kSC * (NP + 4) + kSC * kXS + kSC * kGS + 3 * kSC);
}

// grid (T, groups): out[t][g n + i] = v / sqrt(mean_g(v^2) + eps) * w[g n + i], v = y * silu(z)
__global__ void __launch_bounds__(256) gated_group_norm_kernel(const float* __restrict__ y, const float* __restrict__ z,
                                                               long ldz, const float* __restrict__ w, float eps,
                                                               float* __restrict__ out, uint16_t* __restrict__ out16,
                                                               int n, int inner) {
  __shared__ float red[4];
  const size_t t = blockIdx.x;
  const int c0 = blockIdx.y * n;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float zz = z[t * ldz + c0 + i];
    const float v = y[t * inner + c0 + i] * (zz / (1.0f + expf(-zz)));
    out[t * inner + c0 + i] = v;
    ss = fmaf(v, v, ss);
  }
  ss = block_sum_256(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = out[t * inner + c0 + i] * rstd * w[c0 + i];
    out[t * inner + c0 + i] = v;
    if (out16) out16[t * inner + c0 + i] = f2bf(v);
  }
}

}  // namespace lgs

extern "C" int lgs_conv_silu(const float* u, long ld, const void* w, const void* bias, int w_f32, float* state,
                             const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out, int B,
                             int max_len, int C, int taps, hipStream_t stream) {
  LGA_CHECK_ARG(u && w && bias && state && seq_start && seq_slot && seq_pos0 && out, "lgs_conv_silu: null pointer");
  LGA_CHECK_ARG(B > 0 && B <= 65535 && max_len > 0 && C > 0 && ld >= C, "lgs_conv_silu: bad sizes");
  LGA_CHECK_ARG(taps >= 1 && taps <= lgs::kMaxTaps, "lgs_conv_silu: 1 to 16 taps");
  lgs::ConvArgs p{u, ld, w, bias, state, seq_start, seq_slot, seq_pos0, out, C, taps};
  const int tiles = (max_len + lgs::kConvTile - 1) / lgs::kConvTile;
  LGA_CHECK_ARG(tiles <= 65535, "lgs_conv_silu: a sequence brings too many tokens to one step");
  const dim3 grid((C + 255) / 256, tiles, B);
  if (w_f32) lgs::conv_silu_kernel<true><<<grid, 256, 0, stream>>>(p);
  else lgs::conv_silu_kernel<false><<<grid, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_ssm_scan(const float* xbc, long ldx, const float* dt, long ldd, const float* dt_bias,
                            const float* A_log, const float* D, float* state, const int* seq_start,
                            const int* seq_slot, const int* seq_pos0, float* y, int B, int heads, int groups, int N,
                            int dv, float* ws, float* wdec, int max_chunks, hipStream_t stream) {
  LGA_CHECK_ARG(xbc && dt && dt_bias && A_log && D && state && seq_start && seq_slot && seq_pos0 && y,
                "lgs_ssm_scan: null pointer");
  LGA_CHECK_ARG(B > 0 && B <= 65535 && heads > 0 && heads <= 65535 && groups > 0 && heads % groups == 0,
                "lgs_ssm_scan: heads must be a multiple of the groups");
  LGA_CHECK_ARG(N > 0 && N <= 256 && dv > 0, "lgs_ssm_scan: state size 1 to 256");
  LGA_CHECK_ARG(ldx >= (long)heads * dv + 2L * groups * N && ldd >= heads, "lgs_ssm_scan: rows shorter than their parts");
  if (ws) {  // the prompt form
    LGA_CHECK_ARG(wdec && max_chunks > 0 && N <= 128, "lgs_ssm_scan: the prompt form serves state sizes up to 128");
    LGA_CHECK_ARG((long)B * max_chunks < (1L << 31) && (dv + 63) / 64 <= 65535, "lgs_ssm_scan: too many chunks");
    lgs::SsdArgs p{xbc, ldx, dt, ldd, dt_bias, A_log, D, state, seq_start, seq_slot, seq_pos0, y, ws, wdec,
                   heads, groups, N, dv, max_chunks};
    const size_t lds = lgs::ssd_lds(N);
    for (auto* fn : {lgs::ssd_chunk_kernel<1>, lgs::ssd_chunk_kernel<2>}) {
      const hipError_t e = hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) {
        lga_set_error(hipGetErrorString(e));
        return (int)e;
      }
    }
    const dim3 grid(B * max_chunks, heads, (dv + 63) / 64);
    lgs::ssd_chunk_kernel<1><<<grid, 256, lds, stream>>>(p);
    lgs::ssd_carry_kernel<<<dim3(B, heads, (N * dv + 255) / 256), 256, 0, stream>>>(p);
    lgs::ssd_chunk_kernel<2><<<grid, 256, lds, stream>>>(p);
    LGA_LAUNCH_RETURN();
  }
  lgs::ScanArgs p{xbc, ldx, dt, ldd, dt_bias, A_log, D, state, seq_start, seq_slot, seq_pos0, y, heads, groups, N, dv};
  const dim3 grid((dv + 63) / 64, heads, B);
  const int nr = (N + 3) / 4;
  if (nr <= 8) lgs::ssm_scan_kernel<8><<<grid, 256, 0, stream>>>(p);
  else if (nr <= 16) lgs::ssm_scan_kernel<16><<<grid, 256, 0, stream>>>(p);
  else if (nr <= 32) lgs::ssm_scan_kernel<32><<<grid, 256, 0, stream>>>(p);
  else lgs::ssm_scan_kernel<64><<<grid, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_gated_group_norm(const float* y, const float* z, long ldz, const float* w, float eps, float* out,
                                    void* out_bf16, int T, int inner, int groups, hipStream_t stream) {
  LGA_CHECK_ARG(y && z && w && out && T > 0 && inner > 0, "lgs_gated_group_norm: bad arguments");
  LGA_CHECK_ARG(groups > 0 && groups <= 65535 && inner % groups == 0,
                "lgs_gated_group_norm: inner must divide into the groups");
  lgs::gated_group_norm_kernel<<<dim3(T, groups), 256, 0, stream>>>(y, z, ldz, w, eps, out, (uint16_t*)out_bf16,
                                                                   inner / groups, inner);
  LGA_LAUNCH_RETURN();
}

// Kernels of the mixers with a recurrent state (the Mamba-2 state-space layer, the gated delta rule), of the
// short causal convolution in front of them, and of the element-wise steps around them: Dynamic Tanh, the
// scaled residual add, a gated linear unit's activation, the gated RMS norm in groups, the mean of RMS-normed
// branches.  Everything is 32-bit arithmetic; only an output that feeds a matrix product is rounded to the run's
// dtype.
//
// The scans walk a sequence's tokens in order, one workgroup a (sequence, head, slice of the head's columns),
// the state in registers, and are the same kernel for a prompt and for single tokens: a token's result is made of
// the same operations in the same order however the sequence was cut into steps and whatever else is in the batch.
#include "common.h"

namespace {

__device__ inline float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ inline float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ inline float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ inline float gelu_tanh_f(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

__device__ inline float gelu_erf_f(float z) { return 0.5f * z * (1.f + erff(z * 0.70710678118654752f)); }

enum { ACT_NONE = 0, ACT_SILU = 1, ACT_RELU = 2, ACT_GELU_TANH = 3, ACT_GELU_ERF = 4 };

__device__ inline float activate(float z, int act) {
  switch (act) {
    case ACT_SILU: return silu_f(z);
    case ACT_RELU: return fmaxf(z, 0.f);
    case ACT_GELU_TANH: return gelu_tanh_f(z);
    case ACT_GELU_ERF: return gelu_erf_f(z);
    default: return z;
  }
}

template <typename T>
__device__ inline void store_as(T* p, float v);
template <>
__device__ inline void store_as<float>(float* p, float v) { *p = v; }
template <>
__device__ inline void store_as<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// ---------------------------------------------------------------- Dynamic Tanh and the scaled add
// (x += scale * (piece 0 + piece 1 + ...);)  out = tanh(alpha x) w + b
template <typename T>
__global__ __launch_bounds__(256) void dynamic_tanh_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                                           int pieces, long long piece_stride, float scale,
                                                           const float* __restrict__ w, const float* __restrict__ b,
                                                           const float* __restrict__ alpha, T* __restrict__ out,
                                                           long long n, int width) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float v = x[i];
  if (pieces > 0) {
    float d = delta[i];
    for (int p = 1; p < pieces; ++p) d += delta[i + p * piece_stride];
    v += scale * d;
    x[i] = v;
  }
  const int c = (int)(i % width);
  store_as<T>(out + i, tanhf(alpha[0] * v) * w[c] + b[c]);
}

__global__ __launch_bounds__(256) void add_scaled_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                                         int pieces, long long piece_stride, float scale, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float d = delta[i];
  for (int p = 1; p < pieces; ++p) d += delta[i + p * piece_stride];
  x[i] += scale * d;
}

// out[r, c] = act(gu[r, c] + bias[c]) * (gu[r, I + c] + bias[I + c]); behind the I results `tail` more columns, a
// one and then zeros: with the next product's bias as one more column of its weight, that product adds the bias itself.
// `row_gate` (a logit a row, stride ldrg): the row's results times its sigmoid.  `gated` 0: there is no up half,
// out[r, c] = act(gu[r, c]).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void glu_kernel(const TI* __restrict__ gu, int ld, TO* __restrict__ out, int ldo,
                                                  int I, int act, const float* __restrict__ bias, int tail,
                                                  const float* __restrict__ row_gate, int ldrg, int gated) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= I + tail) return;
  if (c >= I) {
    store_as<TO>(out + (long long)r * ldo + c, c == I ? 1.f : 0.f);
    return;
  }
  float g = to_f32(gu[(long long)r * ld + c]), u = gated ? to_f32(gu[(long long)r * ld + I + c]) : 1.f;
  if (bias != nullptr) g += bias[c], u += bias[I + c];
  if (row_gate != nullptr) u *= sigmoid_f(row_gate[(long long)r * ldrg]);
  store_as<TO>(out + (long long)r * ldo + c, activate(g, act) * u);
}

// out[r, c] = act(x[r, c]) for four neighbouring columns a thread (a 16-byte load, an 8- or 16-byte store): the plain
// activation between the two products of a feed-forward without a gate, whose rows are wide
template <typename TO>
__global__ __launch_bounds__(256) void activation4_kernel(const float* __restrict__ x, int ld, TO* __restrict__ out,
                                                          int ldo, int I, int act) {
  const int r = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (c >= I) return;
  const float4 v = *(const float4*)(x + (long long)r * ld + c);
  const float y0 = activate(v.x, act), y1 = activate(v.y, act), y2 = activate(v.z, act), y3 = activate(v.w, act);
  TO* o = out + (long long)r * ldo + c;
  if constexpr (sizeof(TO) == 2) {
    uint2 packed;
    packed.x = (uint32_t)f32_to_bf16(y0).bits | ((uint32_t)f32_to_bf16(y1).bits << 16);
    packed.y = (uint32_t)f32_to_bf16(y2).bits | ((uint32_t)f32_to_bf16(y3).bits << 16);
    *(uint2*)o = packed;
  } else {
    *(float4*)o = make_float4(y0, y1, y2, y3);
  }
}

// ---------------------------------------------------------------- short causal convolution
// y[t, c] = act(bias[c] + sum_j w[c, j] x[t - (taps - 1) + j, c]); inputs before this step's rows come from
// the sequence's state (its last taps - 1 inputs, zeros at the start of a sequence).
__global__ __launch_bounds__(256) void causal_conv_kernel(const float* __restrict__ x, int ldx,
                                                          const float* __restrict__ w, const float* __restrict__ bias,
                                                          const float* __restrict__ state, float* __restrict__ out,
                                                          int ldo, int C, int taps, const int* __restrict__ row_seq,
                                                          const int* __restrict__ row_pos,
                                                          const int* __restrict__ seq_slot,
                                                          const int* __restrict__ seq_start,
                                                          const int* __restrict__ cu_rows, int act) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int b = row_seq[r];
  const int since = row_pos[r] - seq_start[b];  // rows of this step before this one, in its sequence
  const long long first = cu_rows[b];
  const float* st = state + (long long)seq_slot[b] * (taps - 1) * C;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;  // how many tokens before this one
    const float v = back <= since ? x[(first + since - back) * ldx + c] : st[(long long)(taps - 1 - (back - since)) * C + c];
    acc = fmaf(w[(long long)c * taps + j], v, acc);
  }
  if (bias != nullptr) acc += bias[c];
  out[(long long)r * ldo + c] = activate(acc, act);
}

// The state after the step: the last taps - 1 inputs of each sequence (old ones move up where the step brought fewer).
__global__ __launch_bounds__(256) void conv_state_kernel(const float* __restrict__ x, int ldx, float* __restrict__ state,
                                                         int C, int taps, const int* __restrict__ seq_slot,
                                                         const int* __restrict__ cu_rows) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const long long first = cu_rows[b];
  const int n_new = (int)(cu_rows[b + 1] - first);
  float* st = state + (long long)seq_slot[b] * (taps - 1) * C;
  for (int j = 0; j < taps - 1; ++j) {  // ascending: entry j is written after entry j + n_new was read
    const int src = j + n_new;
    st[(long long)j * C + c] = src < taps - 1 ? st[(long long)src * C + c] : x[(first + src - (taps - 1)) * ldx + c];
  }
}

// ---------------------------------------------------------------- the scans
// A head's state is [columns P][state size N] in memory.  A thread owns, of one column, the entries n = i LN + l
// (i = 0 .. slab - 1): LN threads share a column, LN the power of two with slab = ceil(N / LN) <= 8 (16 for states
// beyond 512), which depends on the model's sizes only.  Sums over n are a thread's own entries in ascending i, then
// an exchange over the LN lanes.  What the columns of a workgroup share of a token (B and C or q and k, the
// workgroup's slice of x or v, the token's decay and step) is staged in LDS for a chunk of tokens at a time, two
// buffers taking turns: the next chunk's loads are in flight while this chunk is computed.
constexpr int PRE = 16;        // registers a thread lends to a chunk's loads of the shared rows
constexpr int MAX_CHUNK = 16;  // tokens a chunk at most

template <int CTRL>
__device__ inline float dpp_swap(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// the sum over the LN lanes of a column; every lane gets it
template <int LN>
__device__ inline float group_sum(float v) {
  if (LN >= 2) v += dpp_swap<0xB1>(v);    // lanes 1 apart (quad_perm [1,0,3,2])
  if (LN >= 4) v += dpp_swap<0x4E>(v);    // 2 apart (quad_perm [2,3,0,1])
  if (LN >= 8) v += dpp_swap<0x141>(v);   // the other quad of eight lanes (row_half_mirror)
  if (LN >= 16) v += dpp_swap<0x140>(v);  // the other half of sixteen (row_mirror)
  if (LN >= 32) v += __shfl_xor(v, 16, LQ_WAVE);
  if (LN >= 64) v += __shfl_xor(v, 32, LQ_WAVE);
  return v;
}

// A launch of the state-space scan in segments, for few long sequences that would leave most of the chip idle: a
// sequence of SEG_MIN_ROWS rows or more is cut into `nseg` segments (whole chunks), one workgroup each.  Pass 1: segment
// 0 runs from the sequence's state, the others from zero without results, each leaving its end state and the product
// of its decays; a short kernel chains them (S_end = prod(decay) S_start + S_end_from_zero); pass 2: segments 1 ..
// run again from their true starts.  Twice the arithmetic, the segments side by side.  Shorter sequences of the same
// launch run whole in pass 1.
constexpr int SEG_MIN_ROWS = 512;
constexpr int SEG_COUNT = 8;
struct SegArgs {
  int nseg, pass;  // nseg 1: no segments (pass 1 alone)
  float *state, *decay;  // [sequences * heads][nseg][P][N], [sequences * heads][nseg]
};

struct ScanShape {
  int heads, groups, P, N;  // groups: of the shared rows (state-space groups, q/k heads)
  const int *seq_slot, *cu_rows;
};

// The chunk-wise staging that both scans share.  `a`, `b`: the two shared rows of a token ([rows, groups * N] each),
// `x`: the per-column input ([rows, heads * P]).  LDS of one buffer: [TT][2 N] then [TT][cols] then [TT][2].
template <int LN, int SLAB, int TH>  // TH: threads a workgroup
struct Stage {
  // entries of a token's two shared rows a thread (2 N <= 2 SLAB LN)
  static constexpr int PER = 2 * SLAB * LN > TH ? 2 * SLAB * LN / TH : 1;
  static constexpr int TT = PRE / PER;                    // tokens a chunk
  static constexpr int XPRE = TT / LN > 0 ? TT / LN : 1;  // chunk * cols / threads at most
  float ab[PRE];
  float xs[XPRE];
  float s0, s1;
};

template <int LN, int SLAB, int TH>
__global__ __launch_bounds__(TH) void ssd_scan_kernel(const float* __restrict__ x, int ldx,
                                                       const float* __restrict__ Bm, int ldb,
                                                       const float* __restrict__ Cm, int ldc,
                                                       const float* __restrict__ dt, int lddt,
                                                       const float* __restrict__ dt_bias,
                                                       const float* __restrict__ a_log,
                                                       const float* __restrict__ d_skip, float* __restrict__ state,
                                                       float* __restrict__ y, int ldy, ScanShape sh, SegArgs sg) {
  extern __shared__ float lds[];
  const int heads = sh.heads, P = sh.P, N = sh.N;
  constexpr int TT = Stage<LN, SLAB, TH>::TT, PER = Stage<LN, SLAB, TH>::PER;
  const int b = blockIdx.x / heads, h = blockIdx.x % heads, g = h / (heads / sh.groups);
  const int threads = blockDim.x, cols = threads / LN, tid = threadIdx.x;
  const int l = tid % LN, col = tid / LN, p0 = blockIdx.y * cols, p = p0 + col;
  const bool live = p < P;
  const int slab = (N + LN - 1) / LN;
  long long r0 = sh.cu_rows[b], r1 = sh.cu_rows[b + 1];
  // A long sequence of a launch in segments (see SegArgs): this workgroup's segment, where it starts from and
  // where it leaves its state.
  const int seg = blockIdx.z;
  const int nseg = (sg.nseg > 1 && r1 - r0 >= SEG_MIN_ROWS) ? sg.nseg : 1;
  if (seg >= nseg || (sg.pass == 2 && seg == 0)) return;
  if (nseg > 1) {
    const long long len = ((r1 - r0 + nseg - 1) / nseg + TT - 1) / TT * TT;
    r0 = min(r1, r0 + seg * len);
    r1 = min(r1, r0 + len);
  }
  const bool write_y = sg.pass == 2 || seg == 0;
  float* sp = state + (((long long)sh.seq_slot[b] * heads + h) * P + (live ? p : 0)) * N;
  float* seg_sp = nseg > 1 ? sg.state + ((((long long)blockIdx.x * sg.nseg + seg) * P + (live ? p : 0)) * N) : nullptr;
  const float* from = nseg > 1 && sg.pass == 2 ? seg_sp : sp;
  const bool from_zero = nseg > 1 && sg.pass == 1 && seg > 0;
  float* to = nseg == 1 ? sp : sg.pass == 1 ? seg_sp : nullptr;
  float dprod = 1.f;  // the product of the segment's decays
  constexpr int NP = LN * SLAB;  // a shared row in LDS, padded with zeros: entries past N take part as zeros
  const int buf_floats = TT * (2 * NP + 2 * cols + 2);  // shared rows, inputs, decay and step, outputs
  float S[SLAB];
#pragma unroll
  for (int i = 0; i < SLAB; ++i) {
    const int n = i * LN + l;
    S[i] = (live && !from_zero && i < slab && n < N) ? from[n] : 0.f;
  }
  const float A = -expf(a_log[h]), bias = dt_bias[h], D = d_skip[h];
  Stage<LN, SLAB, TH> st;

  auto fetch = [&](long long c0, int nt) {  // the chunk's loads, into registers
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int jj = 0; jj < PER; ++jj) {
        const int j = tid + jj * threads;
        if (t < nt && j < 2 * N)
          st.ab[t * PER + jj] = j < N ? Bm[(c0 + t) * ldb + g * N + j] : Cm[(c0 + t) * ldc + g * N + j - N];
      }
#pragma unroll
    for (int i = 0; i < Stage<LN, SLAB, TH>::XPRE; ++i) {
      const int e = tid + i * threads;
      if (e < nt * cols) {
        const int t = e / cols, c = e - t * cols;
        st.xs[i] = p0 + c < P ? x[(c0 + t) * ldx + h * P + p0 + c] : 0.f;
      }
    }
    if (tid < nt) st.s0 = dt[(c0 + tid) * lddt + h];
  };
  auto stash = [&](float* buf, int nt) {  // registers to LDS
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int jj = 0; jj < PER; ++jj) {
        const int c = tid + jj * threads;
        if (t < nt && c < 2 * N) buf[t * 2 * NP + (c < N ? c : NP + c - N)] = st.ab[t * PER + jj];
      }
#pragma unroll
    for (int i = 0; i < Stage<LN, SLAB, TH>::XPRE; ++i) {
      const int e = tid + i * threads;
      if (e < nt * cols) buf[TT * 2 * NP + e] = st.xs[i];
    }
    if (tid < nt) {
      const float step = softplus_f(st.s0 + bias);
      buf[TT * (2 * NP + cols) + 2 * tid] = expf(A * step);
      buf[TT * (2 * NP + cols) + 2 * tid + 1] = step;
    }
  };

  auto flush = [&](const float* buf, long long c0, int nt) {  // a chunk's outputs, from LDS to memory
    if (!write_y) return;
    for (int e = tid; e < nt * cols; e += threads) {
      const int t = e / cols, c = e - t * cols;
      if (p0 + c < P) y[(c0 + t) * ldy + h * P + p0 + c] = buf[TT * (2 * NP + cols + 2) + e];
    }
  };
  for (int e = tid; e < 2 * buf_floats; e += threads) lds[e] = 0.f;
  __syncthreads();
  int cur = 0;
  if (r1 > r0) {
    const int nt = (int)min((long long)TT, r1 - r0);
    fetch(r0, nt);
    stash(lds, nt);
  }
  __syncthreads();
  for (long long c0 = r0; c0 < r1; c0 += TT, cur ^= 1) {
    const int nt = (int)min((long long)TT, r1 - c0);
    const int next = (int)min((long long)TT, r1 - c0 - TT);
    if (c0 > r0) flush(lds + (cur ^ 1) * buf_floats, c0 - TT, TT);  // the chunk before: its stores are long done
    if (next > 0) fetch(c0 + TT, next);                             // when the wait for these loads comes
    float* buf = lds + cur * buf_floats;
    const float* scal = buf + TT * (2 * NP + cols);
    float* outs = buf + TT * (2 * NP + cols + 2);
    // a token's operands are read from LDS into registers while the token before it is computed (two sets of
    // registers take turns: a read placed after the LDS store of a result could not pass it)
    struct Tok {
      float b[SLAB], c[SLAB], decay, step, x;
    };
    auto load = [&](Tok& k, int t) {
      k.decay = scal[2 * t], k.step = scal[2 * t + 1], k.x = buf[TT * 2 * NP + t * cols + col];
#pragma unroll
      for (int i = 0; i < SLAB; ++i) k.b[i] = buf[t * 2 * NP + i * LN + l], k.c[i] = buf[t * 2 * NP + NP + i * LN + l];
    };
    auto compute = [&](const Tok& k, int t) {
      const float dx = k.step * k.x;
      dprod *= k.decay;
      float acc = 0.f, acc1 = 0.f;  // (two chains of multiply-adds, even and odd entries, added at the end)
#pragma unroll
      for (int i = 0; i < SLAB; i += 2) {
        S[i] = fmaf(k.b[i], dx, k.decay * S[i]);
        S[i + 1] = fmaf(k.b[i + 1], dx, k.decay * S[i + 1]);
        acc = fmaf(S[i], k.c[i], acc);
        acc1 = fmaf(S[i + 1], k.c[i + 1], acc1);
      }
      acc = group_sum<LN>(acc + acc1);
      if (l == 0) outs[t * cols + col] = fmaf(D, k.x, acc);
    };
    Tok ka, kb;
    load(ka, 0);
#pragma unroll
    for (int t = 0; t < TT; t += 2) {  // (unrolled: a token's places in LDS are constants)
      if (t >= nt) break;
      if (t + 1 < nt) load(kb, t + 1);
      compute(ka, t);
      if (t + 1 < nt) {
        if (t + 2 < nt) load(ka, t + 2);
        compute(kb, t + 1);
      }
    }
    if (next > 0) stash(lds + (cur ^ 1) * buf_floats, next);
    __syncthreads();
  }
  if (r1 > r0) {  // the last chunk's outputs (cur has moved on once more)
    const long long rows = r1 - r0, last = r0 + (rows - 1) / TT * TT;
    flush(lds + (cur ^ 1) * buf_floats, last, (int)(r1 - last));
  }
  if (live && to != nullptr) {
#pragma unroll
    for (int i = 0; i < SLAB; ++i) {
      const int n = i * LN + l;
      if (i < slab && n < N) to[n] = S[i];
    }
  }
  if (nseg > 1 && sg.pass == 1 && tid == 0 && blockIdx.y == 0) sg.decay[(long long)blockIdx.x * sg.nseg + seg] = dprod;
}

// Between the two passes of a launch in segments: segment 0 left the state at its true end, every other segment the
// state it reaches from zero and the product of its decays.  In order, every segment's true start takes the place
// of what it left, and the last segment's true end goes into the cache.
__global__ __launch_bounds__(256) void ssd_chain_kernel(float* __restrict__ state, int heads, int PN, SegArgs sg,
                                                        const int* __restrict__ seq_slot,
                                                        const int* __restrict__ cu_rows) {
  const int bh = blockIdx.x, b = bh / heads, h = bh % heads;
  if (cu_rows[b + 1] - cu_rows[b] < SEG_MIN_ROWS) return;
  const int e = blockIdx.y * 256 + threadIdx.x;
  if (e >= PN) return;
  float* seg = sg.state + (long long)bh * sg.nseg * PN + e;
  float S = seg[0];
  for (int s = 1; s < sg.nseg; ++s) {
    const float local = seg[(long long)s * PN];
    seg[(long long)s * PN] = S;
    S = fmaf(sg.decay[(long long)bh * sg.nseg + s], S, local);
  }
  state[((long long)seq_slot[b] * heads + h) * PN + e] = S;
}


// q and k of every (row, q/k head) made unit vectors in place, x / sqrt(sum x^2 + eps), q also times q_scale: one
// wavefront a (row, head), ahead of the scan (nothing of it depends on the state).
__global__ __launch_bounds__(64) void unit_heads_kernel(float* __restrict__ q, int ldq, float* __restrict__ k, int ldk,
                                                        int D, float q_scale, float eps) {
  float* qr = q + (long long)blockIdx.x * ldq + blockIdx.y * D;
  float* kr = k + (long long)blockIdx.x * ldk + blockIdx.y * D;
  float sq = 0.f, sk = 0.f;
  for (int d = threadIdx.x; d < D; d += 64) sq = fmaf(qr[d], qr[d], sq), sk = fmaf(kr[d], kr[d], sk);
  const float qinv = q_scale / sqrtf(wave_sum(sq) + eps), kinv = 1.f / sqrtf(wave_sum(sk) + eps);
  for (int d = threadIdx.x; d < D; d += 64) qr[d] *= qinv, kr[d] *= kinv;
}

// Gated delta rule: S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q, with q and k unit vectors (made so
// by the kernel above), beta = sigmoid(raw), g = exp(-exp(A_log) softplus(raw + bias)).
// (ScanShape: groups = q/k heads, N = key size.)
template <int LN, int SLAB, int TH>
__global__ __launch_bounds__(TH) void delta_scan_kernel(const float* __restrict__ q, int ldq,
                                                         const float* __restrict__ k, int ldk,
                                                         const float* __restrict__ v, int ldv,
                                                         const float* __restrict__ beta, int ldbeta,
                                                         const float* __restrict__ a, int lda,
                                                         const float* __restrict__ dt_bias,
                                                         const float* __restrict__ a_log, float* __restrict__ state,
                                                         float* __restrict__ out, int ldo, ScanShape sh) {
  extern __shared__ float lds[];
  const int heads = sh.heads, P = sh.P, N = sh.N;
  constexpr int TT = Stage<LN, SLAB, TH>::TT, PER = Stage<LN, SLAB, TH>::PER;
  const int b = blockIdx.x / heads, h = blockIdx.x % heads, j = h / (heads / sh.groups);
  const int threads = blockDim.x, cols = threads / LN, tid = threadIdx.x;
  const int l = tid % LN, col = tid / LN, p0 = blockIdx.y * cols, p = p0 + col;
  const bool live = p < P;
  const int slab = (N + LN - 1) / LN;
  const long long r0 = sh.cu_rows[b], r1 = sh.cu_rows[b + 1];
  float* sp = state + (((long long)sh.seq_slot[b] * heads + h) * P + (live ? p : 0)) * N;
  constexpr int NP = LN * SLAB;  // a shared row in LDS, padded with zeros: entries past N take part as zeros
  const int buf_floats = TT * (2 * NP + 2 * cols + 2);  // shared rows, inputs, decay and step, outputs
  float S[SLAB];
#pragma unroll
  for (int i = 0; i < SLAB; ++i) {
    const int n = i * LN + l;
    S[i] = (live && i < slab && n < N) ? sp[n] : 0.f;
  }
  const float A = -expf(a_log[h]), bias = dt_bias[h];
  Stage<LN, SLAB, TH> st;

  auto fetch = [&](long long c0, int nt) {
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int jj = 0; jj < PER; ++jj) {
        const int c = tid + jj * threads;
        if (t < nt && c < 2 * N)
          st.ab[t * PER + jj] = c < N ? q[(c0 + t) * ldq + j * N + c] : k[(c0 + t) * ldk + j * N + c - N];
      }
#pragma unroll
    for (int i = 0; i < Stage<LN, SLAB, TH>::XPRE; ++i) {
      const int e = tid + i * threads;
      if (e < nt * cols) {
        const int t = e / cols, c = e - t * cols;
        st.xs[i] = p0 + c < P ? v[(c0 + t) * ldv + h * P + p0 + c] : 0.f;
      }
    }
    if (tid < nt) {
      st.s0 = a[(c0 + tid) * lda + h];
      st.s1 = beta[(c0 + tid) * ldbeta + h];
    }
  };
  auto stash = [&](float* buf, int nt) {
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int jj = 0; jj < PER; ++jj) {
        const int c = tid + jj * threads;
        if (t < nt && c < 2 * N) buf[t * 2 * NP + (c < N ? c : NP + c - N)] = st.ab[t * PER + jj];
      }
#pragma unroll
    for (int i = 0; i < Stage<LN, SLAB, TH>::XPRE; ++i) {
      const int e = tid + i * threads;
      if (e < nt * cols) buf[TT * 2 * NP + e] = st.xs[i];
    }
    if (tid < nt) {
      buf[TT * (2 * NP + cols) + 2 * tid] = expf(A * softplus_f(st.s0 + bias));
      buf[TT * (2 * NP + cols) + 2 * tid + 1] = sigmoid_f(st.s1);
    }
  };

  auto flush = [&](const float* buf, long long c0, int nt) {  // a chunk's outputs, from LDS to memory
    for (int e = tid; e < nt * cols; e += threads) {
      const int t = e / cols, c = e - t * cols;
      if (p0 + c < P) out[(c0 + t) * ldo + h * P + p0 + c] = buf[TT * (2 * NP + cols + 2) + e];
    }
  };
  for (int e = tid; e < 2 * buf_floats; e += threads) lds[e] = 0.f;
  __syncthreads();
  int cur = 0;
  if (r1 > r0) {
    const int nt = (int)min((long long)TT, r1 - r0);
    fetch(r0, nt);
    stash(lds, nt);
  }
  __syncthreads();
  for (long long c0 = r0; c0 < r1; c0 += TT, cur ^= 1) {
    const int nt = (int)min((long long)TT, r1 - c0);
    const int next = (int)min((long long)TT, r1 - c0 - TT);
    if (c0 > r0) flush(lds + (cur ^ 1) * buf_floats, c0 - TT, TT);  // the chunk before: its stores are long done
    if (next > 0) fetch(c0 + TT, next);                             // when the wait for these loads comes
    float* buf = lds + cur * buf_floats;
    const float* scal = buf + TT * (2 * NP + cols);
    float* outs = buf + TT * (2 * NP + cols + 2);
    struct Tok {  // (as in the state-space scan: the next token's operands are read while this one is computed)
      float q[SLAB], k[SLAB], decay, beta, v;
    };
    auto load = [&](Tok& k, int t) {
      k.decay = scal[2 * t], k.beta = scal[2 * t + 1], k.v = buf[TT * 2 * NP + t * cols + col];
#pragma unroll
      for (int i = 0; i < SLAB; ++i) k.q[i] = buf[t * 2 * NP + i * LN + l], k.k[i] = buf[t * 2 * NP + NP + i * LN + l];
    };
    auto compute = [&](const Tok& k, int t) {
      float sk = 0.f, sk1 = 0.f;  // (two chains, even and odd entries)
#pragma unroll
      for (int i = 0; i < SLAB; i += 2) {
        S[i] *= k.decay;
        S[i + 1] *= k.decay;
        sk = fmaf(S[i], k.k[i], sk);
        sk1 = fmaf(S[i + 1], k.k[i + 1], sk1);
      }
      const float u = k.beta * (k.v - group_sum<LN>(sk + sk1));
      float o = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < SLAB; i += 2) {
        S[i] = fmaf(k.k[i], u, S[i]);
        S[i + 1] = fmaf(k.k[i + 1], u, S[i + 1]);
        o = fmaf(S[i], k.q[i], o);
        o1 = fmaf(S[i + 1], k.q[i + 1], o1);
      }
      o = group_sum<LN>(o + o1);
      if (l == 0) outs[t * cols + col] = o;
    };
    Tok ka, kb;
    load(ka, 0);
#pragma unroll
    for (int t = 0; t < TT; t += 2) {  // (unrolled: a token's places in LDS are constants)
      if (t >= nt) break;
      if (t + 1 < nt) load(kb, t + 1);
      compute(ka, t);
      if (t + 1 < nt) {
        if (t + 2 < nt) load(ka, t + 2);
        compute(kb, t + 1);
      }
    }
    if (next > 0) stash(lds + (cur ^ 1) * buf_floats, next);
    __syncthreads();
  }
  if (r1 > r0) {  // the last chunk's outputs (cur has moved on once more)
    const long long rows = r1 - r0, last = r0 + (rows - 1) / TT * TT;
    flush(lds + (cur ^ 1) * buf_floats, last, (int)(r1 - last));
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < SLAB; ++i) {
      const int n = i * LN + l;
      if (i < slab && n < N) sp[n] = S[i];
    }
  }
}

// Gated linear attention: S <- diag(a) S + k v^T;  o = S^T (q q_scale), with a decay for every key channel,
// a = sigmoid(z + bias)^(inv_tau), taken as exp(inv_tau * log sigmoid(z + bias)) in 32-bit.
// (ScanShape: groups = heads, N = key size, P = value size; the state [slots, heads, P, N].)
// A chunk of TT tokens is staged in LDS (q, k and the decays of the head, the workgroup's slice of v), two buffers
// taking turns: the next chunk's loads are in flight while this chunk is computed token by token, and a chunk's
// results leave together.  A token's sums are a thread's own entries in ascending order, then the exchange over the
// column's lanes: the same in every launch.
constexpr int gla_tokens(int np, int th, int ln) {
  // tokens a chunk: at most 24 registers a thread for the shared rows, and two buffers within 64 KB of LDS
  const int by_regs = 24 * th / (3 * np), by_lds = 8192 / (3 * np + 2 * (th / ln));
  const int t = by_regs < by_lds ? by_regs : by_lds;
  return t >= 16 ? 16 : t >= 8 ? 8 : t >= 4 ? 4 : t >= 2 ? 2 : 1;
}

template <int LN, int SLAB, int TH>
__global__ __launch_bounds__(TH) void gla_scan_kernel(const float* __restrict__ q, int ldq, const float* __restrict__ k,
                                                       int ldk, const float* __restrict__ v, int ldv,
                                                       const float* __restrict__ z, int ldz,
                                                       const float* __restrict__ bias, float* __restrict__ state,
                                                       float* __restrict__ out, int ldo, ScanShape sh, float q_scale,
                                                       float inv_tau, SegArgs sg) {
  extern __shared__ float lds[];
  constexpr int NP = LN * SLAB;  // a shared row in LDS, padded with zeros: entries past N take part as zeros
  constexpr int TT = gla_tokens(NP, TH, LN);
  constexpr int PER = (3 * TT * NP + TH - 1) / TH;
  constexpr int cols = TH / LN;
  constexpr int XPRE = (TT * cols + TH - 1) / TH;
  constexpr int BUF = TT * (3 * NP + 2 * cols);  // q, k, decays [TT][NP] each, then v and the results [TT][cols]
  const int heads = sh.heads, P = sh.P, N = sh.N;
  const int b = blockIdx.x / heads, h = blockIdx.x % heads;
  const int tid = threadIdx.x, l = tid % LN, col = tid / LN, p0 = blockIdx.y * cols, p = p0 + col;
  const bool live = p < P;
  long long r0 = sh.cu_rows[b], r1 = sh.cu_rows[b + 1];
  // A long sequence of a launch in segments (see SegArgs; here a segment leaves the product of its decays for
  // every key channel): this workgroup's segment, where it starts from and where it leaves its state.
  const int seg = blockIdx.z;
  const int nseg = (sg.nseg > 1 && r1 - r0 >= SEG_MIN_ROWS) ? sg.nseg : 1;
  if (seg >= nseg || (sg.pass == 2 && seg == 0)) return;
  if (nseg > 1) {
    const long long len = ((r1 - r0 + nseg - 1) / nseg + TT - 1) / TT * TT;
    r0 = min(r1, r0 + seg * len);
    r1 = min(r1, r0 + len);
  }
  const bool write_out = sg.pass == 2 || seg == 0;
  float* sp = state + (((long long)sh.seq_slot[b] * heads + h) * P + (live ? p : 0)) * N;
  float* seg_sp = nseg > 1 ? sg.state + ((((long long)blockIdx.x * sg.nseg + seg) * P + (live ? p : 0)) * N) : nullptr;
  const float* from = nseg > 1 && sg.pass == 2 ? seg_sp : sp;
  const bool from_zero = nseg > 1 && sg.pass == 1 && seg > 0;
  float* to = nseg == 1 ? sp : sg.pass == 1 ? seg_sp : nullptr;
  float S[SLAB], aprod[SLAB];  // aprod: the product of the segment's decays of this thread's channels
#pragma unroll
  for (int i = 0; i < SLAB; ++i) {
    const int n = i * LN + l;
    S[i] = (live && !from_zero && n < N) ? from[n] : 0.f;
    aprod[i] = 1.f;
  }
  float pre[PER], xpre[XPRE];
  auto fetch = [&](long long c0, int nt) {  // the chunk's loads, into registers
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = tid + j * TH, which = e / (TT * NP), rem = e - which * (TT * NP), t = rem / NP, n = rem - t * NP;
      float val = 0.f;
      if (which < 3 && t < nt && n < N) {
        const long long r = c0 + t;
        val = which == 0 ? q[r * ldq + h * N + n] : which == 1 ? k[r * ldk + h * N + n] : z[r * ldz + h * N + n];
      }
      pre[j] = val;
    }
#pragma unroll
    for (int j = 0; j < XPRE; ++j) {
      const int e = tid + j * TH, t = e / cols, c = e - t * cols;
      xpre[j] = (t < nt && p0 + c < P) ? v[(c0 + t) * ldv + h * P + p0 + c] : 0.f;
    }
  };
  auto stash = [&](float* buf) {  // registers to LDS; the decay is made of its logit here
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = tid + j * TH, which = e / (TT * NP), n = e % NP;
      if (which >= 3) continue;
      float val = pre[j];
      if (which == 0) val *= q_scale;
      else if (which == 2) val = n < N ? expf(-softplus_f(-(val + bias[h * N + n])) * inv_tau) : 0.f;
      buf[e] = val;
    }
#pragma unroll
    for (int j = 0; j < XPRE; ++j) {
      const int e = tid + j * TH;
      if (e < TT * cols) buf[3 * TT * NP + e] = xpre[j];
    }
  };
  int cur = 0;
  if (r1 > r0) {
    fetch(r0, (int)min((long long)TT, r1 - r0));
    stash(lds);
  }
  __syncthreads();
  for (long long c0 = r0; c0 < r1; c0 += TT, cur ^= 1) {
    const int nt = (int)min((long long)TT, r1 - c0);
    const int next = (int)min((long long)TT, r1 - c0 - TT);
    if (next > 0) fetch(c0 + TT, next);
    float* buf = lds + cur * BUF;
    const float *qs = buf, *ks = buf + TT * NP, *as = buf + 2 * TT * NP, *vs = buf + 3 * TT * NP;
    float* os = buf + 3 * TT * NP + TT * cols;
    // a token's operands are read from LDS into registers while the token before it is computed (two sets of
    // registers take turns: a read placed after the LDS store of a result could not pass it)
    struct Tok {
      float q[SLAB], k[SLAB], a[SLAB], v;
    };
    auto load = [&](Tok& x, int t) {
      x.v = vs[t * cols + col];
#pragma unroll
      for (int i = 0; i < SLAB; ++i) {
        const int n = t * NP + i * LN + l;
        x.q[i] = qs[n], x.k[i] = ks[n], x.a[i] = as[n];
      }
    };
    auto compute = [&](const Tok& x, int t) {
      float acc = 0.f, acc1 = 0.f;  // (two chains of multiply-adds, even and odd entries, added at the end)
#pragma unroll
      for (int i = 0; i < SLAB; i += 2) {
        S[i] = fmaf(x.k[i], x.v, x.a[i] * S[i]);
        S[i + 1] = fmaf(x.k[i + 1], x.v, x.a[i + 1] * S[i + 1]);
        acc = fmaf(S[i], x.q[i], acc);
        acc1 = fmaf(S[i + 1], x.q[i + 1], acc1);
      }
      if (from_zero) {
#pragma unroll
        for (int i = 0; i < SLAB; ++i) aprod[i] *= x.a[i];
      }
      acc = group_sum<LN>(acc + acc1);
      if (l == 0) os[t * cols + col] = acc;
    };
    Tok ta, tb;
    load(ta, 0);
#pragma unroll
    for (int t = 0; t < TT; t += 2) {  // (unrolled: a token's places in LDS are constants)
      if (t >= nt) break;
      if (t + 1 < nt) load(tb, t + 1);
      compute(ta, t);
      if (t + 1 < nt) {
        if (t + 2 < nt) load(ta, t + 2);
        compute(tb, t + 1);
      }
    }
    if (next > 0) stash(lds + (cur ^ 1) * BUF);
    __syncthreads();
    if (write_out)
      for (int e = tid; e < nt * cols; e += TH) {
        const int t = e / cols, c = e - t * cols;
        if (p0 + c < P) out[(c0 + t) * ldo + h * P + p0 + c] = os[e];
      }
  }
  if (live && to != nullptr) {
#pragma unroll
    for (int i = 0; i < SLAB; ++i) {
      const int n = i * LN + l;
      if (n < N) to[n] = S[i];
    }
  }
  if (from_zero && col == 0 && blockIdx.y == 0) {
#pragma unroll
    for (int i = 0; i < SLAB; ++i) {
      const int n = i * LN + l;
      if (n < N) sg.decay[((long long)blockIdx.x * sg.nseg + seg) * N + n] = aprod[i];
    }
  }
}

// Between the two passes of a gated-linear-attention launch in segments: segment 0 left the state at its true end,
// every other segment the state it reaches from zero and, for every key channel, the product of its decays.  In
// order, every segment's true start takes the place of what it left, and the last segment's true end goes into the
// cache.
__global__ __launch_bounds__(256) void gla_chain_kernel(float* __restrict__ state, int heads, int P, int N, SegArgs sg,
                                                        const int* __restrict__ seq_slot, const int* __restrict__ cu_rows) {
  const int b = blockIdx.x / heads, h = blockIdx.x % heads;
  if (cu_rows[b + 1] - cu_rows[b] < SEG_MIN_ROWS) return;
  const long long PN = (long long)P * N, idx = (long long)blockIdx.y * 256 + threadIdx.x;
  if (idx >= PN) return;
  const int n = (int)(idx % N);
  float* segs = sg.state + (long long)blockIdx.x * sg.nseg * PN + idx;
  float cur = segs[0];
  for (int s = 1; s < sg.nseg; ++s) {
    const float reached = segs[s * PN], a = sg.decay[((long long)blockIdx.x * sg.nseg + s) * N + n];
    segs[s * PN] = cur;
    cur = fmaf(a, cur, reached);
  }
  state[((long long)seq_slot[b] * heads + h) * PN + idx] = cur;
}

// Gated delta rule with a decay for every key channel: S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;
// o = S^T q, with q and k unit vectors (made so by `unit_heads_kernel`), beta = sigmoid(raw) and
// g = exp(-exp(A_log_h) softplus(z + bias)) for every key channel of every head, made of its logit where the chunk is
// staged.  (ScanShape: groups = q/k heads, N = key size, P = value size; the state [slots, heads, P, N].)  The
// staging is that of the gated linear attention scan (q, k and the decays of a chunk of tokens in LDS, two buffers
// taking turns), with one more number a token, beta.
constexpr int dch_tokens(int np, int th, int ln) {
  const int by_regs = 24 * th / (3 * np), by_lds = 8192 / (3 * np + 2 * (th / ln) + 1);
  const int t = by_regs < by_lds ? by_regs : by_lds;
  return t >= 16 ? 16 : t >= 8 ? 8 : t >= 4 ? 4 : t >= 2 ? 2 : 1;
}

// SINGLE: chunks of one token, for a step of single tokens: a workgroup's LDS is then a few hundred bytes where a chunk
// of 16 tokens takes 50 KB, so all of a compute unit's workgroups are resident at once.  A token's operations and their
// order are the same either way.
template <int LN, int SLAB, int TH, bool SINGLE>
__global__ __launch_bounds__(TH) void delta_channel_scan_kernel(const float* __restrict__ q, int ldq,
                                                                 const float* __restrict__ k, int ldk,
                                                                 const float* __restrict__ v, int ldv,
                                                                 const float* __restrict__ beta, int ldbeta,
                                                                 const float* __restrict__ z, int ldz,
                                                                 const float* __restrict__ dt_bias,
                                                                 const float* __restrict__ a_log,
                                                                 float* __restrict__ state, float* __restrict__ out,
                                                                 int ldo, ScanShape sh) {
  extern __shared__ float lds[];
  constexpr int NP = LN * SLAB;  // a shared row in LDS, padded with zeros: entries past N take part as zeros
  constexpr int TT = SINGLE ? 1 : dch_tokens(NP, TH, LN);
  constexpr int PER = (3 * TT * NP + TH - 1) / TH;
  constexpr int cols = TH / LN;
  constexpr int XPRE = (TT * cols + TH - 1) / TH;
  constexpr int BUF = TT * (3 * NP + 2 * cols + 1);  // q, k, decays [TT][NP]; v, results [TT][cols]; beta [TT]
  const int heads = sh.heads, P = sh.P, N = sh.N;
  const int b = blockIdx.x / heads, h = blockIdx.x % heads, j = h / (heads / sh.groups);
  const int tid = threadIdx.x, l = tid % LN, col = tid / LN, p0 = blockIdx.y * cols, p = p0 + col;
  const bool live = p < P;
  const long long r0 = sh.cu_rows[b], r1 = sh.cu_rows[b + 1];
  float* sp = state + (((long long)sh.seq_slot[b] * heads + h) * P + (live ? p : 0)) * N;
  float S[SLAB];
#pragma unroll
  for (int i = 0; i < SLAB; ++i) {
    const int n = i * LN + l;
    S[i] = (live && n < N) ? sp[n] : 0.f;
  }
  const float A = -expf(a_log[h]);
  float pre[PER], xpre[XPRE], bpre = 0.f;
  auto fetch = [&](long long c0, int nt) {  // the chunk's loads, into registers
#pragma unroll
    for (int jj = 0; jj < PER; ++jj) {
      const int e = tid + jj * TH, which = e / (TT * NP), rem = e - which * (TT * NP), t = rem / NP, n = rem - t * NP;
      float val = 0.f;
      if (which < 3 && t < nt && n < N) {
        const long long r = c0 + t;
        val = which == 0 ? q[r * ldq + j * N + n] : which == 1 ? k[r * ldk + j * N + n] : z[r * ldz + h * N + n];
      }
      pre[jj] = val;
    }
#pragma unroll
    for (int jj = 0; jj < XPRE; ++jj) {
      const int e = tid + jj * TH, t = e / cols, c = e - t * cols;
      xpre[jj] = (t < nt && p0 + c < P) ? v[(c0 + t) * ldv + h * P + p0 + c] : 0.f;
    }
    bpre = tid < nt ? beta[(c0 + tid) * ldbeta + h] : 0.f;
  };
  auto stash = [&](float* buf) {  // registers to LDS; the decay is made of its logit here
#pragma unroll
    for (int jj = 0; jj < PER; ++jj) {
      const int e = tid + jj * TH, which = e / (TT * NP), n = e % NP;
      if (which >= 3) continue;
      float val = pre[jj];
      if (which == 2) val = n < N ? expf(A * softplus_f(val + dt_bias[h * N + n])) : 0.f;
      buf[e] = val;
    }
#pragma unroll
    for (int jj = 0; jj < XPRE; ++jj) {
      const int e = tid + jj * TH;
      if (e < TT * cols) buf[3 * TT * NP + e] = xpre[jj];
    }
    if (tid < TT) buf[3 * TT * NP + 2 * TT * cols + tid] = sigmoid_f(bpre);
  };
  int cur = 0;
  if (r1 > r0) {
    fetch(r0, (int)min((long long)TT, r1 - r0));
    stash(lds);
  }
  __syncthreads();
  for (long long c0 = r0; c0 < r1; c0 += TT, cur ^= 1) {
    const int nt = (int)min((long long)TT, r1 - c0);
    const int next = (int)min((long long)TT, r1 - c0 - TT);
    if (next > 0) fetch(c0 + TT, next);
    float* buf = lds + cur * BUF;
    const float *qs = buf, *ks = buf + TT * NP, *as = buf + 2 * TT * NP, *vs = buf + 3 * TT * NP;
    const float* bs = buf + 3 * TT * NP + 2 * TT * cols;
    float* os = buf + 3 * TT * NP + TT * cols;
    struct Tok {  // (the next token's operands are read while this one is computed)
      float q[SLAB], k[SLAB], a[SLAB], v, beta;
    };
    auto load = [&](Tok& x, int t) {
      x.v = vs[t * cols + col], x.beta = bs[t];
#pragma unroll
      for (int i = 0; i < SLAB; ++i) {
        const int n = t * NP + i * LN + l;
        x.q[i] = qs[n], x.k[i] = ks[n], x.a[i] = as[n];
      }
    };
    auto compute = [&](const Tok& x, int t) {
      float sk = 0.f, sk1 = 0.f;  // (two chains, even and odd entries)
#pragma unroll
      for (int i = 0; i < SLAB; i += 2) {
        S[i] *= x.a[i];
        S[i + 1] *= x.a[i + 1];
        sk = fmaf(S[i], x.k[i], sk);
        sk1 = fmaf(S[i + 1], x.k[i + 1], sk1);
      }
      const float u = x.beta * (x.v - group_sum<LN>(sk + sk1));
      float o = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < SLAB; i += 2) {
        S[i] = fmaf(x.k[i], u, S[i]);
        S[i + 1] = fmaf(x.k[i + 1], u, S[i + 1]);
        o = fmaf(S[i], x.q[i], o);
        o1 = fmaf(S[i + 1], x.q[i + 1], o1);
      }
      o = group_sum<LN>(o + o1);
      if (l == 0) os[t * cols + col] = o;
    };
    Tok ta, tb;
    load(ta, 0);
#pragma unroll
    for (int t = 0; t < TT; t += 2) {  // (unrolled: a token's places in LDS are constants)
      if (t >= nt) break;
      if (t + 1 < nt) load(tb, t + 1);
      compute(ta, t);
      if (t + 1 < nt) {
        if (t + 2 < nt) load(ta, t + 2);
        compute(tb, t + 1);
      }
    }
    if (next > 0) stash(lds + (cur ^ 1) * BUF);
    __syncthreads();
    for (int e = tid; e < nt * cols; e += TH) {
      const int t = e / cols, c = e - t * cols;
      if (p0 + c < P) out[(c0 + t) * ldo + h * P + p0 + c] = os[e];
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < SLAB; ++i) {
      const int n = i * LN + l;
      if (n < N) sp[n] = S[i];
    }
  }
}

// ---------------------------------------------------------------- norms after the scans
// One workgroup a (row, group of `group` columns).  gate_first: v = y silu(z), out = v / rms(v) w;
// else: out = y / rms(y) w silu(z).  `sigmoid_gate`: sigmoid(z) in the place of silu(z).  w has `wlen` entries and repeats (one weight for all groups, or one a column).
template <typename T>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ y, int ldy, const float* __restrict__ z, int ldz,
                                     const float* __restrict__ w, int wlen, float eps, int group, T* __restrict__ out,
                                     int ldo, int gate_first, int sigmoid_gate) {
  __shared__ float red[16];
  const int r = blockIdx.y, c0 = blockIdx.x * group;
  const float* yr = y + (long long)r * ldy + c0;
  const float* zr = z + (long long)r * ldz + c0;
  float ss = 0.f;
  for (int c = threadIdx.x; c < group; c += blockDim.x) {
    const float v = gate_first ? yr[c] * (sigmoid_gate ? sigmoid_f(zr[c]) : silu_f(zr[c])) : yr[c];
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / group + eps);
  for (int c = threadIdx.x; c < group; c += blockDim.x) {
    const float gate = sigmoid_gate ? sigmoid_f(zr[c]) : silu_f(zr[c]);
    const float v = gate_first ? yr[c] * gate * inv * w[(c0 + c) % wlen] : yr[c] * inv * w[(c0 + c) % wlen] * gate;
    store_as<T>(out + (long long)r * ldo + c0 + c, v);
  }
}

struct MeanInputs {
  const float* x[4];
  const float* w[4];
};

// out = (1 / n) sum_i x_i / rms(x_i) w_i, row by row.  The branches' sums of squares are taken in one pass (their
// loads are in flight together), each with the block's fixed tree.
__global__ void rmsnorm_mean_kernel(MeanInputs in, int n_in, float eps, float* __restrict__ out, int width) {
  __shared__ float red[16];
  const long long r = blockIdx.x;
  float ss[4] = {0.f, 0.f, 0.f, 0.f};
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float v = i < n_in ? in.x[i][r * width + c] : 0.f;
      ss[i] = fmaf(v, v, ss[i]);
    }
  }
  float inv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) inv[i] = i < n_in ? 1.f / sqrtf(block_sum(ss[i], red) / width + eps) : 0.f;
  const float share = 1.f / n_in;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < n_in) acc += in.x[i][r * width + c] * inv[i] * in.w[i][c];
    out[r * width + c] = acc * share;
  }
}

// How a scan over states of N entries a column and P columns a head is launched; all of it follows from the
// model's sizes, nothing from the step, so that a token's sums are the same in every launch.
struct ScanLaunch {
  int ln, slab, threads, cols, tt;
  size_t lds;
};

bool scan_launch(int N, int P, long long work, ScanLaunch& s) {
  // Workgroups of 256 threads, fewer where a head has fewer columns than they would hold.  (Smaller workgroups for
  // launches that leave compute units idle were measured and are not taken: every workgroup stages the whole shared
  // rows of its tokens, and a chunk of fewer tokens pays its barrier more often; `work`, the (sequence, head,
  // segment) triples of the launch, is kept for that choice.)  Nothing of a token's arithmetic depends on the size.
  (void)work;
  s.slab = N > 512 ? 16 : 8;
  s.ln = 1;
  while ((N + s.ln - 1) / s.ln > s.slab) s.ln <<= 1;
  if (s.ln > 64) return false;
  s.threads = 256;
  while (s.threads > 64 && s.threads / 2 >= s.ln && 2 * s.slab * s.ln <= PRE * (s.threads / 2) &&
         s.threads / s.ln >= 2 * P)
    s.threads >>= 1;
  const int per = 2 * s.slab * s.ln > s.threads ? 2 * s.slab * s.ln / s.threads : 1;  // as Stage<LN, SLAB, TH> has them
  s.tt = PRE / per;
  if (s.tt < 1) return false;
  s.cols = s.threads / s.ln;
  s.lds = 2 * (size_t)s.tt * (2 * s.ln * s.slab + 2 * s.cols + 2) * sizeof(float);  // (rows padded to LN * slab)
  return s.lds <= 64 * 1024;
}

}  // namespace

extern "C" int lq_dynamic_tanh(float* x, const float* delta, int pieces, long long piece_stride, float scale,
                               const float* w, const float* b, const float* alpha, void* out, int out_dtype, int rows,
                               int width, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && width > 0, "dynamic_tanh: rows %d and width %d must be positive", rows, width);
  LQ_REQUIRE(x && w && b && alpha && out, "dynamic_tanh: null pointer");
  LQ_REQUIRE(pieces >= 0 && (pieces == 0 || delta != nullptr), "dynamic_tanh: %d pieces of a delta", pieces);
  const long long n = (long long)rows * width;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (out_dtype == LQ_F32)
    dynamic_tanh_kernel<float><<<blocks, 256, 0, stream>>>(x, delta, pieces, piece_stride, scale, w, b, alpha, (float*)out, n, width);
  else if (out_dtype == LQ_BF16)
    dynamic_tanh_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, delta, pieces, piece_stride, scale, w, b, alpha, (bf16_t*)out, n, width);
  else
    LQ_REQUIRE(false, "dynamic_tanh: unknown dtype %d", out_dtype);
  LQ_CHECK_LAUNCH("dynamic_tanh");
  return 0;
}

extern "C" int lq_add_scaled(float* x, const float* delta, int pieces, long long piece_stride, float scale, long long n,
                             hipStream_t stream) {
  LQ_REQUIRE(x && delta && pieces > 0 && n > 0, "add_scaled: bad arguments");
  add_scaled_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, delta, pieces, piece_stride, scale, n);
  LQ_CHECK_LAUNCH("add_scaled");
  return 0;
}

extern "C" int lq_glu(const void* gu, int in_dtype, int ld, void* out, int out_dtype, int ldo, int rows, int I, int act,
                      const float* bias, int tail, const float* row_gate, int ldrg, int gated, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && I > 0 && ld >= (gated ? 2 : 1) * I && tail >= 0 && ldo >= I + tail, "glu: rows %d, inner %d, strides %d and %d", rows, I, ld, ldo);
  LQ_REQUIRE(act >= ACT_SILU && act <= ACT_GELU_ERF, "glu: unknown activation %d", act);
  LQ_REQUIRE(gated || (bias == nullptr && tail == 0), "glu: a plain activation takes no bias and leaves no tail");
  LQ_REQUIRE(row_gate == nullptr || ldrg >= 1, "glu: the rows' gate needs a stride");
  LQ_REQUIRE(rows <= 65535 * 64, "glu: too many rows");
  LQ_REQUIRE(gu && out, "glu: null pointer");
  // a plain activation of 32-bit rows whose columns come in fours on 16 bytes: four columns a thread
  const int out_el = out_dtype == LQ_F32 ? 4 : 2;
  if (!gated && row_gate == nullptr && in_dtype == LQ_F32 && (out_dtype == LQ_F32 || out_dtype == LQ_BF16) && I % 4 == 0 &&
      ld % 4 == 0 && ldo % 4 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % (4 * out_el)) == 0) {
    for (int r0 = 0; r0 < rows; r0 += 65535) {
      const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
      dim3 grid(lq_ceil_div(I / 4, 256), nr);
      if (out_dtype == LQ_F32)
        activation4_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu + (long long)r0 * ld, ld,
                                                            (float*)out + (long long)r0 * ldo, ldo, I, act);
      else
        activation4_kernel<bf16_t><<<grid, 256, 0, stream>>>((const float*)gu + (long long)r0 * ld, ld,
                                                             (bf16_t*)out + (long long)r0 * ldo, ldo, I, act);
    }
    LQ_CHECK_LAUNCH("glu(activation)");
    return 0;
  }
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    dim3 grid(lq_ceil_div(I + tail, 256), nr);
#define LQ_GLU(TI, TO)                                                                                              \
  glu_kernel<TI, TO><<<grid, 256, 0, stream>>>((const TI*)gu + (long long)r0 * ld, ld, (TO*)out + (long long)r0 * ldo, \
                                               ldo, I, act, bias, tail,                                                 \
                                               row_gate ? row_gate + (long long)r0 * ldrg : nullptr, ldrg, gated)
    if (in_dtype == LQ_F32 && out_dtype == LQ_F32) LQ_GLU(float, float);
    else if (in_dtype == LQ_F32 && out_dtype == LQ_BF16) LQ_GLU(float, bf16_t);
    else if (in_dtype == LQ_BF16 && out_dtype == LQ_BF16) LQ_GLU(bf16_t, bf16_t);
    else if (in_dtype == LQ_BF16 && out_dtype == LQ_F32) LQ_GLU(bf16_t, float);
    else LQ_REQUIRE(false, "glu: unknown dtypes %d, %d", in_dtype, out_dtype);
#undef LQ_GLU
  }
  LQ_CHECK_LAUNCH("glu");
  return 0;
}

// x [rows, C] (stride ldx), w [C, taps], bias [C] or null, state [slots, taps - 1, C]; out [rows, C] (stride ldo).
// The state is read for the step's outputs and then moved on by a second launch.
extern "C" int lq_causal_conv(const float* x, int ldx, const float* w, const float* bias, float* state, float* out,
                              int ldo, int rows, int C, int taps, const int* row_seq, const int* row_pos,
                              const int* seq_slot, const int* seq_start, const int* cu_rows, int batch, int act,
                              hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && C > 0 && taps >= 1 && batch > 0, "causal_conv: rows %d, channels %d, taps %d, sequences %d", rows, C,
             taps, batch);
  LQ_REQUIRE(ldx >= C && ldo >= C, "causal_conv: a row stride is smaller than its row");
  LQ_REQUIRE(x && w && out && row_seq && row_pos && seq_slot && seq_start && cu_rows && (taps == 1 || state),
             "causal_conv: null pointer");
  LQ_REQUIRE(act >= ACT_NONE && act <= ACT_GELU_TANH, "causal_conv: unknown activation %d", act);
  LQ_REQUIRE(batch <= 65535, "causal_conv: too many sequences");
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    causal_conv_kernel<<<dim3(lq_ceil_div(C, 256), nr), 256, 0, stream>>>(
        x, ldx, w, bias, state, out + (long long)r0 * ldo, ldo, C, taps, row_seq + r0, row_pos + r0, seq_slot, seq_start,
        cu_rows, act);
  }
  LQ_CHECK_LAUNCH("causal_conv");
  if (taps > 1) {
    conv_state_kernel<<<dim3(lq_ceil_div(C, 256), batch), 256, 0, stream>>>(x, ldx, state, C, taps, seq_slot, cu_rows);
    LQ_CHECK_LAUNCH("causal_conv(state)");
  }
  return 0;
}

#define LQ_SCAN_TH(LAUNCH, LN, SL)                                 \
  if (cfg.threads == 256) LAUNCH(LN, SL, 256);                     \
  else if (cfg.threads == 128) LAUNCH(LN, SL, 128);                \
  else LAUNCH(LN, SL, 64)
#define LQ_SCAN_LANES(LAUNCH)                                      \
  switch (cfg.slab == 16 ? 128 : cfg.ln) {                         \
    case 1: { LQ_SCAN_TH(LAUNCH, 1, 8); } break;                   \
    case 2: { LQ_SCAN_TH(LAUNCH, 2, 8); } break;                   \
    case 4: { LQ_SCAN_TH(LAUNCH, 4, 8); } break;                   \
    case 8: { LQ_SCAN_TH(LAUNCH, 8, 8); } break;                   \
    case 16: { LQ_SCAN_TH(LAUNCH, 16, 8); } break;                 \
    case 32: { LQ_SCAN_TH(LAUNCH, 32, 8); } break;                 \
    case 64: { LQ_SCAN_TH(LAUNCH, 64, 8); } break;                 \
    default: { LQ_SCAN_TH(LAUNCH, 64, 16); } break;                \
  }

// Whether a launch over `batch` sequences, the longest bringing `max_rows` rows, runs in segments, and then the
// float32 scratch it needs: one decision for the query and the launch.
static long long ssd_segment_floats(int batch, int heads, int P, int N, int max_rows) {
  ScanLaunch cfg;
  if (max_rows < SEG_MIN_ROWS || !scan_launch(N, P, 1ll << 40, cfg)) return 0;  // (as workgroups of 256 threads)
  if ((long long)batch * heads * lq_ceil_div(P, cfg.cols) >= 4ll * lq_compute_units()) return 0;  // the chip is full as it is
  return (long long)batch * heads * SEG_COUNT * ((long long)P * N + 1);
}

extern "C" long long lq_ssd_scan_workspace(int batch, int heads, int P, int N, int max_rows) {
  if (batch <= 0 || heads <= 0 || P <= 0 || N <= 0) return 0;
  return ssd_segment_floats(batch, heads, P, N, max_rows);
}

// x [rows, heads * P], B and C [rows, groups * N], dt [rows, heads] (before its softplus), state
// [slots, heads, P, N], y [rows, heads * P]; rows lie sequence by sequence (cu_rows).  `max_rows`: the most rows a
// sequence brings (0: unknown); `scratch`: lq_ssd_scan_workspace(...) floats, or null (then no segments).
extern "C" int lq_ssd_scan(const float* x, int ldx, const float* Bm, int ldb, const float* Cm, int ldc, const float* dt,
                           int lddt, const float* dt_bias, const float* a_log, const float* d_skip, float* state, float* y,
                           int ldy, int heads, int P, int N, int groups, const int* seq_slot, const int* cu_rows, int batch,
                           int max_rows, float* scratch, long long scratch_floats, hipStream_t stream) {
  LQ_REQUIRE(heads > 0 && P > 0 && N > 0 && groups > 0 && heads % groups == 0 && batch > 0, "ssd_scan: bad sizes");
  LQ_REQUIRE(ldx >= heads * P && ldy >= heads * P && ldb >= groups * N && ldc >= groups * N && lddt >= heads,
             "ssd_scan: a row stride is smaller than its row");
  LQ_REQUIRE(x && Bm && Cm && dt && dt_bias && a_log && d_skip && state && y && seq_slot && cu_rows, "ssd_scan: null pointer");
  const long long need = scratch != nullptr ? ssd_segment_floats(batch, heads, P, N, max_rows) : 0;
  ScanLaunch cfg;
  LQ_REQUIRE(scan_launch(N, P, (long long)batch * heads * (need > 0 ? SEG_COUNT : 1), cfg),
             "ssd_scan: state size %d is too large", N);
  LQ_REQUIRE(need <= scratch_floats, "ssd_scan: %lld floats of scratch for a launch in segments, %lld given", need, scratch_floats);
  SegArgs sg = {1, 1, nullptr, nullptr};
  if (need > 0) {
    sg.nseg = SEG_COUNT;
    sg.state = scratch;
    sg.decay = scratch + (long long)batch * heads * SEG_COUNT * P * N;
  }
  ScanShape sh = {heads, groups, P, N, seq_slot, cu_rows};
#define LQ_SSD(LN, SL, TH)                                                                                              \
  ssd_scan_kernel<LN, SL, TH><<<grid, cfg.threads, cfg.lds, stream>>>(x, ldx, Bm, ldb, Cm, ldc, dt, lddt, dt_bias, a_log, \
                                                                  d_skip, state, y, ldy, sh, sg)
  dim3 grid((unsigned)(batch * heads), lq_ceil_div(P, cfg.cols), sg.nseg);
  LQ_SCAN_LANES(LQ_SSD)
  LQ_CHECK_LAUNCH("ssd_scan");
  if (sg.nseg > 1) {
    ssd_chain_kernel<<<dim3((unsigned)(batch * heads), lq_ceil_div(P * N, 256)), 256, 0, stream>>>(state, heads, P * N, sg,
                                                                                               seq_slot, cu_rows);
    LQ_CHECK_LAUNCH("ssd_scan(chain)");
    sg.pass = 2;
    LQ_SCAN_LANES(LQ_SSD)
    LQ_CHECK_LAUNCH("ssd_scan(second pass)");
  }
#undef LQ_SSD
  return 0;
}

// q and k [rows, kv_heads * Dk], v [rows, heads * P], beta and a [rows, heads] (raw), state [slots, heads, P, Dk],
// out [rows, heads * P]
// (q and k are made unit vectors in place)
// `channel_decay`: a [rows, heads * Dk] and dt_bias [heads * Dk], a decay for every key channel of every head
extern "C" int lq_delta_scan(float* q, int ldq, float* k, int ldk, const float* v, int ldv, const float* beta,
                             int ldbeta, const float* a, int lda, const float* dt_bias, const float* a_log, float* state,
                             float* out, int ldo, int heads, int kv_heads, int Dk, int P, float q_scale, float unit_eps,
                             const int* seq_slot, const int* cu_rows, int batch, int rows, int channel_decay,
                             hipStream_t stream) {
  LQ_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && Dk > 0 && P > 0 && batch > 0, "delta_scan: bad sizes");
  LQ_REQUIRE(ldq >= kv_heads * Dk && ldk >= kv_heads * Dk && ldv >= heads * P && ldo >= heads * P && ldbeta >= heads &&
                 lda >= (channel_decay ? heads * Dk : heads), "delta_scan: a row stride is smaller than its row");
  LQ_REQUIRE(q && k && v && beta && a && dt_bias && a_log && state && out && seq_slot && cu_rows, "delta_scan: null pointer");
  ScanLaunch cfg;
  LQ_REQUIRE(scan_launch(Dk, P, (long long)batch * heads, cfg), "delta_scan: key size %d is too large", Dk);
  LQ_REQUIRE(rows > 0 && rows <= 0x7fffffff && kv_heads <= 65535, "delta_scan: %d rows, %d q/k heads", rows, kv_heads);
  unit_heads_kernel<<<dim3((unsigned)rows, kv_heads), 64, 0, stream>>>(q, ldq, k, ldk, Dk, q_scale, unit_eps);
  LQ_CHECK_LAUNCH("delta_scan(unit vectors)");
  dim3 grid((unsigned)(batch * heads), lq_ceil_div(P, cfg.cols));
  ScanShape sh = {heads, kv_heads, P, Dk, seq_slot, cu_rows};
  if (channel_decay) {
    const int np = cfg.ln * cfg.slab;
    const bool single = rows == batch;  // every sequence brings one token
    const size_t lds = 2 * (size_t)(single ? 1 : dch_tokens(np, cfg.threads, cfg.ln)) * (3 * np + 2 * cfg.cols + 1) * sizeof(float);
    LQ_REQUIRE(lds <= 64 * 1024, "delta_scan: key size %d is too large", Dk);
#define LQ_DELTA_CH(LN, SL, TH)                                                                                          \
  do {                                                                                                                   \
    if (single)                                                                                                          \
      delta_channel_scan_kernel<LN, SL, TH, true><<<grid, cfg.threads, lds, stream>>>(                                   \
          q, ldq, k, ldk, v, ldv, beta, ldbeta, a, lda, dt_bias, a_log, state, out, ldo, sh);                            \
    else                                                                                                                 \
      delta_channel_scan_kernel<LN, SL, TH, false><<<grid, cfg.threads, lds, stream>>>(                                  \
          q, ldq, k, ldk, v, ldv, beta, ldbeta, a, lda, dt_bias, a_log, state, out, ldo, sh);                            \
  } while (0)
    LQ_SCAN_LANES(LQ_DELTA_CH)
#undef LQ_DELTA_CH
    LQ_CHECK_LAUNCH("delta_scan(channel decay)");
    return 0;
  }
#define LQ_DELTA(LN, SL, TH)                                                                                             \
  delta_scan_kernel<LN, SL, TH><<<grid, cfg.threads, cfg.lds, stream>>>(q, ldq, k, ldk, v, ldv, beta, ldbeta, a, lda,      \
                                                                    dt_bias, a_log, state, out, ldo, sh)
  LQ_SCAN_LANES(LQ_DELTA)
#undef LQ_DELTA
  LQ_CHECK_LAUNCH("delta_scan");
  return 0;
}

extern "C" int lq_gated_rmsnorm(const float* y, int ldy, const float* z, int ldz, const float* w, int wlen, float eps,
                                int group, void* out, int out_dtype, int ldo, int rows, int n, int gate_first,
                                int sigmoid_gate, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && n > 0 && group > 0 && n % group == 0, "gated_rmsnorm: %d columns in groups of %d", n, group);
  LQ_REQUIRE(wlen > 0 && (wlen == n || group % wlen == 0), "gated_rmsnorm: a weight of %d entries for groups of %d", wlen, group);
  LQ_REQUIRE(ldy >= n && ldz >= n && ldo >= n, "gated_rmsnorm: a row stride is smaller than its row");
  LQ_REQUIRE(y && z && w && out, "gated_rmsnorm: null pointer");
  const int threads = group >= 1024 ? 256 : group > 64 ? 128 : 64;
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    dim3 grid(n / group, nr);
    if (out_dtype == LQ_F32)
      gated_rmsnorm_kernel<float><<<grid, threads, 0, stream>>>(y + (long long)r0 * ldy, ldy, z + (long long)r0 * ldz, ldz, w,
                                                               wlen, eps, group, (float*)out + (long long)r0 * ldo, ldo, gate_first, sigmoid_gate);
    else if (out_dtype == LQ_BF16)
      gated_rmsnorm_kernel<bf16_t><<<grid, threads, 0, stream>>>(y + (long long)r0 * ldy, ldy, z + (long long)r0 * ldz, ldz, w,
                                                                wlen, eps, group, (bf16_t*)out + (long long)r0 * ldo, ldo, gate_first, sigmoid_gate);
    else
      LQ_REQUIRE(false, "gated_rmsnorm: unknown dtype %d", out_dtype);
  }
  LQ_CHECK_LAUNCH("gated_rmsnorm");
  return 0;
}

// stack [n_in, rows, width] dense float32; w0..w3 the branches' weights [width]
extern "C" int lq_rmsnorm_mean(const float* stack, int n_in, const float* w0, const float* w1, const float* w2,
                               const float* w3, float eps, float* out, int rows, int width, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && width > 0 && n_in >= 1 && n_in <= 4, "rmsnorm_mean: %d branches of %d x %d", n_in, rows, width);
  const float* ws[4] = {w0, w1, w2, w3};
  MeanInputs in;
  for (int i = 0; i < 4; ++i) {
    in.x[i] = i < n_in ? stack + (long long)i * rows * width : nullptr;
    in.w[i] = ws[i];
    LQ_REQUIRE(i >= n_in || ws[i] != nullptr, "rmsnorm_mean: branch %d has no weight", i);
  }
  LQ_REQUIRE(stack && out, "rmsnorm_mean: null pointer");
  rmsnorm_mean_kernel<<<rows, width >= 4096 ? 1024 : width >= 1024 ? 256 : 64, 0, stream>>>(in, n_in, eps, out, width);
  LQ_CHECK_LAUNCH("rmsnorm_mean");
  return 0;
}

// Whether a gated-linear-attention launch runs in segments, and then the float32 scratch it needs (as for the
// state-space scan: few long sequences that would leave most of the chip idle).
static long long gla_segment_floats(int batch, int heads, int P, int N, int max_rows) {
  ScanLaunch cfg;
  if (max_rows < SEG_MIN_ROWS || !scan_launch(N, P, 1ll << 40, cfg)) return 0;
  if ((long long)batch * heads * lq_ceil_div(P, cfg.cols) >= 4ll * lq_compute_units()) return 0;
  return (long long)batch * heads * SEG_COUNT * ((long long)P * N + N);
}

extern "C" long long lq_gla_scan_workspace(int batch, int heads, int P, int N, int max_rows) {
  if (batch <= 0 || heads <= 0 || P <= 0 || N <= 0) return 0;
  return gla_segment_floats(batch, heads, P, N, max_rows);
}

// q, k and z [rows, heads * Dk] (z: the decay's logits, before bias), v [rows, heads * P], bias [heads * Dk], state
// [slots, heads, P, Dk], out [rows, heads * P].  `max_rows`: the most rows a sequence brings (0: unknown); `scratch`:
// lq_gla_scan_workspace(...) floats, or null (then no segments).
extern "C" int lq_gla_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* z, int ldz,
                           const float* bias, float* state, float* out, int ldo, int heads, int Dk, int P, float q_scale,
                           float inv_tau, const int* seq_slot, const int* cu_rows, int batch, int max_rows, float* scratch,
                           long long scratch_floats, hipStream_t stream) {
  LQ_REQUIRE(heads > 0 && Dk > 0 && P > 0 && batch > 0, "gla_scan: bad sizes");
  LQ_REQUIRE(ldq >= heads * Dk && ldk >= heads * Dk && ldz >= heads * Dk && ldv >= heads * P && ldo >= heads * P,
             "gla_scan: a row stride is smaller than its row");
  LQ_REQUIRE(q && k && v && z && bias && state && out && seq_slot && cu_rows, "gla_scan: null pointer");
  const long long need = scratch != nullptr ? gla_segment_floats(batch, heads, P, Dk, max_rows) : 0;
  ScanLaunch cfg;
  LQ_REQUIRE(scan_launch(Dk, P, (long long)batch * heads, cfg), "gla_scan: key size %d is too large", Dk);
  LQ_REQUIRE(need <= scratch_floats, "gla_scan: %lld floats of scratch for a launch in segments, %lld given", need, scratch_floats);
  const int np = cfg.ln * cfg.slab;
  const size_t lds = 2 * (size_t)gla_tokens(np, cfg.threads, cfg.ln) * (3 * np + 2 * cfg.cols) * sizeof(float);
  LQ_REQUIRE(lds <= 64 * 1024, "gla_scan: key size %d is too large", Dk);
  SegArgs sg = {1, 1, nullptr, nullptr};
  if (need > 0) {
    sg.nseg = SEG_COUNT;
    sg.state = scratch;
    sg.decay = scratch + (long long)batch * heads * SEG_COUNT * P * Dk;
  }
  dim3 grid((unsigned)(batch * heads), lq_ceil_div(P, cfg.cols), sg.nseg);
  ScanShape sh = {heads, heads, P, Dk, seq_slot, cu_rows};
#define LQ_GLA(LN, SL, TH)                                                                                            \
  gla_scan_kernel<LN, SL, TH><<<grid, cfg.threads, lds, stream>>>(q, ldq, k, ldk, v, ldv, z, ldz, bias, state, out, ldo, \
                                                                  sh, q_scale, inv_tau, sg)
  LQ_SCAN_LANES(LQ_GLA)
  LQ_CHECK_LAUNCH("gla_scan");
  if (sg.nseg > 1) {
    gla_chain_kernel<<<dim3((unsigned)(batch * heads), (unsigned)lq_ceil_div64((long long)P * Dk, 256)), 256, 0, stream>>>(
        state, heads, P, Dk, sg, seq_slot, cu_rows);
    LQ_CHECK_LAUNCH("gla_scan(chain)");
    sg.pass = 2;
    LQ_SCAN_LANES(LQ_GLA)
    LQ_CHECK_LAUNCH("gla_scan(second pass)");
  }
#undef LQ_GLA
  return 0;
}

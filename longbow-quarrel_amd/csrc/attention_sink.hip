// Attention over a sliding window that also keeps the first tokens of a sequence, with an optional sink in the
// softmax's denominator, keys and values of different sizes, and an optional gate per head; over the paged cache.
//
// Row r of the step has position p = row_pos[r] in the sequence row_seq[r] and sees key t when t <= p and
// (p - t < window or t < keep_first); window = 0: every t <= p.  Query head h reads kv head h / (nh / nkv).
// score = q . k * scale; the softmax runs with a maximum that starts at 0 and a sum that starts at 1 when
// there is a sink (a key of score 0 without a value; with `sinks`, a learned score a query head that is not scaled:
// the maximum starts there), at -inf and 0 otherwise.  out = sum p_t v_t, times
// sigmoid(gate[r, h]) where a gate is given.  Scores, probabilities and sums are 32-bit for either dtype of
// q and the cache; the products run on the matrix cores in their 32-bit mode (v_mfma_f32_16x16x4_f32).
//
// Keys are walked in chunks of 64 aligned to absolute positions, the kept first chunks before the window's, so
// the order of every sum depends on the row's position only: not on how the tokens were cut into steps nor on
// what else is in the batch.
//
// Cache layout: K[block][kv head][offset][key size], V[block][kv head][value size][offset].
//
// `maps` > 1: nkv counts key heads of which every `maps` neighbours share one value head, and a cached key row
// holds their keys side by side, K[block][value head][offset][map][key size], V[block][value head][...]: key head j
// reads map j % maps of value head j / maps (differential attention: two score maps over the same values).
// `out_f32`: out is 32-bit whatever the dtype of q and the cache.
#include "common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ inline f32x4 ld4(const float* p) { return *(const f32x4*)p; }
__device__ inline f32x4 ld4(const bf16_t* p) {
  const uint2 v = *(const uint2*)p;
  f32x4 r;
  r.x = __uint_as_float(v.x << 16);
  r.y = __uint_as_float(v.x & 0xffff0000u);
  r.z = __uint_as_float(v.y << 16);
  r.w = __uint_as_float(v.y & 0xffff0000u);
  return r;
}

struct SinkArgs {
  int ldq, ldo, ldg, rows, rows_per_tile, heads_per_tile, nh, nkv, KD, VD;
  const int *row_pos, *row_seq, *seq_slot, *block_table;
  int bt_stride, BS;
  float scale;
  int window, keep_first, sink;
  // single tokens of a bfloat16 run may share a tile's keys out over `ksplit` workgroups (blockIdx.z): each takes
  // the rounds of SPLIT chunks whose number is its own modulo ksplit and leaves its partial result in `part`,
  // which a second launch merges in the order of the workgroups
  int ksplit;
  float* part;
  int maps, out_f32;
  const float* sinks;  // null: the sink's score is 0
};

template <typename T>
__device__ inline void put_out(T* out, long long at, float v, int out_f32) {
  if (out_f32) ((float*)out)[at] = v;
  else out[at] = from_f32<T>(v);
}

constexpr int MAX_KD = 256;

// A workgroup of SPLIT wavefronts takes up to 16 consecutive rows of the step and one query head.  For every
// sequence with rows in the tile it walks the chunks that any of these rows sees, wavefront w the chunks whose
// number (position / 64) is w modulo SPLIT; rows of other sequences and keys that a row does not see take part with
// weight zero.  Per chunk: S^T = K . Q^T (16 keys by 16 rows a product), the softmax of every row over its 64
// scores, O += P . V with the probabilities straight from the registers of the scores.  At the end the wavefronts'
// partial results (maximum, sum, weighted values) meet in LDS and are merged in the order of the wavefronts.  Which
// wavefront takes which chunk follows from positions alone, so a row's sums are the same in every launch.
// A lane (c, g) keeps the part of row c's query that it multiplies (dimensions 16 s + 4 g .. + 3 of every slab s) in
// LDS, where only it reads it: the key size is then a loop bound and no template parameter.  bfloat16 keys and
// queries are multiplied as they are (v_mfma_f32_16x16x16_bf16: the products are exact, the sums 32-bit); the
// probabilities stay 32-bit and meet the widened values in the 32-bit product.
constexpr int SPLIT = 4;
typedef short bf16x4 __attribute__((ext_vector_type(4)));

template <typename T, int HSV>  // HSV: value size / 16
__global__ __launch_bounds__(64 * SPLIT) void sink_tiles_kernel(const T* __restrict__ q, T* __restrict__ out,
                                                                const T* __restrict__ gate,
                                                                const T* __restrict__ kcache,
                                                                const T* __restrict__ vcache, SinkArgs a) {
  constexpr bool HALF = sizeof(T) == 2;
  constexpr int QROW = MAX_KD / 4 + 4;             // a lane's own run of q, padded against bank clashes
  constexpr int PART = 64 * (HSV * 4) + 32;        // a wavefront's partial result: o of every lane, then m and l of 16 rows
  constexpr int LDS_FLOATS = 64 * QROW > (SPLIT - 1) * PART ? 64 * QROW : (SPLIT - 1) * PART;
  __shared__ float smem[LDS_FLOATS];               // first the queries, at the end the partial results
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  // The tile's 16 rows are rows_per_tile rows of the step times heads_per_tile query heads that share a kv head
  // (tile row c: step row c / heads_per_tile, head c % heads_per_tile): their keys and values are read once.
  const int GH = a.heads_per_tile;
  const int hbase = blockIdx.y * GH, kvh = hbase / (a.nh / a.nkv);
  const int nvh = a.nkv / a.maps, vh = kvh / a.maps, kmap = kvh % a.maps;  // value heads; this tile's, and its map
  const long long krow = (long long)a.maps * a.KD;                          // a cached key row of one value head
  const int r0 = blockIdx.x * a.rows_per_tile;
  const int n_rows = min(a.rows_per_tile, a.rows - r0);
  const int HS = a.KD / 16, BS = a.BS;
  const int my_row = r0 + min(c / GH, n_rows - 1), h = hbase + c % GH;
  const int my_pos = a.row_pos[my_row], my_seq = a.row_seq[my_row];
  const int my_lo = (a.window > 0 && my_pos >= a.window) ? my_pos - a.window + 1 : 0;
  float* myq = smem + (g * 16 + c) * QROW;
  if (wave == 0) {
    for (int sl = 0; sl < HS; ++sl) {
      const T* src = q + (long long)my_row * a.ldq + h * a.KD + sl * 16 + 4 * g;
      if constexpr (HALF) *(uint2*)(myq + 4 * sl) = *(const uint2*)src;
      else *(f32x4*)(myq + 4 * sl) = ld4(src);
    }
  }
  __syncthreads();

  // the sink is one more key of score 0 without a value: the first wavefront starts from it
  const bool with_sink = a.sink && wave == 0 && blockIdx.z == 0;
  float m = with_sink ? (a.sinks != nullptr ? a.sinks[h] : 0.f) : -INFINITY, l = with_sink ? 1.f : 0.f;
  f32x4 o[HSV];  // o[dt][e]: row 4 g + e of the tile, value dimension 16 dt + c
#pragma unroll
  for (int dt = 0; dt < HSV; ++dt) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int seq_first = __builtin_amdgcn_readfirstlane(a.row_seq[r0]);
  const int seq_last = __builtin_amdgcn_readfirstlane(a.row_seq[r0 + n_rows - 1]);
  for (int seq = seq_first; seq <= seq_last; ++seq) {
    const bool mine = my_seq == seq && c / GH < n_rows;
    int lo_min = mine ? my_lo : 0x7fffffff, pos_max = mine ? my_pos : -1;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      lo_min = min(lo_min, __shfl_xor(lo_min, off, 64));
      pos_max = max(pos_max, __shfl_xor(pos_max, off, 64));
    }
    lo_min = __builtin_amdgcn_readfirstlane(lo_min);
    pos_max = __builtin_amdgcn_readfirstlane(pos_max);
    if (pos_max < 0) continue;
    const int* table = a.block_table + (long long)a.seq_slot[seq] * a.bt_stride;
    const int wstart = (lo_min / 64) * 64;           // first chunk of the window of any of these rows
    const int kept_end = min(a.keep_first, wstart);  // kept keys that lie below that chunk
    int t0 = kept_end > 0 ? 0 : wstart;
    while (t0 <= pos_max) {
      if (((t0 >> 6) & (SPLIT - 1)) == wave && (a.ksplit == 1 || (t0 >> 8) % a.ksplit == (int)blockIdx.z)) {
        f32x4 st[4];  // st[kt][e]: score of key t0 + 16 kt + 4 g + e for row c
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
          st[kt] = (f32x4){0.f, 0.f, 0.f, 0.f};
          const int t = min(t0 + 16 * kt + c, pos_max);  // this lane's key as an operand row (clamped: finite, masked below)
          const long long blk = table[t / BS];
          const T* kr = kcache + ((blk * nvh + vh) * BS + t % BS) * krow + kmap * a.KD + 4 * g;
          if constexpr (HALF) {
            for (int sl = 0; sl < HS; ++sl) {
              const uint2 kv = *(const uint2*)(kr + sl * 16);
              const uint2 qv = *(const uint2*)(myq + 4 * sl);
              st[kt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(bf16x4, kv),
                                                                 __builtin_bit_cast(bf16x4, qv), st[kt], 0, 0, 0);
            }
          } else {
            for (int sl = 0; sl < HS; ++sl) {
              const f32x4 kv = ld4(kr + sl * 16);
              const f32x4 qv = *(const f32x4*)(myq + 4 * sl);
#pragma unroll
              for (int j = 0; j < 4; ++j) st[kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[j], qv[j], st[kt], 0, 0, 0);
            }
          }
        }
        float cmax = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int t = t0 + 16 * kt + 4 * g + e;
            const bool valid = mine && t <= my_pos && (t >= my_lo || t < a.keep_first);
            st[kt][e] = valid ? st[kt][e] * a.scale : -INFINITY;
            cmax = fmaxf(cmax, st[kt][e]);
          }
        cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
        cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
        const float m_new = fmaxf(m, cmax);
        const bool none = m_new == -INFINITY;  // no key of this row so far and no sink: nothing changes
        const float alpha = none ? 1.f : expf(m - m_new);
        float psum = 0.f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            st[kt][e] = none ? 0.f : expf(st[kt][e] - m_new);
            psum += st[kt][e];
          }
        psum += __shfl_xor(psum, 16, 64);
        psum += __shfl_xor(psum, 32, 64);
        l = l * alpha + psum;
        m = m_new;
        float a4[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) a4[e] = __shfl(alpha, 4 * g + e, 64);
#pragma unroll
        for (int dt = 0; dt < HSV; ++dt)
#pragma unroll
          for (int e = 0; e < 4; ++e) o[dt][e] *= a4[e];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
          // V^T of this lane's dimension 16 dt + c at keys t0 + 16 kt + 4 g .. + 3 (within one block)
          const int t = min(t0 + 16 * kt + 4 * g, pos_max) & ~3;
          const long long blk = table[t / BS];
          const T* vr = vcache + ((blk * nvh + vh) * (long long)(HSV * 16) + c) * BS + t % BS;
          f32x4 vv[HSV];
#pragma unroll
          for (int dt = 0; dt < HSV; ++dt) vv[dt] = ld4(vr + (long long)dt * 16 * BS);
#pragma unroll
          for (int dt = 0; dt < HSV; ++dt)
#pragma unroll
            for (int j = 0; j < 4; ++j) o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(st[kt][j], vv[dt][j], o[dt], 0, 0, 0);
        }
      }
      t0 += 64;
      if (t0 >= kept_end && t0 < wstart) t0 = wstart;  // from the kept first tokens on to the window
    }
  }
  // the wavefronts' partial results meet: 1 .. SPLIT - 1 leave theirs in LDS, the first merges them in order
  __syncthreads();  // (the queries are no longer needed: their room is taken)
  if (wave > 0) {
    float* part = smem + (wave - 1) * PART;
#pragma unroll
    for (int dt = 0; dt < HSV; ++dt) *(f32x4*)(part + (dt * 64 + lane) * 4) = o[dt];
    if (g == 0) part[64 * HSV * 4 + c] = m, part[64 * HSV * 4 + 16 + c] = l;
  }
  __syncthreads();
  if (wave > 0) return;
  float m4[4];  // the running maximum of the rows 4 g + e that this lane's accumulators belong to
#pragma unroll
  for (int e = 0; e < 4; ++e) m4[e] = __shfl(m, 4 * g + e, 64);
  for (int w = 1; w < SPLIT; ++w) {
    const float* part = smem + (w - 1) * PART;
    const float mw = part[64 * HSV * 4 + c], lw = part[64 * HSV * 4 + 16 + c];
    const float m_new = fmaxf(m, mw);
    const bool none = m_new == -INFINITY;
    l = none ? 0.f : l * expf(m - m_new) + lw * expf(mw - m_new);
    m = m_new;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float mo = part[64 * HSV * 4 + 4 * g + e];
      const float mn = fmaxf(m4[e], mo);
      const float fa = mn == -INFINITY ? 0.f : expf(m4[e] - mn), fb = mn == -INFINITY ? 0.f : expf(mo - mn);
      m4[e] = mn;
#pragma unroll
      for (int dt = 0; dt < HSV; ++dt) o[dt][e] = o[dt][e] * fa + part[(dt * 64 + lane) * 4 + e] * fb;
    }
  }
  if (a.ksplit > 1) {  // this workgroup's share of the keys: the merge launch finishes the tile
    float* mine_part = a.part + (((long long)blockIdx.y * gridDim.x + blockIdx.x) * a.ksplit + blockIdx.z) * PART;
#pragma unroll
    for (int dt = 0; dt < HSV; ++dt) *(f32x4*)(mine_part + (dt * 64 + lane) * 4) = o[dt];
    if (g == 0) mine_part[64 * HSV * 4 + c] = m, mine_part[64 * HSV * 4 + 16 + c] = l;
    return;
  }
  float inv4[4];
  const float inv = 1.0f / l;
#pragma unroll
  for (int e = 0; e < 4; ++e) inv4[e] = __shfl(inv, 4 * g + e, 64);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int tr = 4 * g + e, row = tr / GH, hh = hbase + tr % GH;  // tile row -> step row and head
    if (row < n_rows) {
      float f = inv4[e];
      if (gate != nullptr) f /= 1.f + expf(-to_f32(gate[(long long)(r0 + row) * a.ldg + hh]));
      const long long orow = (long long)(r0 + row) * a.ldo + hh * (HSV * 16) + c;
#pragma unroll
      for (int dt = 0; dt < HSV; ++dt) put_out(out, orow + dt * 16, o[dt][e] * f, a.out_f32);
    }
  }
}

// The partial results of the `ksplit` workgroups of a tile, merged in their order (as the wavefronts of a workgroup
// are), then the division by the sum, the gate and the store.  One wavefront a tile.
template <typename T, int HSV>
__global__ __launch_bounds__(64) void sink_merge_kernel(T* __restrict__ out, const T* __restrict__ gate, SinkArgs a) {
  constexpr int PART = 64 * (HSV * 4) + 32;
  const int lane = threadIdx.x, c = lane & 15, g = lane >> 4;
  const int GH = a.heads_per_tile, hbase = blockIdx.y * GH, r0 = blockIdx.x * a.rows_per_tile;
  const int n_rows = min(a.rows_per_tile, a.rows - r0);
  const float* part = a.part + ((long long)blockIdx.y * gridDim.x + blockIdx.x) * a.ksplit * PART;
  f32x4 o[HSV];
#pragma unroll
  for (int dt = 0; dt < HSV; ++dt) o[dt] = *(const f32x4*)(part + (dt * 64 + lane) * 4);
  float m = part[64 * HSV * 4 + c], l = part[64 * HSV * 4 + 16 + c];
  float m4[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) m4[e] = part[64 * HSV * 4 + 4 * g + e];
  for (int w = 1; w < a.ksplit; ++w) {
    part += PART;
    const float mw = part[64 * HSV * 4 + c], lw = part[64 * HSV * 4 + 16 + c];
    const float m_new = fmaxf(m, mw);
    const bool none = m_new == -INFINITY;
    l = none ? 0.f : l * expf(m - m_new) + lw * expf(mw - m_new);
    m = m_new;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float mo = part[64 * HSV * 4 + 4 * g + e];
      const float mn = fmaxf(m4[e], mo);
      const float fa = mn == -INFINITY ? 0.f : expf(m4[e] - mn), fb = mn == -INFINITY ? 0.f : expf(mo - mn);
      m4[e] = mn;
#pragma unroll
      for (int dt = 0; dt < HSV; ++dt) o[dt][e] = o[dt][e] * fa + part[(dt * 64 + lane) * 4 + e] * fb;
    }
  }
  const float inv = 1.0f / l;
  float inv4[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) inv4[e] = __shfl(inv, 4 * g + e, 64);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int tr = 4 * g + e, row = tr / GH, hh = hbase + tr % GH;
    if (row < n_rows) {
      float f = inv4[e];
      if (gate != nullptr) f /= 1.f + expf(-to_f32(gate[(long long)(r0 + row) * a.ldg + hh]));
      const long long orow = (long long)(r0 + row) * a.ldo + hh * (HSV * 16) + c;
#pragma unroll
      for (int dt = 0; dt < HSV; ++dt) put_out(out, orow + dt * 16, o[dt][e] * f, a.out_f32);
    }
  }
}

// Any sizes: one wavefront per (row, head), a lane a key of the chunk for the scores and a value dimension (or
// several) for the sums.
constexpr int MAX_DIM = 1024;

template <typename T>
__global__ __launch_bounds__(64) void sink_rows_kernel(const T* __restrict__ q, T* __restrict__ out,
                                                       const T* __restrict__ gate, const T* __restrict__ kcache,
                                                       const T* __restrict__ vcache, SinkArgs a) {
  __shared__ float qs[MAX_DIM];
  __shared__ float ps[64];
  __shared__ long long vbase[64];
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (a.nh / a.nkv), BS = a.BS, KD = a.KD, VD = a.VD;
  const int nvh = a.nkv / a.maps, g = kvh / a.maps, kmap = kvh % a.maps;  // g: the value head
  const int p = a.row_pos[r];
  const int lo = (a.window > 0 && p >= a.window) ? p - a.window + 1 : 0;
  const int* table = a.block_table + (long long)a.seq_slot[a.row_seq[r]] * a.bt_stride;
  for (int d = lane; d < KD; d += 64) qs[d] = to_f32(q[(long long)r * a.ldq + h * KD + d]);
  float m = a.sink ? (a.sinks != nullptr ? a.sinks[h] : 0.f) : -INFINITY, l = a.sink ? 1.f : 0.f;
  float acc[MAX_DIM / 64];
#pragma unroll
  for (int j = 0; j < MAX_DIM / 64; ++j) acc[j] = 0.f;
  const int wstart = (lo / 64) * 64, kept_end = min(a.keep_first, wstart);
  int t0 = kept_end > 0 ? 0 : wstart;
  while (t0 <= p) {
    const int t = t0 + lane;
    const bool valid = t <= p && (t >= lo || t < a.keep_first);
    __syncthreads();
    float s = -INFINITY;
    if (valid) {
      const long long blk = table[t / BS];
      const int off = t % BS;
      vbase[lane] = (blk * nvh + g) * (long long)VD * BS + off;
      const T* kr = kcache + ((blk * nvh + g) * BS + off) * (long long)a.maps * KD + kmap * KD;
      float dot = 0.f;
      for (int d = 0; d < KD; ++d) dot = fmaf(qs[d], to_f32(kr[d]), dot);
      s = dot * a.scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const bool none = m_new == -INFINITY;
    const float alpha = none ? 1.f : expf(m - m_new);
    ps[lane] = (valid && !none) ? expf(s - m_new) : 0.f;
    __syncthreads();
    const int nchunk = min(64, p - t0 + 1);
    float psum = 0.f;
    for (int i = 0; i < nchunk; ++i) psum += ps[i];
    l = l * alpha + psum;
#pragma unroll
    for (int j = 0; j < MAX_DIM / 64; ++j) {
      const int d = lane + 64 * j;
      if (d < VD) {
        float v = acc[j] * alpha;
        for (int i = 0; i < nchunk; ++i) {
          const float w = ps[i];
          if (w != 0.f) v = fmaf(w, to_f32(vcache[vbase[i] + (long long)d * BS]), v);
        }
        acc[j] = v;
      }
    }
    m = m_new;
    t0 += 64;
    if (t0 >= kept_end && t0 < wstart) t0 = wstart;
  }
  float f = 1.0f / l;
  if (gate != nullptr) f /= 1.f + expf(-to_f32(gate[(long long)r * a.ldg + h]));
#pragma unroll
  for (int j = 0; j < MAX_DIM / 64; ++j) {
    const int d = lane + 64 * j;
    if (d < VD) put_out(out, (long long)r * a.ldo + h * VD + d, acc[j] * f, a.out_f32);
  }
}

// k [rows, nkv * KD], v [rows, nkv * VD] into the paged cache at the rows' positions
template <typename T>
__global__ __launch_bounds__(256) void kv_store_kernel(const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
                                                       int nkv, int KD, int VD, const int* __restrict__ row_pos,
                                                       const int* __restrict__ row_seq, const int* __restrict__ seq_slot,
                                                       const int* __restrict__ block_table, int bt_stride,
                                                       T* __restrict__ kcache, T* __restrict__ vcache, int BS) {
  const int r = blockIdx.x;
  const int p = row_pos[r];
  const long long blk = block_table[(long long)seq_slot[row_seq[r]] * bt_stride + p / BS];
  const int off = p % BS;
  for (int e = threadIdx.x; e < nkv * KD; e += 256) {
    const int g = e / KD, d = e - g * KD;
    kcache[((blk * nkv + g) * BS + off) * (long long)KD + d] = k[(long long)r * ldk + e];
  }
  for (int e = threadIdx.x; e < nkv * VD; e += 256) {
    const int g = e / VD, d = e - g * VD;
    vcache[((blk * nkv + g) * (long long)VD + d) * BS + off] = v[(long long)r * ldv + e];
  }
}

// How a launch is cut into tiles, and over how many workgroups a tile's keys are shared out: one decision for the
// query about scratch and for the launch.  Keys are shared out for single tokens of a bfloat16 run only (a float32
// row's sums keep the one order that depends on its position alone), where the tiles alone leave most of the chip
// idle and a wavefront would walk several rounds of chunks.
struct TileShape {
  bool tiles;
  int heads_per_tile, rows_per_tile, grid_x, grid_y, ksplit;
  long long part_floats;  // scratch for the partial results (0: no sharing out)
};

TileShape tile_shape(int el, int rows, int batch, int nh, int nkv, int KD, int VD, int BS, int window, int keep_first,
                     int max_len) {
  TileShape t = {false, 1, 1, 0, 0, 1, 0};
  if (KD % 16 != 0 || VD % 16 != 0 || KD > MAX_KD || VD > 256 || BS % 16 != 0) return t;
  const int hsv = VD / 16;
  if (!(hsv <= 10 || hsv == 12 || hsv == 16)) return t;
  t.tiles = true;
  // the query heads of a kv head share a tile where their number is a power of two (or a multiple of 16)
  const int group = nh / nkv;
  t.heads_per_tile = group % 16 == 0 ? 16 : (group & (group - 1)) == 0 ? group : 1;
  t.rows_per_tile = rows == batch ? 1 : 16 / t.heads_per_tile;  // single tokens: a tile a row of the step
  t.grid_x = lq_ceil_div(rows, t.rows_per_tile), t.grid_y = nh / t.heads_per_tile;
  if (el == 2 && rows == batch && max_len > 0) {
    const int keys = window > 0 ? (max_len < window + keep_first + 128 ? max_len : window + keep_first + 128) : max_len;
    const int rounds = lq_ceil_div(lq_ceil_div(keys, 64), SPLIT);
    const long long tiles = (long long)t.grid_x * t.grid_y;
    long long k = 2ll * lq_compute_units() / (tiles > 0 ? tiles : 1);
    if (k > rounds) k = rounds;
    if (k > 8) k = 8;
    if (k >= 2) {
      t.ksplit = (int)k;
      t.part_floats = tiles * k * (64ll * hsv * 4 + 32);
    }
  }
  return t;
}

template <typename T>
bool launch_tiles(const void* q, void* out, const void* gate, const void* kcache, const void* vcache, const SinkArgs& a,
                  int batch, int max_len, float* part, long long part_floats, hipStream_t stream) {
  const int el = (int)sizeof(T);
  if (a.ldq % 4 != 0 || ((uintptr_t)q % (4 * el)) != 0 || ((uintptr_t)kcache % (4 * el)) != 0 ||
      ((uintptr_t)vcache % (4 * el)) != 0)
    return false;
  const TileShape t = tile_shape(el, a.rows, batch, a.nh, a.nkv, a.KD, a.VD, a.BS, a.window, a.keep_first,
                                 part != nullptr ? max_len : 0);
  if (!t.tiles) return false;
  SinkArgs b = a;
  b.heads_per_tile = t.heads_per_tile, b.rows_per_tile = t.rows_per_tile;
  b.ksplit = t.part_floats > 0 && t.part_floats <= part_floats ? t.ksplit : 1;
  b.part = part;
  dim3 grid(t.grid_x, t.grid_y, b.ksplit);
#define LQ_SINK(HSV)                                                                                                  \
  case HSV:                                                                                                           \
    sink_tiles_kernel<T, HSV><<<grid, 64 * SPLIT, 0, stream>>>((const T*)q, (T*)out, (const T*)gate, (const T*)kcache,        \
                                                       (const T*)vcache, b);                                          \
    if (b.ksplit > 1) sink_merge_kernel<T, HSV><<<dim3(t.grid_x, t.grid_y), 64, 0, stream>>>((T*)out, (const T*)gate, b);   \
    return true;
  switch (a.VD / 16) {
    LQ_SINK(1) LQ_SINK(2) LQ_SINK(3) LQ_SINK(4) LQ_SINK(5) LQ_SINK(6) LQ_SINK(7) LQ_SINK(8) LQ_SINK(9) LQ_SINK(10)
    LQ_SINK(12) LQ_SINK(16)
  }
#undef LQ_SINK
  return false;
}

}  // namespace

extern "C" int lq_kv_store(const void* k, int ldk, const void* v, int ldv, int dtype, int rows, int nkv, int KD, int VD,
                           const int* row_pos, const int* row_seq, const int* seq_slot, const int* block_table,
                           int bt_stride, void* kcache, void* vcache, int block_size, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && nkv > 0 && KD > 0 && VD > 0 && block_size > 0 && bt_stride > 0, "kv_store: bad sizes");
  LQ_REQUIRE(ldk >= nkv * KD && ldv >= nkv * VD, "kv_store: a row stride is smaller than its row");
  LQ_REQUIRE(k && v && row_pos && row_seq && seq_slot && block_table && kcache && vcache, "kv_store: null pointer");
  if (dtype == LQ_F32)
    kv_store_kernel<float><<<rows, 256, 0, stream>>>((const float*)k, ldk, (const float*)v, ldv, nkv, KD, VD, row_pos, row_seq,
                                                     seq_slot, block_table, bt_stride, (float*)kcache, (float*)vcache, block_size);
  else if (dtype == LQ_BF16)
    kv_store_kernel<bf16_t><<<rows, 256, 0, stream>>>((const bf16_t*)k, ldk, (const bf16_t*)v, ldv, nkv, KD, VD, row_pos,
                                                      row_seq, seq_slot, block_table, bt_stride, (bf16_t*)kcache,
                                                      (bf16_t*)vcache, block_size);
  else
    LQ_REQUIRE(false, "kv_store: unknown dtype %d", dtype);
  LQ_CHECK_LAUNCH("kv_store");
  return 0;
}

// Float32 entries of scratch with which a launch of single tokens shares its keys out over several workgroups a tile
// (0: it does not).  `max_len`: an upper bound of the sequences' lengths.
extern "C" long long lq_sink_attention_workspace(int dtype, int rows, int batch, int nh, int nkv, int KD, int VD,
                                                 int block_size, int window, int keep_first, int max_len) {
  if (rows <= 0 || batch <= 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || block_size <= 0) return 0;
  return tile_shape(dtype == LQ_BF16 ? 2 : 4, rows, batch, nh, nkv, KD, VD, block_size, window, keep_first, max_len).part_floats;
}

// `gate`: null, or [rows, nh] logits (stride ldg) in the dtype of q.  `rows == batch` means single tokens.  `part`:
// lq_sink_attention_workspace(...) floats for `max_len`, or null.
extern "C" int lq_sink_attention(const void* q, int ldq, void* out, int ldo, const void* gate, int ldg, int dtype, int rows,
                                 int batch, int nh, int nkv, int KD, int VD, const int* row_pos, const int* row_seq,
                                 const int* seq_slot, const int* block_table, int bt_stride, const void* kcache,
                                 const void* vcache, int block_size, float scale, int window, int keep_first, int sink,
                                 int force_rows, int max_len, float* part, long long part_floats, const float* sinks,
                                 int maps, int out_f32, hipStream_t stream) {
  LQ_REQUIRE(maps >= 1 && nkv % maps == 0, "sink_attention: %d key heads in runs of %d that share a value head", nkv, maps);
  LQ_REQUIRE(sinks == nullptr || sink, "sink_attention: learned sink scores without a sink");
  LQ_REQUIRE(rows > 0 && batch > 0 && rows >= batch, "sink_attention: rows %d and sequences %d", rows, batch);
  LQ_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0 && nh <= 65535, "sink_attention: %d heads over %d kv heads", nh, nkv);
  LQ_REQUIRE(KD > 0 && VD > 0 && KD <= MAX_DIM && VD <= MAX_DIM, "sink_attention: key size %d, value size %d", KD, VD);
  LQ_REQUIRE(block_size > 0 && bt_stride > 0 && window >= 0 && keep_first >= 0, "sink_attention: bad sizes");
  LQ_REQUIRE(ldq >= nh * KD && ldo >= nh * VD && (gate == nullptr || ldg >= nh), "sink_attention: a row stride is smaller than its row");
  LQ_REQUIRE(q && out && row_pos && row_seq && seq_slot && block_table && kcache && vcache, "sink_attention: null pointer");
  LQ_REQUIRE(dtype == LQ_F32 || dtype == LQ_BF16, "sink_attention: unknown dtype %d", dtype);
  SinkArgs a;
  a.ldq = ldq, a.ldo = ldo, a.ldg = ldg, a.rows = rows, a.rows_per_tile = 1, a.heads_per_tile = 1, a.nh = nh, a.nkv = nkv, a.KD = KD, a.VD = VD;
  a.row_pos = row_pos, a.row_seq = row_seq, a.seq_slot = seq_slot, a.block_table = block_table;
  a.bt_stride = bt_stride, a.BS = block_size, a.scale = scale, a.window = window, a.keep_first = keep_first, a.sink = sink;
  a.ksplit = 1, a.part = nullptr;
  a.maps = maps, a.out_f32 = out_f32 || dtype == LQ_F32, a.sinks = sinks;
  if (!force_rows) {
    const bool done = dtype == LQ_F32
                          ? launch_tiles<float>(q, out, gate, kcache, vcache, a, batch, max_len, part, part_floats, stream)
                          : launch_tiles<bf16_t>(q, out, gate, kcache, vcache, a, batch, max_len, part, part_floats, stream);
    if (done) {
      LQ_CHECK_LAUNCH("sink_attention(tiles)");
      return 0;
    }
  }
  LQ_REQUIRE(rows <= 0x7fffffff, "sink_attention: too many rows");
  dim3 grid(rows, nh);
  if (dtype == LQ_F32)
    sink_rows_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, (float*)out, (const float*)gate, (const float*)kcache,
                                                     (const float*)vcache, a);
  else
    sink_rows_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)gate,
                                                      (const bf16_t*)kcache, (const bf16_t*)vcache, a);
  LQ_CHECK_LAUNCH("sink_attention(rows)");
  return 0;
}


namespace {

// both [rows, kv heads, 2, group, VD] (32-bit: the two maps' results of the query heads of every key/value head),
// out [rows, heads, VD]: o = a1 - lam a2, divided by its root mean square over VD (eps inside the root), times gain.
// One wavefront a (row, head).
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const float* __restrict__ both, int ldb, T* __restrict__ out,
                                                           int ldo, int nh, int group, int VD, float lam, float eps,
                                                           float gain) {
  const int r = blockIdx.x, lane = threadIdx.x & 63;
  const int h = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (h >= nh) return;
  const int kv = h / group, hg = h % group;
  const float* a1 = both + (long long)r * ldb + ((long long)(kv * 2) * group + hg) * VD;
  const float* a2 = a1 + (long long)group * VD;
  float ss = 0.f;
  for (int d = lane; d < VD; d += 64) {
    const float o = a1[d] - lam * a2[d];
    ss = fmaf(o, o, ss);
  }
  const float inv = gain / sqrtf(wave_sum(ss) / (float)VD + eps);
  T* orow = out + (long long)r * ldo + (long long)h * VD;
  for (int d = lane; d < VD; d += 64) orow[d] = from_f32<T>((a1[d] - lam * a2[d]) * inv);
}

}  // namespace

extern "C" int lq_diff_combine(const float* both, int ldb, void* out, int out_dtype, int ldo, int rows, int nh, int nkv,
                               int VD, float lam, float eps, float gain, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && rows <= 0x7fffffff && nh > 0 && nkv > 0 && nh % nkv == 0 && VD > 0, "diff_combine: rows %d, %d heads over %d, size %d",
             rows, nh, nkv, VD);
  LQ_REQUIRE(ldb >= 2 * nh * VD && ldo >= nh * VD, "diff_combine: a row stride is smaller than its row");
  LQ_REQUIRE(both && out, "diff_combine: null pointer");
  LQ_REQUIRE(lq_ceil_div(nh, 4) <= 65535, "diff_combine: too many heads");
  const dim3 grid(rows, lq_ceil_div(nh, 4));
  if (out_dtype == LQ_F32)
    diff_combine_kernel<float><<<grid, 256, 0, stream>>>(both, ldb, (float*)out, ldo, nh, nh / nkv, VD, lam, eps, gain);
  else if (out_dtype == LQ_BF16)
    diff_combine_kernel<bf16_t><<<grid, 256, 0, stream>>>(both, ldb, (bf16_t*)out, ldo, nh, nh / nkv, VD, lam, eps, gain);
  else LQ_REQUIRE(false, "diff_combine: unknown dtype %d", out_dtype);
  LQ_CHECK_LAUNCH("diff_combine");
  return 0;
}

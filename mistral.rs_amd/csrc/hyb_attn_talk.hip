// hyb_attn_talk.hip -- paged sigmoid attention with a distance bias and mixed head scores, on ragged batches (same batch description as hyb_kernels.hip).
//
// Query i of head g scores key j as   s_g = scale (q_g . k_j) - slope_g (i - j);   the heads' scores of one (i, j) pair are mixed,   s'_h = sum_g talk[h, g] s_g;   a visible
// key (0 <= i - j < window; window <= 0: every j <= i) weighs   p_h = sigmoid(s'_h + pb_h)   -- no normalisation over the keys, so there is no running maximum or sum and
// the keys can be consumed in any order --   o_h = sum_j p_h v_j,   and the head's output is multiplied by sigmoid(gate logit of (row, h)).  Scores, weights and sums are f32.
//
// Because every output head needs the scores of ALL heads, one workgroup (NT = 256 or 512 threads) owns NQ consecutive rows of one entry (a tile of a segment; NQ = 1 for
// decoded tokens) for every head.  Keys go by in passes of 64:
//   A  wave w scores heads w, w + NT / 64, ..: a lane = a key, its row is read in 16-byte loads and multiplied with the NQ query vectors in LDS      -> s [H][64][NQ] (LDS)
//   B  a thread = (4 output heads, key, query): sum over g with talk^T rows as float4 broadcasts, visibility, sigmoid                            -> p [H][64][NQ] (LDS)
//   C  a thread = IT x (head, VW values): the values of key j are read once (one 16-byte load when VW = 8) and added into the NQ accumulators (registers).  When there
//      are fewer (head, value group) items than threads, JS thread groups share the keys of a pass (j = group, group + JS, ..) and their sums meet in LDS at the end
// Few rows (decoded tokens): the passes are dealt to KS workgroups per tile (grid.z); since the sum over keys has no normaliser the partial sums simply add -- they go to
// an f32 scratch [KS][rows][H * Dv] and a second kernel adds them in a fixed order, applies the gate and rounds.
// Grouped heads: query head h reads key / value head h / (H / G).
#include "common.cuh"
#include <float.h>
#include <stdlib.h>

namespace mrs {
namespace hyb {

static thread_local char g_terr[256];
static int tfail(const char *m) { snprintf(g_terr, sizeof g_terr, "%s", m); return 1; }

struct TalkArgs {
  const void *q;            // [rows, H * D] in T
  const void *k_cache, *v_cache;  // [blocks, G, block_size, D | Dv] in T
  const int *block_tables;  // [entries, max_blocks]
  const int *tok_pos;
  const float *talk;        // [H, H]: row h = the weights of output head h over the source heads
  const float *pb;          // [H] added to the mixed score
  const float *slopes;      // [H]
  const float *gate;        // [rows, ldg] gate logits (nullable)
  void *out;                // [rows, H * Dv] in T
  const int *seg_entry, *seg_row0, *seg_len;
  int ldg, H, G, D, Dv, block_size, max_blocks, window, vec_k, vec_v;
  float scale;
  float *scratch;           // key splits > 1: [splits][rows][H * Dv] partial sums (no gate)
  int rows, pass_per_split;
};

template <class T> struct TLd;
template <> struct TLd<bf16_t> {
  static __device__ __forceinline__ void v8(const bf16_t *p, float *o) {
    const int4 v = *(const int4 *)p;
    const unsigned u[4] = {(unsigned)v.x, (unsigned)v.y, (unsigned)v.z, (unsigned)v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) { o[2 * j] = __uint_as_float(u[j] << 16); o[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u); }
  }
  static __device__ __forceinline__ void v2(const bf16_t *p, float &x, float &y) {
    const unsigned u = *(const unsigned *)p;
    x = __uint_as_float(u << 16); y = __uint_as_float(u & 0xffff0000u);
  }
};
template <> struct TLd<float> {
  static __device__ __forceinline__ void v8(const float *p, float *o) {
    const float4 x = *(const float4 *)p, y = *(const float4 *)(p + 4);
    o[0] = x.x; o[1] = x.y; o[2] = x.z; o[3] = x.w; o[4] = y.x; o[5] = y.y; o[6] = y.z; o[7] = y.w;
  }
  static __device__ __forceinline__ void v2(const float *p, float &x, float &y) { const float2 v = *(const float2 *)p; x = v.x; y = v.y; }
};

template <class T, int NQ, int IT, int VW, int NT> __global__ void __launch_bounds__(NT) talk_sigmoid_attn_kernel(TalkArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int z = blockIdx.y;
  const int t0 = a.seg_row0[z] + blockIdx.x * NQ;
  int nq = a.seg_row0[z] + a.seg_len[z] - t0;
  if (nq <= 0) return;
  nq = nq > NQ ? NQ : nq;
  const int H = a.H, D = a.D, Dv = a.Dv, rep = H / a.G, bs = a.block_size;
  const int Dp = (D + 7) & ~7, Hp = (H + 3) & ~3;
  float *qs = lds;                          // [H][NQ][Dp]
  float *sc = qs + (size_t)H * NQ * Dp;     // [H][64][NQ]
  float *pw = sc + (size_t)H * 64 * NQ;     // [H][64][NQ]
  float *tk = pw + (size_t)H * 64 * NQ;     // [H][Hp]: tk[g][h] = talk[h][g]
  long long *base0 = (long long *)(tk + (size_t)H * Hp);  // [64]: page row of the pass's keys for key / value head 0 (-1: past the end)
  const int s = a.seg_entry[z], i0 = a.tok_pos[t0];
  for (int e = tid; e < H * NQ * Dp; e += NT) {
    const int g = e / (NQ * Dp), r = e - g * NQ * Dp, q = r / Dp, d = r - q * Dp;
    qs[e] = (q < nq && d < D) ? to_f<T>(((const T *)a.q)[((size_t)(t0 + q) * H + g) * D + d]) : 0.f;
  }
  for (int e = tid; e < H * Hp; e += NT) {
    const int g = e / Hp, h = e - g * Hp;
    tk[e] = h < H ? a.talk[(size_t)h * H + g] : 0.f;
  }
  const int *bt = a.block_tables + (size_t)s * a.max_blocks;
  int lo = a.window > 0 ? i0 - a.window + 1 : 0;
  if (lo < 0) lo = 0;
  const int hi = i0 + nq - 1, total = hi - lo + 1;
  const int DvG = (Dv + VW - 1) / VW, items = H * DvG;   // (head, group of VW values)
  int JS = 1;                                            // thread groups that share a pass's keys
  while (JS < 8 && items * JS * 2 <= NT * IT) JS <<= 1;
  int it_h[IT], it_d[IT], it_j[IT];                      // a thread's items: head, first value, key group (-1: none)
  float o[IT][NQ][VW];
#pragma unroll
  for (int u = 0; u < IT; ++u) {
    const int sidx = tid + u * NT, item = sidx % items, jp = sidx / items;
    it_h[u] = item / DvG;
    it_d[u] = (item - it_h[u] * DvG) * VW;
    it_j[u] = jp < JS ? jp : -1;
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int e = 0; e < VW; ++e) o[u][q][e] = 0.f;
  }
  const int v_lo = blockIdx.z * a.pass_per_split * 64;
  int v_hi = v_lo + a.pass_per_split * 64;
  if (v_hi > total) v_hi = total;

  for (int v0 = v_lo; v0 < v_hi; v0 += 64) {
    if (tid < 64) {
      const int key = lo + v0 + tid;
      base0[tid] = key <= hi ? (long long)bt[key / bs] * a.G * bs + key % bs : -1;
    }
    __syncthreads();  // also: q and talk are in LDS (first pass)
    // ---- A: raw scores with the distance bias
    {
      const long long b0 = base0[lane];
      const int key = lo + v0 + lane;
      for (int g = wave; g < H; g += NT / 64) {
        float acc[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) acc[q] = 0.f;
        if (b0 >= 0) {
          const T *kr = (const T *)a.k_cache + (size_t)(b0 + (long long)(g / rep) * bs) * D;
          const float *qg = qs + (size_t)g * NQ * Dp;
          if (a.vec_k) {
            for (int d = 0; d < D; d += 8) {
              float kv[8];
              TLd<T>::v8(kr + d, kv);
#pragma unroll
              for (int q = 0; q < NQ; ++q) {
                const float4 qa = *(const float4 *)(qg + q * Dp + d), qb = *(const float4 *)(qg + q * Dp + d + 4);
                float c = acc[q];
                c = fmaf(qa.x, kv[0], c); c = fmaf(qa.y, kv[1], c); c = fmaf(qa.z, kv[2], c); c = fmaf(qa.w, kv[3], c);
                c = fmaf(qb.x, kv[4], c); c = fmaf(qb.y, kv[5], c); c = fmaf(qb.z, kv[6], c); c = fmaf(qb.w, kv[7], c);
                acc[q] = c;
              }
            }
          } else {
            for (int d = 0; d < D; ++d) {
              const float kvv = to_f<T>(kr[d]);
#pragma unroll
              for (int q = 0; q < NQ; ++q) acc[q] = fmaf(qg[q * Dp + d], kvv, acc[q]);
            }
          }
          const float sl = a.slopes[g];
#pragma unroll
          for (int q = 0; q < NQ; ++q) acc[q] = acc[q] * a.scale - sl * (float)(i0 + q - key);
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) sc[((size_t)g * 64 + lane) * NQ + q] = acc[q];
      }
    }
    __syncthreads();
    // ---- B: mix the heads, visibility, sigmoid
    for (int it = tid; it < (Hp >> 2) * 64 * NQ; it += NT) {
      const int jq = it % (64 * NQ), h0 = (it / (64 * NQ)) << 2;
      const int j = jq / NQ, q = jq - j * NQ;
      float m0 = 0.f, m1 = 0.f, m2 = 0.f, m3 = 0.f;
      for (int g = 0; g < H; ++g) {
        const float sv = sc[(size_t)g * 64 * NQ + jq];
        const float4 t4 = *(const float4 *)(tk + (size_t)g * Hp + h0);
        m0 = fmaf(t4.x, sv, m0); m1 = fmaf(t4.y, sv, m1); m2 = fmaf(t4.z, sv, m2); m3 = fmaf(t4.w, sv, m3);
      }
      const int key = lo + v0 + j, iq = i0 + q;
      const bool vis = key <= hi && q < nq && key <= iq && (a.window <= 0 || iq - key < a.window);
      const float mm[4] = {m0, m1, m2, m3};
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (h0 + u < H) pw[(size_t)(h0 + u) * 64 * NQ + jq] = vis ? 1.0f / (1.0f + expf(-(mm[u] + a.pb[h0 + u]))) : 0.f;
    }
    __syncthreads();
    // ---- C: weighted value sums
    const int cnt = v_hi - v0 < 64 ? v_hi - v0 : 64;
#pragma unroll
    for (int u = 0; u < IT; ++u) {
      if (it_j[u] < 0) continue;
      const int h = it_h[u], d = it_d[u];
      const T *vb = (const T *)a.v_cache + (size_t)(h / rep) * bs * Dv + d;
      const float *ph = pw + (size_t)h * 64 * NQ;
#pragma unroll 4
      for (int j = it_j[u]; j < cnt; j += JS) {
        const T *vr = vb + (size_t)base0[j] * Dv;
        float x[VW];
        if (VW == 8) TLd<T>::v8(vr, x);
        else if (a.vec_v) TLd<T>::v2(vr, x[0], x[1]);
        else { x[0] = to_f<T>(vr[0]); x[1] = d + 1 < Dv ? to_f<T>(vr[1]) : 0.f; }
        float pj[NQ];
        if (NQ >= 4) {
#pragma unroll
          for (int q4 = 0; q4 < NQ; q4 += 4) {
            const float4 p4 = *(const float4 *)(ph + j * NQ + q4);
            pj[q4] = p4.x; pj[q4 + 1] = p4.y; pj[q4 + 2] = p4.z; pj[q4 + 3] = p4.w;
          }
        } else {
#pragma unroll
          for (int q = 0; q < NQ; ++q) pj[q] = ph[j * NQ + q];
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
          for (int e = 0; e < VW; ++e) o[u][q][e] = fmaf(pj[q], x[e], o[u][q][e]);
      }
    }
    __syncthreads();  // p and the row indices of this pass are consumed
  }
  if (JS > 1) {  // the key groups' sums meet in LDS (everything else there has been consumed), one query at a time; group 0 keeps the total
    float *red = lds;  // [NT * IT][VW]
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      __syncthreads();
#pragma unroll
      for (int u = 0; u < IT; ++u)
        if (it_j[u] > 0)
#pragma unroll
          for (int e = 0; e < VW; ++e) red[(size_t)(tid + u * NT) * VW + e] = o[u][q][e];
      __syncthreads();
#pragma unroll
      for (int u = 0; u < IT; ++u)
        if (it_j[u] == 0)
          for (int p = 1; p < JS; ++p)
#pragma unroll
            for (int e = 0; e < VW; ++e) o[u][q][e] += red[(size_t)(tid + u * NT + p * items) * VW + e];
    }
  }
#pragma unroll
  for (int u = 0; u < IT; ++u) {
    if (it_j[u] != 0) continue;
    const int h = it_h[u], d = it_d[u];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if (q >= nq) break;
      if (a.scratch) {
        float *out = a.scratch + ((size_t)blockIdx.z * a.rows + (t0 + q)) * H * Dv + (size_t)h * Dv + d;
#pragma unroll
        for (int e = 0; e < VW; ++e)
          if (d + e < Dv) out[e] = o[u][q][e];
      } else {
        const float gl = a.gate ? 1.0f / (1.0f + expf(-a.gate[(size_t)(t0 + q) * a.ldg + h])) : 1.0f;
        T *out = (T *)a.out + ((size_t)(t0 + q) * H + h) * Dv + d;
#pragma unroll
        for (int e = 0; e < VW; ++e)
          if (d + e < Dv) out[e] = from_f<T>(o[u][q][e] * gl);
      }
    }
  }
}

// the key splits' partial sums, added in split order; gate; rounding
template <class T> __global__ void __launch_bounds__(256) talk_reduce_kernel(const float *__restrict__ scratch, int splits, int rows, int HDv, int Dv, const float *__restrict__ gate,
                                                                             int ldg, T *__restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, n = (size_t)rows * HDv;
  if (i >= n) return;
  const int t = (int)(i / HDv), c = (int)(i - (size_t)t * HDv);
  float acc = 0.f;
  for (int k = 0; k < splits; ++k) acc += scratch[(size_t)k * n + i];
  const float gl = gate ? 1.0f / (1.0f + expf(-gate[(size_t)t * ldg + c / Dv])) : 1.0f;
  out[i] = from_f<T>(acc * gl);
}

template <class T, int NQ, int IT, int VW, int NT> static int launch_talk(const TalkArgs &a, dim3 grid, size_t lds, hipStream_t st) {
  if (lds > 65536) {
    static thread_local size_t granted = 0;  // per instantiation
    if (lds > granted) {
      if (hipFuncSetAttribute((const void *)talk_sigmoid_attn_kernel<T, NQ, IT, VW, NT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return tfail("mrs_hyb_paged_talk_sigmoid_attn: the heads' queries and scores do not fit into LDS");
      }
      granted = lds;
    }
  }
  hipLaunchKernelGGL((talk_sigmoid_attn_kernel<T, NQ, IT, VW, NT>), grid, dim3(NT), lds, st, a);
  return 0;
}

}  // namespace hyb
}  // namespace mrs

using namespace mrs::hyb;

extern "C" const char *mrs_hyb_talk_last_error() { return g_terr; }

/* Rows are addressed through the batch's segment table (seg_entry / seg_row0 / seg_len [segments], at most seg_rows rows each: 1 when every entry brings one decoded token).
 * gate [rows, ldg]: logits whose sigmoid multiplies the head outputs (nullable).  talk [H, H], pb [H], slopes [H] f32 on the device.  scratch (nullable): f32
 * [scratch_splits][rows][H * Dv]; with it, a step of few workgroups deals every tile's keys to up to scratch_splits workgroups. */
extern "C" int mrs_hyb_paged_talk_sigmoid_attn(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_pos, const float *talk,
                                               const float *pb, const float *slopes, const float *gate, int ldg, void *out, int rows, int H, int G, int D, int Dv, int block_size,
                                               int max_blocks, int window, float scale, int dtype, const int *seg_entry, const int *seg_row0, const int *seg_len, int segments,
                                               int seg_rows, float *scratch, int scratch_splits, void *stream) {
  if (rows <= 0 || segments <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0) return tfail("mrs_hyb_paged_talk_sigmoid_attn: head sizes (heads % kv_heads == 0)");
  if (!seg_entry || !seg_row0 || !seg_len || seg_rows <= 0 || segments > 65535) return tfail("mrs_hyb_paged_talk_sigmoid_attn: the segment table is missing or too long");
  if (dtype != 1 && dtype != 2) return tfail("mrs_hyb_paged_talk_sigmoid_attn: dtype");
  const int esz = dtype == 1 ? 2 : 4;
  const int vw = (Dv % 8 == 0 && ((uintptr_t)v_cache % 16) == 0) ? 8 : 2;
  TalkArgs a{q, k_cache, v_cache, block_tables, tok_pos, talk, pb, slopes, gate, out, seg_entry, seg_row0, seg_len, ldg, H, G, D, Dv, block_size, max_blocks, window,
             (D % 8 == 0 && ((uintptr_t)k_cache % 16) == 0) ? 1 : 0, (Dv % 2 == 0 && ((uintptr_t)v_cache % (2 * esz)) == 0) ? 1 : 0, scale, nullptr, rows, 1 << 24};
  const int items = H * ((Dv + vw - 1) / vw);
  const int nt = (vw == 8 && H >= 8) ? 512 : 256;   // eight waves when there are heads for them: twice the waves per byte of LDS
  int it = (items + nt - 1) / nt;
  it = it <= 1 ? 1 : (it <= 2 ? 2 : (it <= 4 ? 4 : 8));
  if (items > 8 * nt) return tfail("mrs_hyb_paged_talk_sigmoid_attn: heads * value size too large for one workgroup");
  static const int lds_kb = getenv("MRS_TALK_LDS_KB") ? atoi(getenv("MRS_TALK_LDS_KB")) : 79;   // tile choice: LDS per workgroup (79: two workgroups per compute unit)
  const int Dp = (D + 7) & ~7, Hp = (H + 3) & ~3, cap = vw == 8 ? 8 : 16;   // accumulator registers: NQ * IT * VW <= 64 (32 for pairs)
  auto lds_of = [&](int nq) {
    const size_t work = ((size_t)H * nq * Dp + 2 * (size_t)H * 64 * nq + (size_t)H * Hp) * 4 + 64 * 8, red = (size_t)nt * it * vw * 4;
    return work > red ? work : red;
  };
  int nq = 1;
  if (seg_rows > 1)  // some entry brings a portion: the widest tile that keeps the accumulators in registers and leaves room for two workgroups' LDS per compute unit
    for (int c = 8; c > 1; c >>= 1)
      if (c * it <= cap && c <= seg_rows && lds_of(c) <= (size_t)lds_kb * 1024) { nq = c; break; }
  if (nq * it > cap) return tfail("mrs_hyb_paged_talk_sigmoid_attn: heads * value size too large for one workgroup");
  if (vw == 2 && nq == 8) nq = 4;   // pairs: tiles of 1, 2 and 4 queries
  const size_t lds = lds_of(nq);
  if (lds > 160 * 1024) return tfail("mrs_hyb_paged_talk_sigmoid_attn: the heads' queries and scores do not fit into LDS");
  const int tiles = (seg_rows + nq - 1) / nq;
  int splits = 1;
  if (scratch && scratch_splits > 1 && (long long)tiles * segments < 256) {
    const long long ctx = (long long)max_blocks * block_size, span = window > 0 && window + nq - 1 < ctx ? window + nq - 1 : ctx;
    const int passes = (int)((span + 63) / 64), want = (int)((512 + (long long)tiles * segments - 1) / ((long long)tiles * segments));
    splits = passes < want ? passes : want;
    if (splits > scratch_splits) splits = scratch_splits;
    if (splits > 1) {
      a.pass_per_split = (passes + splits - 1) / splits;
      splits = (passes + a.pass_per_split - 1) / a.pass_per_split;
    }
    if (splits > 1) a.scratch = scratch;
  }
  dim3 grid(tiles, segments, splits);
  hipStream_t st = (hipStream_t)stream;
  int rc = 1;
#define MRS_TALK_L(T, NQ_, IT_, VW_) do { if (VW_ == 8 && nt == 512) rc = launch_talk<T, NQ_, IT_, VW_, (VW_ == 8 ? 512 : 256)>(a, grid, lds, st); else rc = launch_talk<T, NQ_, IT_, VW_, 256>(a, grid, lds, st); } while (0)
#define MRS_TALK(T) do { \
    if (vw == 8) { \
      if (nq == 8) MRS_TALK_L(T, 8, 1, 8); \
      else if (nq == 4) { if (it == 1) MRS_TALK_L(T, 4, 1, 8); else MRS_TALK_L(T, 4, 2, 8); } \
      else if (nq == 2) { if (it == 1) MRS_TALK_L(T, 2, 1, 8); else if (it == 2) MRS_TALK_L(T, 2, 2, 8); else MRS_TALK_L(T, 2, 4, 8); } \
      else { if (it == 1) MRS_TALK_L(T, 1, 1, 8); else if (it == 2) MRS_TALK_L(T, 1, 2, 8); else if (it == 4) MRS_TALK_L(T, 1, 4, 8); else MRS_TALK_L(T, 1, 8, 8); } \
    } else { \
      if (nq == 4) { if (it == 1) MRS_TALK_L(T, 4, 1, 2); else if (it == 2) MRS_TALK_L(T, 4, 2, 2); else MRS_TALK_L(T, 4, 4, 2); } \
      else if (nq == 2) { if (it == 1) MRS_TALK_L(T, 2, 1, 2); else if (it == 2) MRS_TALK_L(T, 2, 2, 2); else if (it == 4) MRS_TALK_L(T, 2, 4, 2); else MRS_TALK_L(T, 2, 8, 2); } \
      else { if (it == 1) MRS_TALK_L(T, 1, 1, 2); else if (it == 2) MRS_TALK_L(T, 1, 2, 2); else if (it == 4) MRS_TALK_L(T, 1, 4, 2); else MRS_TALK_L(T, 1, 8, 2); } \
    } } while (0)
  if (dtype == 1) MRS_TALK(mrs::bf16_t); else MRS_TALK(float);
#undef MRS_TALK
#undef MRS_TALK_L
  if (rc) return rc;
  if (splits > 1) {
    const size_t n = (size_t)rows * H * Dv;
    if (dtype == 1) hipLaunchKernelGGL(talk_reduce_kernel<mrs::bf16_t>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, scratch, splits, rows, H * Dv, Dv, gate, ldg, (mrs::bf16_t *)out);
    else hipLaunchKernelGGL(talk_reduce_kernel<float>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, scratch, splits, rows, H * Dv, Dv, gate, ldg, (float *)out);
  }
  if (hipGetLastError() != hipSuccess) return tfail("mrs_hyb_paged_talk_sigmoid_attn: launch failed");
  return 0;
}

// hyb_attn_talk.hip -- paged sigmoid attention with a distance bias and mixed head scores, on ragged batches (same batch description as hyb_kernels.hip).
//
// Query i of head g scores key j as   s_g = scale (q_g . k_j) - slope_g (i - j);   the heads' scores of one (i, j) pair are mixed,   s'_h = sum_g talk[h, g] s_g;   a visible
// key (0 <= i - j < window; window <= 0: every j <= i) weighs   p_h = sigmoid(s'_h + pb_h)   -- no normalisation over the keys, so there is no running maximum or sum and
// the keys can be consumed in any order --   o_h = sum_j p_h v_j,   and the head's output is multiplied by sigmoid(gate logit of (row, h)).  Scores, weights and sums are f32.
//
// Because every output head needs the scores of ALL heads, one workgroup owns NQ consecutive rows of one entry (a tile of a segment; NQ = 1 for decoded tokens) for every
// head.  Keys go by in passes of 64:
//   A  wave w scores heads w, w + 4, ..: a lane = a key, its row is read in 16-byte loads and multiplied with the NQ query vectors in LDS      -> s [H][64][NQ] (LDS)
//   B  a thread = (4 output heads, key, query): sum over g with talk^T rows as float4 broadcasts, visibility, sigmoid                            -> p [H][64][NQ] (LDS)
//   C  a thread = IT x (head, value pair): the value pair of key j is read once and added into the NQ accumulators (registers)
// Grouped heads: query head h reads key / value head h / (H / G).
#include "common.cuh"
#include <float.h>

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

template <class T, int NQ, int IT> __global__ void __launch_bounds__(256) talk_sigmoid_attn_kernel(TalkArgs a) {
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
  for (int e = tid; e < H * NQ * Dp; e += 256) {
    const int g = e / (NQ * Dp), r = e - g * NQ * Dp, q = r / Dp, d = r - q * Dp;
    qs[e] = (q < nq && d < D) ? to_f<T>(((const T *)a.q)[((size_t)(t0 + q) * H + g) * D + d]) : 0.f;
  }
  for (int e = tid; e < H * Hp; e += 256) {
    const int g = e / Hp, h = e - g * Hp;
    tk[e] = h < H ? a.talk[(size_t)h * H + g] : 0.f;
  }
  const int *bt = a.block_tables + (size_t)s * a.max_blocks;
  int lo = a.window > 0 ? i0 - a.window + 1 : 0;
  if (lo < 0) lo = 0;
  const int hi = i0 + nq - 1, total = hi - lo + 1;
  const int Dvh = (Dv + 1) >> 1, items = H * Dvh;
  float o[IT][NQ][2];
#pragma unroll
  for (int u = 0; u < IT; ++u)
#pragma unroll
    for (int q = 0; q < NQ; ++q) o[u][q][0] = o[u][q][1] = 0.f;

  for (int v0 = 0; v0 < total; v0 += 64) {
    if (tid < 64) {
      const int key = lo + v0 + tid;
      base0[tid] = key <= hi ? (long long)bt[key / bs] * a.G * bs + key % bs : -1;
    }
    __syncthreads();  // also: q and talk are in LDS (first pass); the previous pass has consumed p and the row indices
    // ---- A: raw scores with the distance bias
    {
      const long long b0 = base0[lane];
      const int key = lo + v0 + lane;
      for (int g = wave; g < H; g += 4) {
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
    for (int it = tid; it < (Hp >> 2) * 64 * NQ; it += 256) {
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
    const int cnt = total - v0 < 64 ? total - v0 : 64;
#pragma unroll
    for (int u = 0; u < IT; ++u) {
      const int item = tid + u * 256;
      if (item < items) {
        const int h = item / Dvh, d = (item - h * Dvh) << 1;
        const T *vb = (const T *)a.v_cache + (size_t)(h / rep) * bs * Dv + d;
        const float *ph = pw + (size_t)h * 64 * NQ;
        const bool two = d + 1 < Dv;
#pragma unroll 2
        for (int j = 0; j < cnt; ++j) {
          const T *vr = vb + (size_t)base0[j] * Dv;
          float x, y = 0.f;
          if (a.vec_v) TLd<T>::v2(vr, x, y);
          else { x = to_f<T>(vr[0]); if (two) y = to_f<T>(vr[1]); }
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
          for (int q = 0; q < NQ; ++q) {
            o[u][q][0] = fmaf(pj[q], x, o[u][q][0]);
            o[u][q][1] = fmaf(pj[q], y, o[u][q][1]);
          }
        }
      }
    }
    __syncthreads();  // p and the row indices of this pass are consumed
  }
#pragma unroll
  for (int u = 0; u < IT; ++u) {
    const int item = tid + u * 256;
    if (item >= items) continue;
    const int h = item / Dvh, d = (item - h * Dvh) << 1;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if (q >= nq) break;
      const float gl = a.gate ? 1.0f / (1.0f + expf(-a.gate[(size_t)(t0 + q) * a.ldg + h])) : 1.0f;
      T *out = (T *)a.out + ((size_t)(t0 + q) * H + h) * Dv + d;
      out[0] = from_f<T>(o[u][q][0] * gl);
      if (d + 1 < Dv) out[1] = from_f<T>(o[u][q][1] * gl);
    }
  }
}

template <class T, int NQ, int IT> static int launch_talk(const TalkArgs &a, dim3 grid, size_t lds, hipStream_t st) {
  if (lds > 65536) {
    static thread_local size_t granted = 0;  // per instantiation
    if (lds > granted) {
      if (hipFuncSetAttribute((const void *)talk_sigmoid_attn_kernel<T, NQ, IT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return tfail("mrs_hyb_paged_talk_sigmoid_attn: the heads' queries and scores do not fit into LDS");
      }
      granted = lds;
    }
  }
  hipLaunchKernelGGL((talk_sigmoid_attn_kernel<T, NQ, IT>), grid, dim3(256), lds, st, a);
  return 0;
}

}  // namespace hyb
}  // namespace mrs

using namespace mrs::hyb;

extern "C" const char *mrs_hyb_talk_last_error() { return g_terr; }

/* Rows are addressed through the batch's segment table (seg_entry / seg_row0 / seg_len [segments], at most seg_rows rows each: 1 when every entry brings one decoded token).  gate [rows, ldg]: logits whose sigmoid
 * multiplies the head outputs (nullable).  talk [H, H], pb [H], slopes [H] f32 on the device. */
extern "C" int mrs_hyb_paged_talk_sigmoid_attn(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_pos, const float *talk,
                                               const float *pb, const float *slopes, const float *gate, int ldg, void *out, int rows, int H, int G, int D, int Dv, int block_size,
                                               int max_blocks, int window, float scale, int dtype, const int *seg_entry, const int *seg_row0, const int *seg_len, int segments,
                                               int seg_rows, void *stream) {
  if (rows <= 0 || segments <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0) return tfail("mrs_hyb_paged_talk_sigmoid_attn: head sizes (heads % kv_heads == 0)");
  if (!seg_entry || !seg_row0 || !seg_len || seg_rows <= 0 || segments > 65535) return tfail("mrs_hyb_paged_talk_sigmoid_attn: the segment table is missing or too long");
  if (dtype != 1 && dtype != 2) return tfail("mrs_hyb_paged_talk_sigmoid_attn: dtype");
  const int esz = dtype == 1 ? 2 : 4;
  TalkArgs a{q, k_cache, v_cache, block_tables, tok_pos, talk, pb, slopes, gate, out, seg_entry, seg_row0, seg_len, ldg, H, G, D, Dv, block_size, max_blocks, window,
             (D % 8 == 0 && ((uintptr_t)k_cache % 16) == 0) ? 1 : 0, (Dv % 2 == 0 && ((uintptr_t)v_cache % (2 * esz)) == 0) ? 1 : 0, scale};
  const int items = H * ((Dv + 1) / 2);
  int it = (items + 255) / 256;
  it = it <= 1 ? 1 : (it <= 2 ? 2 : (it <= 4 ? 4 : 8));
  if (items > 8 * 256) return tfail("mrs_hyb_paged_talk_sigmoid_attn: heads * value size above 4096");
  const int Dp = (D + 7) & ~7, Hp = (H + 3) & ~3;
  auto lds_of = [&](int nq) { return ((size_t)H * nq * Dp + 2 * (size_t)H * 64 * nq + (size_t)H * Hp) * 4 + 64 * 8; };
  int nq = 1;
  if (seg_rows > 1)  // some entry brings a portion: the widest tile that keeps the accumulators in registers and the scores in 64 KB of LDS
    for (int c = 8; c > 1; c >>= 1)
      if (c * it <= 16 && c <= seg_rows && lds_of(c) <= 65536) { nq = c; break; }
  const size_t lds = lds_of(nq);
  if (lds > 160 * 1024) return tfail("mrs_hyb_paged_talk_sigmoid_attn: the heads' queries and scores do not fit into LDS");
  dim3 grid((seg_rows + nq - 1) / nq, segments);
  hipStream_t st = (hipStream_t)stream;
  int rc = 1;
#define MRS_TALK_IT(T, NQ_) (it == 1 ? launch_talk<T, NQ_, 1>(a, grid, lds, st) : it == 2 ? launch_talk<T, NQ_, 2>(a, grid, lds, st) : tfail("mrs_hyb_paged_talk_sigmoid_attn: tile"))
#define MRS_TALK(T) do { \
    if (nq == 8) rc = MRS_TALK_IT(T, 8); \
    else if (nq == 4) rc = it <= 2 ? MRS_TALK_IT(T, 4) : launch_talk<T, 4, 4>(a, grid, lds, st); \
    else if (nq == 2) rc = it <= 2 ? MRS_TALK_IT(T, 2) : (it == 4 ? launch_talk<T, 2, 4>(a, grid, lds, st) : launch_talk<T, 2, 8>(a, grid, lds, st)); \
    else rc = it <= 2 ? MRS_TALK_IT(T, 1) : (it == 4 ? launch_talk<T, 1, 4>(a, grid, lds, st) : launch_talk<T, 1, 8>(a, grid, lds, st)); } while (0)
  if (dtype == 1) MRS_TALK(mrs::bf16_t); else MRS_TALK(float);
#undef MRS_TALK
#undef MRS_TALK_IT
  if (rc) return rc;
  if (hipGetLastError() != hipSuccess) return tfail("mrs_hyb_paged_talk_sigmoid_attn: launch failed");
  return 0;
}

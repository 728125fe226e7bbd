// Softmax attention whose heads' scores are mixed before the softmax, over a paged cache, with a
// sliding window that keeps a sequence's first tokens.
//
//   raw_g[i, j] = scale * q_g[i] . k_kv(g)[j]              (kv(g) = g / (H / KV))
//   s_h[i, j]   = sum_g mix[h, g] * raw_g[i, j]            (mix null: s_h = raw_h)
//   j visible from i:  j <= i  and  (window <= 0  or  i - j < window  or  j < keep_first)
//   out_h[i]    = sum_j softmax_j(s_h[i, :]) v_kv(h)[j]
//
// Every head of a query needs every other head's score of the same key, so a workgroup owns all H
// heads of a work item: TQ consecutive queries of one row (TQ = 1: a single token).  It walks the
// pages the item can see (the kept first tokens' pages, then the window's) in chunks of up to 64
// key slots, three phases a chunk, LDS between them:
//   1. raw scores: a lane owns a key slot, a wave a (kv head, four queries): the key row comes from the
//      page 16 bytes at a time, the queries from LDS (every lane the same address);
//   2. mixing, mask and the running softmax: a lane owns a key slot, a wave a (query, head) row;
//   3. weights times values: a thread owns output coordinates (head, d) for all TQ queries and reads a
//      page's values of its coordinate in one piece (pages hold values transposed, [D, block_size]).
// Scores, weights, maxima and sums are fp32 in both precisions; outputs accumulate in fp32.
// Masked slots are multiplied by a weight of zero, not skipped: the pools only hold finite numbers.
#include "common.h"

#define AM_THREADS 256
#define AM_WAVES 4
#define AM_KC 64     // key slots of a chunk: one per lane
#define AM_GMAX 8    // query heads of a kv head that phase 1 takes in one walk over the key's row
#define AM_QSUB 4    // queries of a phase-1 unit

template <typename T> struct Piece8;
template <> struct Piece8<float> {
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
};
template <> struct Piece8<bf16> {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ void load(const bf16* p, float* v) {
    const bf16x8 r = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)r[i];
  }
};

struct MixArgs {
  const void* q;
  const void* k_pages;
  const void* v_pages;
  const int* items;
  const int* positions;
  const int* tok_row;
  const int* tables;
  int table_width;
  const float* mix;
  void* out;
  int H, KV, D, Dout, bs;  // Dout <= D: the coordinates of a head that the output keeps (the rest is padding)
  float scale;
  int window, keep_first;
};

// accumulators of phase 3 per thread: RMAX (head, d) coordinates by TQ queries
template <int TQ> struct MixShape { static constexpr int RMAX = TQ >= 16 ? 4 : (TQ >= 8 ? 8 : (TQ >= 4 ? 16 : 32)); };

template <typename T, int TQ>
__global__ __launch_bounds__(AM_THREADS) void attn_headmix_kernel(MixArgs a) {
  constexpr int RMAX = MixShape<TQ>::RMAX;
  constexpr int QS = (TQ + AM_QSUB - 1) / AM_QSUB;  // query sub-tiles of phase 1
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int H = a.H, KV = a.KV, D = a.D, bs = a.bs, group = H / KV;
  const int HD = H * D;
  // LDS: queries (T), raw scores and weights (fp32 [H][TQ][KC] each), the mixing matrix, row statistics, pages
  float* sraw = reinterpret_cast<float*>(lds_raw);
  float* pw = sraw + (size_t)H * TQ * AM_KC;
  float* mixs = pw + (size_t)H * TQ * AM_KC;
  float* row_m = mixs + H * H;
  float* row_l = row_m + TQ * H;
  float* row_a = row_l + TQ * H;
  int* pages = reinterpret_cast<int*>(row_a + TQ * H);  // AM_KC entries: the physical page of every slot's page
  T* qs = reinterpret_cast<T*>((reinterpret_cast<uintptr_t>(pages + AM_KC) + 15) & ~(uintptr_t)15);  // [TQ][H][D]

  const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  int first, count, row, p0;
  if (TQ == 1) {
    first = a.items[blockIdx.x];
    count = 1;
    row = a.tok_row ? a.tok_row[first] : first;
    p0 = a.positions[first];
  } else {
    const int* it = a.items + 4 * blockIdx.x;
    first = it[0]; count = it[1]; row = it[2]; p0 = it[3];
  }
  const int* table = a.tables + (size_t)row * a.table_width;
  const T* q = reinterpret_cast<const T*>(a.q);
  const T* kp = reinterpret_cast<const T*>(a.k_pages);
  const T* vp = reinterpret_cast<const T*>(a.v_pages);

  // the pages this item can see: those of the kept first tokens that lie before the window's, then the window's
  const int hi = p0 + count - 1;
  const int lo = a.window > 0 ? max(0, p0 - a.window + 1) : 0;
  const int pb0 = lo / bs, pb1 = hi / bs;
  const int kept = min(a.keep_first, hi + 1);
  const int pa_end = min((kept + bs - 1) / bs, pb0);
  const int NP = pa_end + (pb1 - pb0 + 1);
  const int ppc = AM_KC / bs > 0 ? AM_KC / bs : 1;  // pages of a chunk (block sizes above 64 are refused)
  const int kc = ppc * bs;                          // its key slots (<= 64)
  const int chunks = (NP + ppc - 1) / ppc;

  for (int i = tid; i < TQ * HD; i += AM_THREADS) {
    const int qi = i / HD;
    qs[i] = qi < count ? q[(size_t)(first + qi) * HD + (i - qi * HD)] : from_f32<T>(0.f);
  }
  for (int i = tid; i < H * H; i += AM_THREADS) mixs[i] = a.mix ? a.mix[i] : ((i / H) == (i % H) ? 1.f : 0.f);
  for (int i = tid; i < TQ * H; i += AM_THREADS) { row_m[i] = -INFINITY; row_l[i] = 0.f; }

  float acc[RMAX][TQ];
#pragma unroll
  for (int r = 0; r < RMAX; ++r)
#pragma unroll
    for (int qi = 0; qi < TQ; ++qi) acc[r][qi] = 0.f;

  for (int ch = 0; ch < chunks; ++ch) {
    __syncthreads();  // the chunk before has been read (and, the first time, the queries are in place)
    // this lane's key slot: which page, which position
    const int u = ch * ppc + lane / bs, off = lane % bs;
    const bool slot_valid = lane < kc && u < NP;
    const int lp = u < pa_end ? u : pb0 + (u - pa_end);
    const int jpos = lp * bs + off;
    if (tid < AM_KC) pages[tid] = slot_valid ? table[lp] : 0;
    __syncthreads();
    // ---- phase 1: raw scores ------------------------------------------------------------
    for (int unit = wave; unit < KV * QS; unit += AM_WAVES) {
      const int c = unit / QS, q0 = (unit % QS) * AM_QSUB;
      const T* krow = kp + (((size_t)pages[lane] * KV + c) * bs + off) * D;
      for (int g0 = 0; g0 < group; g0 += AM_GMAX) {
        float s[AM_GMAX][AM_QSUB];
#pragma unroll
        for (int g = 0; g < AM_GMAX; ++g)
#pragma unroll
          for (int qq = 0; qq < AM_QSUB; ++qq) s[g][qq] = 0.f;
        if (slot_valid) {
          for (int d = 0; d < D; d += 8) {
            float kv[8];
            if (d + 8 <= D) {
              Piece8<T>::load(krow + d, kv);
            } else {
#pragma unroll
              for (int i = 0; i < 8; ++i) kv[i] = d + i < D ? to_f32(krow[d + i]) : 0.f;
            }
#pragma unroll
            for (int g = 0; g < AM_GMAX; ++g) {
              if (g0 + g >= group) break;
              const int h = c * group + g0 + g;
#pragma unroll
              for (int qq = 0; qq < AM_QSUB; ++qq) {
                if (q0 + qq >= TQ) break;
                const T* qv = qs + ((size_t)(q0 + qq) * H + h) * D + d;
                float qf[8];
                if (d + 8 <= D) {
                  Piece8<T>::load(qv, qf);
                } else {
#pragma unroll
                  for (int i = 0; i < 8; ++i) qf[i] = d + i < D ? to_f32(qv[i]) : 0.f;
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) s[g][qq] = fmaf(qf[i], kv[i], s[g][qq]);
              }
            }
          }
        }
#pragma unroll
        for (int g = 0; g < AM_GMAX; ++g) {
          if (g0 + g >= group) break;
          const int h = c * group + g0 + g;
#pragma unroll
          for (int qq = 0; qq < AM_QSUB; ++qq) {
            if (q0 + qq >= TQ) break;
            sraw[((size_t)h * TQ + q0 + qq) * AM_KC + lane] = s[g][qq] * a.scale;
          }
        }
      }
    }
    __syncthreads();
    // ---- phase 2: mixing, mask, running softmax -------------------------------------------
    for (int r = wave; r < TQ * H; r += AM_WAVES) {
      const int qi = r / H, h = r % H;
      float sv = 0.f;
      for (int g = 0; g < H; ++g) sv = fmaf(mixs[h * H + g], sraw[((size_t)g * TQ + qi) * AM_KC + lane], sv);
      const int ipos = p0 + qi;
      const bool seen = slot_valid && qi < count && jpos <= ipos &&
                        (a.window <= 0 || ipos - jpos < a.window || jpos < a.keep_first);
      sv = seen ? sv : -INFINITY;
      const float m_old = row_m[r];
      const float m_new = fmaxf(m_old, wave_max(sv));
      float p = 0.f, alpha = 1.f;
      if (m_new > -INFINITY) {
        p = seen ? expf(sv - m_new) : 0.f;
        alpha = m_old > -INFINITY ? expf(m_old - m_new) : 0.f;
      }
      const float sum = wave_sum(p);
      pw[((size_t)h * TQ + qi) * AM_KC + lane] = p;
      if (lane == 0) {
        row_m[r] = m_new;
        row_l[r] = row_l[r] * alpha + sum;
        row_a[r] = alpha;
      }
    }
    __syncthreads();
    // ---- phase 3: weights times values --------------------------------------------------------
    const int np_here = min(ppc, NP - ch * ppc);
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      const int e = tid + r * AM_THREADS;
      if (e >= HD) break;
      const int h = e / D, d = e - h * D, c = h / group;
#pragma unroll
      for (int qi = 0; qi < TQ; ++qi) acc[r][qi] *= row_a[qi * H + h];
      for (int pg = 0; pg < np_here; ++pg) {
        const T* vrow = vp + (((size_t)pages[pg * bs] * KV + c) * D + d) * bs;
        const float* prow = pw + (size_t)h * TQ * AM_KC + pg * bs;
        for (int o = 0; o < bs; ++o) {
          const float v = to_f32(vrow[o]);
#pragma unroll
          for (int qi = 0; qi < TQ; ++qi) acc[r][qi] = fmaf(prow[qi * AM_KC + o], v, acc[r][qi]);
        }
      }
    }
  }
  __syncthreads();
  T* out = reinterpret_cast<T*>(a.out);
#pragma unroll
  for (int r = 0; r < RMAX; ++r) {
    const int e = tid + r * AM_THREADS;
    if (e >= HD) break;
    const int h = e / D, d = e - h * D;
    if (d >= a.Dout) continue;
#pragma unroll
    for (int qi = 0; qi < TQ; ++qi) {
      if (qi >= count) break;
      const float l = row_l[qi * H + h];
      out[((size_t)(first + qi) * H + h) * a.Dout + d] = from_f32<T>(l > 0.f ? acc[r][qi] / l : 0.f);
    }
  }
}

static size_t headmix_lds_bytes(int H, int D, int tq, int elt) {
  size_t floats = 2 * (size_t)H * tq * AM_KC + (size_t)H * H + 3 * (size_t)tq * H + AM_KC;
  return floats * 4 + 16 + (size_t)tq * H * D * elt;  // 16: the queries start on 16 bytes
}

// The largest tile of queries (16, 8, 4, 2, 1) whose accumulators and LDS fit; 0: none (too many heads).
extern "C" int as_attn_headmix_tile(int H, int D, int dtype) {
  const int elt = dtype == DT_F32 ? 4 : 2;
  const int tiles[5] = {16, 8, 4, 2, 1};
  const int rmax[5] = {4, 8, 16, 32, 32};
  for (int i = 0; i < 5; ++i) {
    if ((H * D + AM_THREADS - 1) / AM_THREADS > rmax[i]) continue;
    if (headmix_lds_bytes(H, D, tiles[i], elt) > (size_t)(96 << 10)) continue;
    return tiles[i];
  }
  return 0;
}

template <typename T, int TQ>
static int launch_headmix(const MixArgs& a, int num_items, size_t lds, hipStream_t stream) {
  static bool raised = false;  // a workgroup may ask for more than 64 KB of LDS once the kernel says so
  if (lds > (size_t)(64 << 10) && !raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_headmix_kernel<T, TQ>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 96 << 10) != hipSuccess)
      return AS_LAUNCH_FAILED;
    raised = true;
  }
  attn_headmix_kernel<T, TQ><<<num_items, AM_THREADS, lds, stream>>>(a);
  return launch_status();
}

// items: tile == 1: [num_items] flat tokens (their positions in `positions`, their rows in `tok_row`, or
// token t is row t); else [num_items, 4] = (first flat token, count <= tile, row, first position).
extern "C" int as_attn_headmix(const void* q, const void* k_pages, const void* v_pages, int dtype, const int* items,
                               int num_items, int tile, const int* positions, const int* tok_row,
                               const int* tables, int table_width, const float* mix, void* out, int H, int KV,
                               int D, int Dout, int bs, float scale, int window, int keep_first,
                               hipStream_t stream) {
  if (num_items <= 0) return AS_OK;
  if (H <= 0 || KV <= 0 || H % KV || D <= 0 || bs <= 0 || bs > AM_KC || table_width <= 0 || window < 0 ||
      keep_first < 0 || Dout <= 0 || Dout > D)
    return AS_BAD_SHAPE;
  const int elt = dtype == DT_F32 ? 4 : 2;
  if (D % (16 / elt)) return AS_BAD_SHAPE;  // rows of keys and queries are read 16 bytes at a time
  const int most = as_attn_headmix_tile(H, D, dtype);
  if (most <= 0 || tile > most || tile <= 0) return AS_BAD_SHAPE;
  if (tile == 1 && !positions) return AS_BAD_SHAPE;
  MixArgs a{q, k_pages, v_pages, items, positions, tok_row, tables, table_width, mix, out, H, KV, D, Dout, bs, scale,
            window, keep_first};
  const size_t lds = headmix_lds_bytes(H, D, tile, elt);
#define GO(T)                                                              \
  switch (tile) {                                                          \
    case 1: return launch_headmix<T, 1>(a, num_items, lds, stream);        \
    case 2: return launch_headmix<T, 2>(a, num_items, lds, stream);        \
    case 4: return launch_headmix<T, 4>(a, num_items, lds, stream);        \
    case 8: return launch_headmix<T, 8>(a, num_items, lds, stream);        \
    case 16: return launch_headmix<T, 16>(a, num_items, lds, stream);      \
    default: return AS_BAD_SHAPE;                                          \
  }
  if (dtype == DT_F32) { GO(float) }
  if (dtype == DT_BF16) { GO(bf16) }
#undef GO
  return AS_BAD_DTYPE;
}

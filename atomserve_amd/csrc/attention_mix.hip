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
  int single;  // items are single tokens [N], not (first, count, row, first position) [N, 4]
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
  int item_first, item_count, row, item_p0;
  if (a.single) {
    item_first = a.items[blockIdx.x];
    item_count = 1;
    row = a.tok_row ? a.tok_row[item_first] : item_first;
    item_p0 = a.positions[item_first];
  } else {
    const int* it = a.items + 4 * blockIdx.x;
    item_first = it[0]; item_count = it[1]; row = it[2]; item_p0 = it[3];
  }
  const int* table = a.tables + (size_t)row * a.table_width;
  const T* q = reinterpret_cast<const T*>(a.q);
  const T* kp = reinterpret_cast<const T*>(a.k_pages);
  const T* vp = reinterpret_cast<const T*>(a.v_pages);
  T* out = reinterpret_cast<T*>(a.out);

  // an item of more queries than TQ is taken TQ at a time
  for (int qb = 0; qb < item_count; qb += TQ) {
  const int first = item_first + qb, count = min(TQ, item_count - qb), p0 = item_p0 + qb;
  if (qb) __syncthreads();  // the queries before have been written out of LDS' statistics
  // the pages these queries can see: those of the kept first tokens that lie before the window's, then the window's
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
  }  // the next TQ queries of the item
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
  if (most <= 0 || tile <= 0 || tile > 16) return AS_BAD_SHAPE;
  if (tile == 1 && !positions) return AS_BAD_SHAPE;
  MixArgs a{q, k_pages, v_pages, items, positions, tok_row, tables, table_width, mix, out, H, KV, D, Dout, bs, scale,
            window, keep_first, tile == 1};
  int tq = 1;  // queries a workgroup takes at once: the largest power of two within the items' and what fits
  while (2 * tq <= tile && 2 * tq <= most) tq *= 2;
  tile = tq;
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

// ---- the same on the matrix cores (bf16) ---------------------------------------------------------------
// Heads of D % 32 == 0 coordinates, H / KV a power of two up to 16, pages of 8, 16, 32 or 64 tokens.  The 16 rows of
// a matrix tile are (query, head of one kv head's group): TQ = 16 / group consecutive queries of a row, or one
// token alone (then only `group` rows stand for something).  Per chunk of 64 key slots:
//   1. scores: per kv head one product [16 rows x D] [D x 16 keys] a wave (a wave owns 16 of the chunk's keys), the keys
//      straight from the page as the B operand, the queries from LDS; scaled fp32 scores go to LDS per head;
//   2. mixing, mask and running softmax on the vector unit in fp32: a lane owns a key slot and a wave eight heads
//      of a query at a time, so a raw score is read once for eight sums; weights go to LDS as bf16;
//   3. weights times values: per kv head [16 rows x 64 keys] [64 keys x 16 coordinates] a wave and column tile, the
//      values straight from the transposed page as the B operand, the outputs in registers for all chunks.
// `splits` workgroups share an item's chunks and leave unnormalised outputs, maxima and sums for the merge kernel.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Maxima and sums over all 64 lanes, in every lane, without LDS: within a row of 16 lanes by DPP moves (lane ^ 1,
// lane ^ 2, the mirror image within eight lanes and within sixteen), then over the four rows by v_permlane16_swap /
// v_permlane32_swap (with both operands equal they hand every lane the other rows' values).
template <int CTRL> __device__ __forceinline__ float amm_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float amm_all_max(float v) {
  v = fmaxf(v, amm_dpp<0xB1>(v));   // quad_perm [1, 0, 3, 2]
  v = fmaxf(v, amm_dpp<0x4E>(v));   // quad_perm [2, 3, 0, 1]
  v = fmaxf(v, amm_dpp<0x141>(v));  // row_half_mirror
  v = fmaxf(v, amm_dpp<0x140>(v));  // row_mirror
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float amm_all_sum(float v) {
  v += amm_dpp<0xB1>(v);
  v += amm_dpp<0x4E>(v);
  v += amm_dpp<0x141>(v);
  v += amm_dpp<0x140>(v);
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}
#define AMM_TILES 16  // output tiles (kv head, column tile) a wave keeps: KV * ceil(D / 64) at most
#define AMM_THREADS 512  // eight waves, two to a SIMD
#define AMM_PIECES 32  // 16-byte pieces of keys, and of values, that a lane asks for per chunk: KV * D / 32 at most
#define AMM_MAX_SPLITS 64
// A barrier that waits for this wave's LDS accesses only: a fence would also wait for the loads from memory in flight.
#define AMM_LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

template <int DS>  // a head's coordinates / 32
__global__ __launch_bounds__(AMM_THREADS) void attn_headmix_mfma_kernel(MixArgs a, int tq, int single, int splits,
                                                                       float* __restrict__ part_o,
                                                                       float* __restrict__ part_ml) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  constexpr int D = 32 * DS, CT = 2 * DS, CTW = (CT + 3) / 4;  // column tiles of a head, and of a wave at most
  const int H = a.H, KV = a.KV, bs = a.bs, group = H / KV, gshift = __builtin_ctz(group), gmask = group - 1;
  const int H8 = (H + 7) & ~7, HB = H8 >> 3;
  // rows of scores, weights and queries are a little longer than what they hold, so that the 16 rows a product's
  // operand is read from (and the 4 a product's result is written to) lie in different banks
  constexpr int SROW = AM_KC + 1, PROW = AM_KC + 8, QROW = D + 8;
  float* sraw = reinterpret_cast<float*>(lds_raw);             // [H][tq][SROW]
  float* mixT = sraw + (((size_t)H * tq * SROW + 3) & ~(size_t)3);  // [H][H8]: mixT[g][h] = mix[h][g], read 16 bytes at a time
  float* row_m = mixT + H * H8;
  float* row_l = row_m + tq * H;
  float* row_a = row_l + tq * H;
  int* pages = reinterpret_cast<int*>(row_a + tq * H);         // [64]
  bf16* pb = reinterpret_cast<bf16*>((reinterpret_cast<uintptr_t>(pages + AM_KC) + 15) & ~(uintptr_t)15);  // [H][tq][PROW]
  bf16* qs = pb + (size_t)H * tq * PROW;                       // [tq][H][QROW]

  // eight waves: wave & 3 says which 16 of a chunk's keys (scores) and which column tiles (values) a wave takes,
  // wave >> 2 which half of the kv heads (the even or the odd ones); two waves share a SIMD and fill each other's waits
  const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave8 = tid / WAVE, wave = wave8 & 3, half = wave8 >> 2;
  const int lr = lane & 15, lg = lane >> 4;
  const int KVh = (KV - half + 1) >> 1;  // kv heads of this wave's half: c = 2 c' + half
  const int item = blockIdx.x, split = blockIdx.y;
  int first, count, row, p0;
  if (single) {
    first = a.items[item];
    count = 1;
    row = a.tok_row ? a.tok_row[first] : first;
    p0 = a.positions[first];
  } else {
    const int* it = a.items + 4 * item;
    first = it[0]; count = it[1]; row = it[2]; p0 = it[3];
  }
  const int* table = a.tables + (size_t)row * a.table_width;
  const bf16* q = reinterpret_cast<const bf16*>(a.q);
  const bf16* kp = reinterpret_cast<const bf16*>(a.k_pages);
  const bf16* vp = reinterpret_cast<const bf16*>(a.v_pages);
  const int HD = H * D, rows_used = tq * group;

  const int hi = p0 + count - 1;
  const int lo = a.window > 0 ? max(0, p0 - a.window + 1) : 0;
  const int pb0 = lo / bs, pb1 = hi / bs;
  const int kept = min(a.keep_first, hi + 1);
  const int pa_end = min((kept + bs - 1) / bs, pb0);
  const int NP = pa_end + (pb1 - pb0 + 1);
  const int ppc = AM_KC / bs;
  const int chunks = (NP + ppc - 1) / ppc;
  const int cps = (chunks + splits - 1) / splits;
  const int ch0 = split * cps, ch1 = min(chunks, ch0 + cps);

  for (int i = tid * 8; i < tq * HD; i += AMM_THREADS * 8) {  // 16 bytes a thread: D % 8 == 0
    const int qi = i / HD, rest = i - qi * HD, h = rest / D, d = rest - h * D;
    bf16x8 v;
    if (qi < count) v = *reinterpret_cast<const bf16x8*>(q + (size_t)(first + qi) * HD + rest);
    else
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (bf16)0.f;
    *reinterpret_cast<bf16x8*>(qs + ((size_t)qi * H + h) * QROW + d) = v;
  }
  for (int i = tid; i < H * H8; i += AMM_THREADS) {
    const int g = i / H8, h = i - g * H8;
    mixT[i] = h < H ? (a.mix ? a.mix[h * H + g] : (h == g ? 1.f : 0.f)) : 0.f;
  }
  for (int i = tid; i < tq * H; i += AMM_THREADS) { row_m[i] = -INFINITY; row_l[i] = 0.f; row_a[i] = 1.f; }

  floatx4 acc[AMM_TILES / 2];
#pragma unroll
  for (int t = 0; t < AMM_TILES / 2; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  // the rows this lane meets: as an A operand row lr, as results rows 4 lg + r
  const int a_qi = lr >> gshift, a_g = lr & gmask;
  const bool a_valid = lr < rows_used;

  for (int ch = ch0; ch < ch1; ++ch) {
    __syncthreads();
    const int u = ch * ppc + lane / bs, off = lane % bs;
    const bool slot_valid = u < NP;
    const int lp = u < pa_end ? u : pb0 + (u - pa_end);
    const int jpos = lp * bs + off;
    if (tid < AM_KC) pages[tid] = slot_valid ? table[lp] : 0;
    __syncthreads();
    // ---- phase 1: scores of this wave's 16 keys for every kv head ---------------------------------
    // (kv head, 32 coordinates) pieces of the wave's keys, eight at a time: all eight are asked for before the first
    // product (a wait for memory per eight)
    // what a lane adds to its addresses, hidden from the compiler at every chunk: it would otherwise keep every
    // piece's address in registers of its own for the whole kernel (a hundred of them) and spill the products' operands
    int lg8 = lg * 8, lrv = lr;
    asm volatile("" : "+v"(lg8), "+v"(lrv));
    const int slot = 16 * wave + lrv;
    const size_t kbase = ((size_t)pages[slot] * KV * bs + slot % bs) * D;
    const int total = KVh * DS;
    const size_t q_at = a_valid ? ((size_t)a_qi * H + a_g) * QROW : 0;  // rows that stand for nothing read row 0 (and are not stored)
    {
      floatx4 sc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int h0 = 0; h0 < AMM_PIECES / 2; h0 += 8) {
        if (h0 >= total) break;
        bf16x8 kb[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int f = min(h0 + i, total - 1);
          const int c = 2 * (f / DS) + half, d0 = (f % DS) * 32;
          kb[i] = *reinterpret_cast<const bf16x8*>(kp + kbase + (size_t)c * bs * D + d0 + lg8);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int f = h0 + i;
          if (f < total) {
            const int c = 2 * (f / DS) + half, ds = f % DS;
            const bf16x8 qa = *reinterpret_cast<const bf16x8*>(qs + q_at + (size_t)c * group * QROW + ds * 32 + lg8);
            if (ds == 0) sc = floatx4{0.f, 0.f, 0.f, 0.f};
            sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa, kb[i], sc, 0, 0, 0);
            if (ds == DS - 1) {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int rho = 4 * lg + r;
                if (rho < rows_used) {
                  const int qi = rho >> gshift, g = rho & gmask;
                  sraw[((size_t)(c * group + g) * tq + qi) * SROW + slot] = sc[r] * a.scale;
                }
              }
            }
          }
        }
      }
    }
    // the first eight (output tile, 32 keys) pieces of the chunk's values are asked for now and arrive while the
    // scores are mixed; a piece that stands for nothing loads what another piece loads and multiplies nothing
    const int vtotal = 2 * KVh * CTW;
    auto value_piece = [&](int f) {
      const int t = min(f >> 1, max(KVh * CTW - 1, 0)), ks = f & 1;
      const int c = min(2 * (t / CTW) + half, KV - 1), ct = min(wave + 4 * (t % CTW), CT - 1);
      const int slot0 = ks * 32 + lg8;  // eight slots of one page: pages hold a multiple of 8 tokens
      return *reinterpret_cast<const bf16x8*>(vp + (((size_t)pages[slot0] * KV + c) * D + ct * 16 + lrv) * bs + slot0 % bs);
    };
    bf16x8 vb0[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) vb0[i] = value_piece(i);
    AMM_LDS_BARRIER();
    // ---- phase 2: mixing, mask, running softmax ------------------------------------------------------
    for (int unit = wave8; unit < tq * HB; unit += 8) {
      const int qi = unit / HB, h0 = (unit - qi * HB) * 8;
      float mixed[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) mixed[j] = 0.f;
#pragma unroll 2
      for (int g = 0; g < H; ++g) {
        const float r = sraw[((size_t)g * tq + qi) * SROW + lane];
        const float4 t0 = *reinterpret_cast<const float4*>(mixT + g * H8 + h0);
        const float4 t1 = *reinterpret_cast<const float4*>(mixT + g * H8 + h0 + 4);
        mixed[0] = fmaf(t0.x, r, mixed[0]); mixed[1] = fmaf(t0.y, r, mixed[1]);
        mixed[2] = fmaf(t0.z, r, mixed[2]); mixed[3] = fmaf(t0.w, r, mixed[3]);
        mixed[4] = fmaf(t1.x, r, mixed[4]); mixed[5] = fmaf(t1.y, r, mixed[5]);
        mixed[6] = fmaf(t1.z, r, mixed[6]); mixed[7] = fmaf(t1.w, r, mixed[7]);
      }
      const int ipos = p0 + qi;
      const bool seen = slot_valid && qi < count && jpos <= ipos &&
                        (a.window <= 0 || ipos - jpos < a.window || jpos < a.keep_first);
      // four rows' maxima and sums at a time, by lane swaps that do not pass through LDS
#pragma unroll
      for (int j0 = 0; j0 < 8; j0 += 4) {
        if (h0 + j0 >= H) break;
        float sv[4], mx[4], m_old[4], pr[4], al[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          sv[j] = seen ? mixed[j0 + j] : -INFINITY;
          mx[j] = sv[j];
          m_old[j] = h0 + j0 + j < H ? row_m[qi * H + h0 + j0 + j] : -INFINITY;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) mx[j] = amm_all_max(mx[j]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          mx[j] = fmaxf(m_old[j], mx[j]);  // the new maximum
          pr[j] = 0.f;
          al[j] = 1.f;
          if (mx[j] > -INFINITY) {
            pr[j] = seen ? expf(sv[j] - mx[j]) : 0.f;
            al[j] = m_old[j] > -INFINITY ? expf(m_old[j] - mx[j]) : 0.f;
          }
          sv[j] = pr[j];  // to be summed over the lanes
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) sv[j] = amm_all_sum(sv[j]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int h = h0 + j0 + j;
          if (h >= H) break;
          const int rr = qi * H + h;
          pb[((size_t)h * tq + qi) * PROW + lane] = (bf16)pr[j];
          if (lane == 0) {
            row_m[rr] = mx[j];
            row_l[rr] = row_l[rr] * al[j] + sv[j];
            row_a[rr] = al[j];
          }
        }
      }
    }
    AMM_LDS_BARRIER();
    // ---- phase 3: weights times values ------------------------------------------------------------------
    const size_t p_at = a_valid ? ((size_t)a_g * tq + a_qi) * PROW : 0;
    auto weigh = [&](int f, const bf16x8& vb, floatx4& o) {  // f static: the tile's accumulator is a register
      const int t = f >> 1, ks = f & 1;
      const int c = 2 * (t / CTW) + half, ct = wave + 4 * (t % CTW);
      if (t < KVh * CTW && ct < CT) {
        if (ks == 0) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int rho = 4 * lg + r;
            if (rho < rows_used) {
              const int qi = rho >> gshift, g = rho & gmask;
              o[r] *= row_a[qi * H + c * group + g];
            }
          }
        }
        const bf16x8 pa = *reinterpret_cast<const bf16x8*>(pb + p_at + (size_t)c * group * tq * PROW + ks * 32 + lg8);
        o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, vb, o, 0, 0, 0);
      }
    };
#pragma unroll
    for (int f = 0; f < 8; ++f) weigh(f, vb0[f], acc[f >> 1]);
    if (vtotal > 8) {  // the other eight pieces (a model of many kv heads or wide heads)
#pragma unroll
      for (int i = 0; i < 8; ++i) vb0[i] = value_piece(8 + i);
#pragma unroll
      for (int f = 8; f < 16; ++f) weigh(f, vb0[f - 8], acc[f >> 1]);
    }
  }
  __syncthreads();
  bf16* out = reinterpret_cast<bf16*>(a.out);
  const size_t pbase = ((size_t)item * splits + split) * tq;
#pragma unroll
  for (int t = 0; t < AMM_TILES / 2; ++t) {
    if (t >= KVh * CTW) break;
    const int c = 2 * (t / CTW) + half, ct = wave + 4 * (t % CTW);
    if (ct >= CT) continue;
    const int d = ct * 16 + lr;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int rho = 4 * lg + r;
      if (rho >= rows_used) continue;
      const int qi = rho >> gshift, h = c * group + (rho & gmask);
      if (qi >= count) continue;
      if (splits == 1) {
        const float l = row_l[qi * H + h];
        if (d < a.Dout) out[((size_t)(first + qi) * H + h) * a.Dout + d] = (bf16)(l > 0.f ? acc[t][r] / l : 0.f);
      } else {
        part_o[((pbase + qi) * H + h) * D + d] = acc[t][r];
      }
    }
  }
  if (splits > 1)
    for (int i = tid; i < tq * H; i += AMM_THREADS) {
      part_ml[(pbase * H + i) * 2] = row_m[i];
      part_ml[(pbase * H + i) * 2 + 1] = row_l[i];
    }
}

// Puts an item's splits together: out = sum_s e^(m_s - M) o_s / sum_s e^(m_s - M) l_s.  A workgroup per (item, head):
// the splits' weights are made once in LDS, then a thread owns a coordinate and its loads do not wait for one another.
__global__ __launch_bounds__(128) void attn_headmix_merge_kernel(const int* __restrict__ items, int single, int tq,
                                                                 int splits, const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml,
                                                                 bf16* __restrict__ out, int H, int D, int Dout) {
  __shared__ float wts[AMM_MAX_SPLITS];
  __shared__ float inv_den;
  const int item = blockIdx.x, h = blockIdx.y;
  const int first = single ? items[item] : items[4 * item], count = single ? 1 : items[4 * item + 1];
  for (int qi = 0; qi < count; ++qi) {
    __syncthreads();
    if (threadIdx.x < WAVE) {  // splits <= 64: one lane each
      const int s = threadIdx.x;
      const size_t at = (((size_t)item * splits + min(s, splits - 1)) * tq + qi) * H + h;
      const float m = s < splits ? part_ml[at * 2] : -INFINITY;
      const float M = wave_max(m);
      const float w = (s < splits && m > -INFINITY) ? expf(m - M) : 0.f;
      const float den = wave_sum(s < splits ? w * part_ml[at * 2 + 1] : 0.f);
      wts[s] = w;
      if (s == 0) inv_den = den > 0.f ? 1.0f / den : 0.f;
    }
    __syncthreads();
    for (int d = threadIdx.x; d < Dout; d += blockDim.x) {
      float num = 0.f;
      for (int s = 0; s < splits; ++s)
        num = fmaf(wts[s], part_o[((((size_t)item * splits + s) * tq + qi) * H + h) * D + d], num);
      out[((size_t)(first + qi) * H + h) * Dout + d] = (bf16)(num * inv_den);
    }
  }
}

static size_t headmix_mfma_lds(int H, int D, int tq) {
  const int H8 = (H + 7) & ~7;
  return ((((size_t)H * tq * (AM_KC + 1) + 3) & ~(size_t)3) + (size_t)H * H8 + 3 * (size_t)tq * H + AM_KC) * 4 + 16 +
         ((size_t)H * tq * (AM_KC + 8) + (size_t)tq * H * (D + 8)) * 2;  // rows padded against bank conflicts
}

// Whether the matrix-core kernel takes these sizes with items of up to `tq` queries (tq * group rows of a tile).
static bool headmix_mfma_takes(int H, int KV, int D, int bs, int tq) {
  if (H <= 0 || KV <= 0 || H % KV || H > 64 || tq < 1) return false;
  const int group = H / KV;
  if (group * tq > 16 || (group & (group - 1))) return false;  // the rows of a tile are cut by shifts
  if (D % 32 || D > 256 || D == 160 || D == 224 || KV * ((D + 63) / 64) > AMM_TILES) return false;
  if (bs % 8 || bs > AM_KC || AM_KC % bs) return false;
  return headmix_mfma_lds(H, D, tq) <= (size_t)(128 << 10);
}

// part_o [num_items, splits, tq, H, D] and part_ml [num_items, splits, tq, H, 2] fp32 where splits > 1.
extern "C" int as_attn_headmix_mfma(const void* q, const void* k_pages, const void* v_pages, const int* items,
                                    int num_items, int tq, int single, const int* positions, const int* tok_row,
                                    const int* tables, int table_width, const float* mix, void* out, int H, int KV,
                                    int D, int Dout, int bs, float scale, int window, int keep_first, int splits,
                                    float* part_o, float* part_ml, hipStream_t stream) {
  if (num_items <= 0) return AS_OK;
  if (single) tq = 1;
  if (!headmix_mfma_takes(H, KV, D, bs, tq) || table_width <= 0 || window < 0 || keep_first < 0 || Dout <= 0 || Dout > D || splits < 1 ||
      splits > AMM_MAX_SPLITS || (splits > 1 && (!part_o || !part_ml)) || (single && !positions))
    return AS_BAD_SHAPE;
  MixArgs a{q, k_pages, v_pages, items, positions, tok_row, tables, table_width, mix, out, H, KV, D, Dout, bs, scale,
            window, keep_first, single};
  const size_t lds = headmix_mfma_lds(H, D, tq);
#define GO(DS)                                                                                                     \
  case DS: {                                                                                                       \
    static bool raised = false; /* a workgroup may ask for more than 64 KB of LDS once the kernel says so */       \
    if (lds > (size_t)(64 << 10) && !raised) {                                                                     \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_headmix_mfma_kernel<DS>),                        \
                              hipFuncAttributeMaxDynamicSharedMemorySize, 128 << 10) != hipSuccess)                \
        return AS_LAUNCH_FAILED;                                                                                   \
      raised = true;                                                                                               \
    }                                                                                                              \
    attn_headmix_mfma_kernel<DS><<<dim3(num_items, splits), AMM_THREADS, lds, stream>>>(a, tq, single, splits,      \
                                                                                       part_o, part_ml);           \
    break;                                                                                                         \
  }
  switch (D / 32) {
    GO(1) GO(2) GO(3) GO(4) GO(6) GO(8)
    default: return AS_BAD_SHAPE;
  }
#undef GO
  if (splits > 1)
    attn_headmix_merge_kernel<<<dim3(num_items, H), 128, 0, stream>>>(items, single, tq, splits, part_o, part_ml,
                                                                      (bf16*)out, H, D, Dout);
  return launch_status();
}

// The max-plus table from short candidate lists.
//
// best[t,u] = max over v != blank of E[t,v] + P[u,v], arg = lowest such v
// (transducer/transducer_cpu.cpp:158-171) costs one add and one compare per (t, u, v) when every
// column is looked at.  Nearly all of them cannot win: with a threshold tE[t] for the frame's
// row of E and tP[u] for the label position's row of P,
//   A_t = { v : E[t,v] > tE[t] },   C_u = { v : P[u,v] > tP[u] },
// every column outside both sets has E[t,v] + P[u,v] <= tE[t] + tP[u] (rounding is monotone, so
// this holds for the rounded sums too).  If the best sum over A_t and C_u is strictly above
// that bound, it is the row's maximum and every column that reaches it is in one of the two
// sets: maximum and lowest index are exact.  A cell that fails the test is flagged and
// evaluated over all columns afterwards.  The thresholds only decide how long the lists are
// and how many cells fail, never what is returned.
//
//   * cand_lists_p_kernel: threshold and ascending list for every row of P, plus P transposed
//     (cand_transpose_p_kernel) so that one candidate column's 64 label positions are one
//     256-byte read;
//   * cand_rows_kernel: per frame, the row of E goes into LDS and gets its threshold and list,
//     and the four wavefronts of the workgroup (64 label positions each, half of either list)
//     evaluate A_t against the transposed P and C_u against the LDS row;
//   * a sample of the cells goes first (two utterances, one frame in kCdSampleEvery): if too many of
//     them fail the test -- scores with a hard upper edge do -- the sample is taken again with
//     lists half as long again (kCdLongE, kCdLongP), and if that fails too everything else
//     returns at once and the all-columns kernel (maxplus_kernel) builds the whole table;
//   * otherwise tiles of 128 frames x 64 label positions with more than kCdTileLimit flagged
//     cells are redone by that kernel, the others' flagged cells one by one, from one list for
//     the whole call that all wavefronts of cand_cells_kernel share: the cost of a failed test
//     is bounded either way.
//
// A threshold is a value with at most `rank` of a wavefront's 64 per-thread maxima above it.
// The rank is chosen (list_rank) so that about 2.3 sqrt(V) columns of a row of E and 0.75 sqrt(V)
// of a row of P end up on a list if the scores are drawn independently, whatever their scale
// (230 and 75 of 10000; the square root keeps the share of cells that fail the test level as
// the vocabulary grows; an entry of P's lists costs twice the bytes of one of E's, hence the
// shorter lists there; one cell in 300 to 800 then fails the test for 5000 to 17000 normally
// distributed columns, and each of those costs the 80 KB of its two rows once more; heavier
// tails fail far less often, scores with a hard upper edge -- uniform, or the sum of two
// uniform ones -- one cell in 50 or more, which is where the sample's limit of one in
// kCdSampleOdds sends a call on to the longer lists, and from there back to every column).  A constant or heavily tied row gets an
// empty list instead of a full one.
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>

#include "rnnt_internal.h"

namespace rnnt {
namespace {

constexpr float kNegInf = -__builtin_huge_valf();
constexpr int kCdThreads = 256;  // four wavefronts
constexpr int kCdWaves = kCdThreads / 64;
constexpr int kCdCap = 192;      // entries per wavefront's quarter of a row's list
constexpr int kCdSeg = kCdCap + 16;  // a quarter's slots: two batches of padding can follow a full one
constexpr int kCdDepth = 384;    // entries of a stored list of P
constexpr int kCdStored = kCdDepth + 16;  // with two batches of padding behind a full list
constexpr float kCdListE = 2.31f;  // list lengths the ranks are derived from, in units of sqrt(V): rows of E
constexpr float kCdListP = 0.88f;  // ... rows of P (their one threshold per row is the largest of four
                                   // wavefronts' values: the lists come out a fifth shorter than that)
constexpr float kCdLongE = 3.5f, kCdLongP = 1.3f;  // the same for the longer lists that a call falls back
                                   // to when too many cells of its sample fail with the usual ones
                                   // (scores with a hard upper edge: uniform ones fail 1 cell in 12
                                   // with the usual lists and 1 in 500 with these)
constexpr int kCdBisect = 16;    // halvings of the key interval
constexpr int kCdFrames = 8;     // frames per workgroup of cand_rows_kernel (16: 5 % slower, more utterances'
                                 // transposed P in flight per die; 4: level; 2: 3 % slower)
constexpr int kCdSampleEvery = 16;  // the sample takes one frame in this many (a multiple of kCdFrames)
constexpr int kCdAheadShort = 10;  // 16-byte pieces of the next row a thread holds while a row is
constexpr int kCdAheadLong = 17;   // evaluated: rows of up to 10240 / 17408 columns
constexpr int kCdBatch = 8;      // candidates per batch (two batches in flight)
constexpr int kCdTileT = 128, kCdTileU = 64;  // the all-columns kernel's tile
constexpr int kCdTileLimit = 128;  // flagged cells a tile may hold and still be redone cell by cell
constexpr int kCdCellGroups = 2048;  // workgroups (of four wavefronts) that share the flagged cells
constexpr int kCdStats = 8;       // ints of CandScratch::stats
constexpr int kCdSampleOdds = 150; // lists go on if at most one sampled cell in this many was flagged
constexpr int kCdSampleMin = 1000; // ... and the sample held at least this many cells (two empty or
                                   // very short utterances say nothing about the scores)
constexpr int kNone = 0x7fffffff;
static_assert(kCdCap % kCdBatch == 0 && kCdDepth % kCdBatch == 0 && kCdBatch % 4 == 0 &&
                  kCdSeg % 4 == 0 &&
                  kCdSampleEvery % kCdFrames == 0,
              "whole batches, read four entries at a time");

// order-preserving map of the floats onto the unsigned integers, and back
__device__ inline unsigned float_key(float x) {
  const unsigned b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ inline float key_float(unsigned k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

__device__ inline int lanes_below(unsigned long long mask) {
  return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0));
}
template <int kLane>
__device__ inline float lane_value(float x) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), kLane));
}

// LDS of one workgroup: the row (Vp floats, Vp = V rounded up to 256), then this
struct RowLists {
  int idx[kCdWaves * kCdSeg];     // columns above the threshold, ascending: wavefront w's quarter
  float val[kCdWaves * kCdSeg];   // of the row in [w kCdSeg, w kCdSeg + n[w]), then {0, -inf}
                                  // up to the next multiple of 2 kCdBatch and one batch more
  unsigned off[kCdWaves * kCdSeg];  // byte offset of the column's row in the transposed P
  int n[kCdWaves];                // entries of each quarter (without the padding)
  float tau[kCdWaves];            // each wavefront's threshold for its own sub-maxima
  int bad[2];                     // a quarter did not fit: the list is not the whole set (by frame parity)
  int quit[2];                    // every tile this frame's cells lie in is redone whole anyway
  float mtop[2][2][64];           // what the second wavefront of a block of label positions
  int marg[2][2][64];             // found, for the first one to merge ([parity][block][lane])
};

__host__ __device__ inline int padded_row(int V) { return (V + 255) & ~255; }
__host__ inline size_t cand_lds_bytes(int V) {
  return sizeof(float) * (size_t)padded_row(V) + sizeof(RowLists);
}

// One row of V scores -> LDS copy (blank and padding at -inf), thresholds, list.  Each wavefront
// owns one quarter of the row (at most 256 kPieces columns) from the load on: fetch_quarter
// requests it into registers -- in cand_rows_kernel one frame ahead, while the previous frame is
// evaluated -- and commit_quarter writes it to LDS and lists the wavefront's columns from those
// registers with the wavefront's own threshold.  Any threshold is valid per column; the row's
// bound is the largest of the four (L->tau).  No wavefront waits for another before the one
// barrier the caller places behind commit_quarter.
// The threshold: every lane keeps the maximum of its own share of the quarter (interleaved
// pieces of four columns); the wavefront finds, by halving the interval of float keys, a value
// with at most `rank` of its 64 maxima above it.
template <int kPieces>
struct QuarterRegs {
  float4 x[kPieces];
};
// A quarter as its loads return it (16-bit scores stay 16-bit until the row is committed: a
// conversion next to the load would wait for it there and then).
template <int kPieces, typename TIO>
struct QuarterBits {
  decltype(load4_bits_once(static_cast<const TIO*>(nullptr))) x[kPieces];
};
template <bool kVec, int kPieces, typename TIO>
__device__ inline void fetch_quarter(const TIO* __restrict__ src, int V,
                                     QuarterBits<kPieces, TIO>& r) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int quarter = padded_row(V) >> 2, c0 = wave * quarter;
#pragma unroll
  for (int i = 0; i < kPieces; ++i) {
    const int c = 256 * i + 4 * lane, v = c0 + c;
    if (c < quarter) {
      if (kVec) r.x[i] = load4_bits_once(src + min(v, V - 4));
      else r.x[i] = load4_any_bits(src, min(v, V - 1), V);
    }
  }
}

// Writes the quarter to LDS (blank and padding at -inf; `r` keeps the padded values) and returns
// the wavefront's threshold.
template <bool kVec, int kPieces, typename TIO>
__device__ inline float quarter_threshold(const QuarterBits<kPieces, TIO>& in,
                                         QuarterRegs<kPieces>& r, int V, int blank, int rank,
                                         float* row) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int quarter = padded_row(V) >> 2, c0 = wave * quarter;
  const float4 none = make_float4(kNegInf, kNegInf, kNegInf, kNegInf);
  float m = kNegInf;
#pragma unroll
  for (int i = 0; i < kPieces; ++i) {
    const int c = 256 * i + 4 * lane, v = c0 + c;
    float4 y = none;
    if (c < quarter) {
      y = widen4(in.x[i], static_cast<const TIO*>(nullptr));
      if (kVec) {
        if (v >= V) y = none;
      } else {
        y.x = v < V ? y.x : kNegInf;
        y.y = v + 1 < V ? y.y : kNegInf;
        y.z = v + 2 < V ? y.z : kNegInf;
        y.w = v + 3 < V ? y.w : kNegInf;
      }
      *reinterpret_cast<float4*>(row + v) = y;
      m = fmaxf(m, fmaxf(fmaxf(y.x, y.y), fmaxf(y.z, y.w)));
    }
    r.x[i] = y;
  }
  const int blank_wave = blank / quarter;  // uniform
  if (wave == blank_wave && lane == (((blank - c0) & 255) >> 2)) row[blank] = kNegInf;

  const unsigned key = float_key(m);
  unsigned lo = 0u, hi = 0xffffffffu;
  for (int it = 0; it < kCdBisect; ++it) {
    const unsigned mid = lo + ((hi - lo) >> 1);
    if (__builtin_popcountll(__ballot(key > mid)) > rank) lo = mid; else hi = mid;
  }
  return key_float(hi);
}

// Lists the wavefront's columns above `tau`, in column order, from the registers; leaves the
// count and `tau` (for the row's bound) in L.
template <int kPieces>
__device__ inline void quarter_list(const QuarterRegs<kPieces>& r, float tau, int V, int blank,
                                    unsigned pitch, int parity, RowLists* L) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int quarter = padded_row(V) >> 2, c0 = wave * quarter;
  const int blank_wave = blank / quarter;  // uniform
  int* idx = L->idx + wave * kCdSeg;
  float* val = L->val + wave * kCdSeg;
  unsigned* off = L->off + wave * kCdSeg;
  int count = 0;
#pragma unroll
  for (int i = 0; i < kPieces; ++i) {
    const float4 y = r.x[i];
    const bool h0 = y.x > tau, h1 = y.y > tau, h2 = y.z > tau, h3 = y.w > tau;
    const unsigned long long m0 = __ballot(h0), m1 = __ballot(h1), m2 = __ballot(h2),
                             m3 = __ballot(h3);
    if (m0 | m1 | m2 | m3) {  // column order: lane after lane, a lane's four columns in turn
      int pos = count + lanes_below(m0) + lanes_below(m1) + lanes_below(m2) + lanes_below(m3);
      const int col = c0 + 256 * i + 4 * lane;
      const float e[4] = {y.x, y.y, y.z, y.w};
      const bool h[4] = {h0, h1, h2, h3};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (h[j]) {
          if (pos < kCdCap) {
            idx[pos] = col + j;
            val[pos] = e[j];
            off[pos] = (unsigned)(col + j) * pitch;
          }
          ++pos;
        }
      }
      count += __builtin_popcountll(m0) + __builtin_popcountll(m1) + __builtin_popcountll(m2) +
               __builtin_popcountll(m3);
    }
  }
  const int kept = min(count, kCdCap);
  if (wave == blank_wave) {  // the registers still hold the blank's score: out of the list with it
#pragma unroll 1
    for (int k = lane; k < kept; k += 64)
      if (idx[k] == blank) val[k] = kNegInf;
  }
  if (lane < ((-kept) & (kCdBatch - 1)) + 2 * kCdBatch) {
    idx[kept + lane] = 0;
    val[kept + lane] = kNegInf;
    off[kept + lane] = 0u;
  }
  if (lane == 0) {
    L->n[wave] = kept;
    L->tau[wave] = tau;
    if (count > kCdCap) L->bad[parity] = 1;
  }
}

// Both at once, with the wavefront's own threshold (rows of E).
template <bool kVec, int kPieces, typename TIO>
__device__ inline void commit_quarter(const QuarterBits<kPieces, TIO>& in, int V, int blank,
                                      unsigned pitch, int rank, int parity, float* row,
                                      RowLists* L) {
  QuarterRegs<kPieces> r;
  const float tau = quarter_threshold<kVec, kPieces>(in, r, V, blank, rank, row);
  quarter_list<kPieces>(r, tau, V, blank, pitch, parity, L);
}

// ------------------------------------------------------------------ lists of P
// Scratch of the list path (Uq = U rounded up to 4, Ub64 = U rounded up to 64)
struct CandScratch {
  float* PT;      // [B][V][Uq]   P transposed
  int2* plist;    // [B][Ub64 / 64][kCdDepth][64]   {4 x column, score bits} of label position
                  // 64 block + lane, ascending columns, padded with {0, -inf}
  int* pcount;    // [B][U]   entries of each list
  float* ptau;    // [B][U]   thresholds (+inf where the list did not fit)
  int* tile_fail; // [B][tiles of 128 frames][tiles of 64 label positions]   flagged cells
  int2* cells;      // [cell_cap]   the flagged cells of the whole call, in the order they were
                    // found: {b T + t, u}
  int cell_cap;     // tiles x kCdTileLimit: room for every cell of every tile that is not redone whole
  int* stats;       // [0] flagged cells of the sample, [1] cells of the sample, [2] the tier the call
                    // goes on with (0: every column, 1: lists, 2: the longer lists), [3] the first
                    // sample failed and the second is to run, [4] entries of `cells`
};

// Which utterances a launch takes, and with which lists.  Phase 0 (a sample): utterance `first`
// (grid index 0) and `second` (index 1, if any), with the lists of `tier` (1: the usual
// lengths, 2: the longer ones; the second sample runs only if the first one failed, stats[3]).
// Phase 1 (the rest): every utterance but those two, with the lists of the tier the samples
// settled on, and nothing at all if that is none (stats[2]).
struct Pass {
  int phase, first, second, tier;
};
__device__ inline int pass_tier(const Pass& ps, const int* stats) {
  if (ps.phase == 0) return (ps.tier == 1 || stats[3] != 0) ? ps.tier : 0;
  return stats[2];
}
__device__ inline int pass_utterance(const Pass& ps, int index, const int* stats) {
  if (pass_tier(ps, stats) == 0) return -1;
  if (ps.phase == 0) return index == 0 ? ps.first : ps.second;
  if (index == ps.first || index == ps.second) return -1;
  return index;
}

template <bool kVec, typename TIO>
__global__ __launch_bounds__(kCdThreads) void cand_lists_p_kernel(const TIO* __restrict__ P,
                                                                  CandScratch w, Dims d, Pass ps,
                                                                  int4 ranks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float* row = reinterpret_cast<float*>(lds_raw);
  RowLists* L = reinterpret_cast<RowLists*>(row + padded_row(d.V));
  const int b = pass_utterance(ps, blockIdx.y, w.stats), u = blockIdx.x, tid = threadIdx.x;
  if (b < 0) return;
  const int blocks = (d.U + 63) >> 6;
  int2* out = w.plist + (((size_t)b * blocks + (u >> 6)) * kCdStored) * 64 + (u & 63);
  const int2 nothing = make_int2(0, __float_as_int(kNegInf));
  if (u >= d.U) {  // a lane of the last block that no label position stands behind
    for (int k = tid; k < kCdStored; k += kCdThreads) out[(size_t)k * 64] = nothing;
    return;
  }
  const TIO* src = P + ((size_t)b * d.U + u) * d.V;
  QuarterBits<kCdAheadLong, TIO> bits;
  QuarterRegs<kCdAheadLong> regs;
  fetch_quarter<kVec, kCdAheadLong>(src, d.V, bits);
  if (tid == 0) L->bad[0] = 0;
  __syncthreads();
  // one threshold for the whole row, the largest of the four wavefronts' (their own would put a
  // fifth more columns on the list for the same bound; for a row of E that is the price of not
  // waiting for the other wavefronts, here the list is built once and walked for every frame)
  const int rank = pass_tier(ps, w.stats) == 2 ? ranks.w : ranks.y;
  const float tau_own = quarter_threshold<kVec, kCdAheadLong>(bits, regs, d.V, d.blank, rank, row);
  if ((tid & 63) == 0) L->tau[tid >> 6] = tau_own;
  __syncthreads();
  const float tau = fmaxf(fmaxf(L->tau[0], L->tau[1]), fmaxf(L->tau[2], L->tau[3]));
  __syncthreads();  // (quarter_list writes L->tau again)
  quarter_list<kCdAheadLong>(regs, tau, d.V, d.blank, 0u, 0, L);
  __syncthreads();
  const int c1 = L->n[0], c2 = c1 + L->n[1], c3 = c2 + L->n[2], total = c3 + L->n[3];
  const bool bad = L->bad[0] != 0 || total > kCdDepth;
  for (int k = tid; k < kCdStored; k += kCdThreads) {
    int2 e = nothing;
    if (!bad && k < total) {
      const int slot = k < c1 ? k : (k < c2 ? kCdSeg + k - c1
                                            : (k < c3 ? 2 * kCdSeg + k - c2 : 3 * kCdSeg + k - c3));
      e = make_int2(4 * L->idx[slot], __float_as_int(L->val[slot]));
    }
    out[(size_t)k * 64] = e;
  }
  if (tid == 0) {
    w.pcount[(size_t)b * d.U + u] = bad ? 0 : total;
    w.ptau[(size_t)b * d.U + u] = bad ? __builtin_huge_valf() : tau;
  }
}

// PT[b][v][u] = P[b][u][v]
template <typename TIO>
__global__ __launch_bounds__(256) void cand_transpose_p_kernel(const TIO* __restrict__ P,
                                                               float* __restrict__ PT, Dims d,
                                                               int Uq, Pass ps,
                                                               const int* __restrict__ stats) {
  __shared__ float tile[32][33];
  const int b = pass_utterance(ps, blockIdx.z, stats), v0 = blockIdx.x * 32, u0 = blockIdx.y * 32;
  if (b < 0) return;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int i = ty; i < 32; i += 8) {
    const int u = u0 + i, v = v0 + tx;
    tile[i][tx] = (u < d.U && v < d.V) ? ldf(P + ((size_t)b * d.U + u) * d.V + v) : 0.0f;
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    const int v = v0 + i, u = u0 + tx;
    if (v < d.V && u < Uq) PT[((size_t)b * d.V + v) * Uq + u] = tile[tx][i];
  }
}

// ------------------------------------------------------------------ rows of E
// A workgroup takes kCdFrames frames of one utterance, one at a time.  Wavefronts 0 and 1 own
// label positions [0, 64) and [64, 128) of a block of 128 and take the first half of either
// list (quarters 0 and 1 of the frame's list, the lower positions of the label positions'
// lists); wavefronts 2 and 3 own the same label positions and take the second half, and hand
// what they found to the first two through LDS.
// A list is walked in batches of kCdBatch candidates: the batch's largest sum is one add and
// half a three-way maximum per candidate, and a lane only notes the first batch that reached
// its maximum.  Afterwards it walks that one batch again, from its last candidate down, and
// keeps the lowest column whose sum equals the maximum.  Lists are in column order, so that
// is the lowest column of the whole half; halves and lists are then merged by (larger sum,
// lower column).
// While a frame is evaluated, every wavefront already holds its quarter of the next frame's row
// in registers (requested right after this frame's row was committed, as the loads return it),
// so the wait for HBM lies behind the evaluation.  The rows are loaded as read-once, and the
// workgroups are dealt to the dies by utterance, so that a die's L2 keeps the transposed P of
// the one or two utterances it is working on.
// kPieces: 16-byte pieces per lane of a wavefront's quarter of a row.
template <bool kVec, int kPieces, typename TIO>
__global__ __launch_bounds__(kCdThreads) void cand_rows_kernel(const TIO* __restrict__ E,
                                                               const int* __restrict__ inLen,
                                                               const int* __restrict__ labLen,
                                                               float* __restrict__ best,
                                                               int* __restrict__ arg,
                                                               CandScratch w, Dims d, int Uq, Pass ps,
                                                               int4 ranks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float* row = reinterpret_cast<float*>(lds_raw);
  RowLists* L = reinterpret_cast<RowLists*>(row + padded_row(d.V));
  // The sample: every kCdSampleEvery-th frame of the sample's utterances, one per workgroup.
  // The rest: every other frame of those, and all frames of the others, kCdFrames per workgroup.
  int b = blockIdx.y, group = blockIdx.x;
  const int tier = pass_tier(ps, w.stats);
  if (tier == 0) return;
  const int rank = tier == 2 ? ranks.z : ranks.x;
  if (ps.phase == 0) b = b == 0 ? ps.first : ps.second;
  else {
    // Workgroups are dealt to the eight dies in launch order, one each in turn; die k takes the
    // k-th eighth of the (utterance, run of frames) pairs, so that at any time its L2 holds the
    // transposed P of one or two utterances instead of everybody's.
    const unsigned n = gridDim.x * gridDim.y, lin = blockIdx.x + gridDim.x * blockIdx.y;
    const unsigned k = lin & 7, slot = lin >> 3, share = n >> 3, extra = n & 7;
    const unsigned pair = k * share + min(k, extra) + slot;
    b = (int)(pair / gridDim.x);
    group = (int)(pair % gridDim.x);
  }
  const bool sampled = b == ps.first || b == ps.second;
  int t_lo = group * (ps.phase == 0 ? kCdSampleEvery : kCdFrames);
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (t_lo >= Tb || Ub == 0) return;
  int t_hi = min(t_lo + kCdFrames, Tb);
  if (ps.phase == 0) t_hi = t_lo + 1;
  else if (sampled && t_lo % kCdSampleEvery == 0) ++t_lo;
  if (t_lo >= t_hi) return;
  const int phase = ps.phase;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int blk = wave & 1, part = wave >> 1;
  const TIO* Eb = E + (size_t)b * d.T * d.V;
  const char* ptb = reinterpret_cast<const char*>(w.PT + (size_t)b * d.V * Uq);
  const char* rowb = reinterpret_cast<const char*>(row);
  const unsigned pitch = 4u * (unsigned)Uq;
  const int blocks = (d.U + 63) >> 6;
  const int tiles_t = (d.T + kCdTileT - 1) / kCdTileT, tiles_u = (d.U + kCdTileU - 1) / kCdTileU;
  // what the first block of 128 label positions needs of P's lists is the same for every frame
  const int u_first = 64 * blk + lane;
  const bool first_valid = u_first < Ub;
  const float ptau_first = first_valid ? w.ptau[(size_t)b * d.U + u_first] : 0.0f;
  int nmax_first = first_valid ? w.pcount[(size_t)b * d.U + u_first] : 0;
#pragma unroll
  for (int s = 1; s < 64; s <<= 1) nmax_first = max(nmax_first, __shfl_xor(nmax_first, s, 64));
  nmax_first = __builtin_amdgcn_readfirstlane(nmax_first);

  // With at most 128 label positions (a lane meets one cell per frame) a lane keeps its results
  // until a group of four anti-diagonals is complete -- its cells of consecutive frames are
  // neighbours in the skewed planes -- and stores the group as one aligned 16-byte piece per plane:
  // a 4-byte store per frame reaches memory as a sector of its own more often than not.  The
  // group a lane is in depends on its label position, so a quarter of the lanes store per frame;
  // what a workgroup's run of frames leaves incomplete at either end goes cell by cell.
  const bool gathered = Ub <= 2 * 64;
  float qtop[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  int qarg[4] = {0, 0, 0, 0};
  QuarterBits<kPieces, TIO> ahead;
  // Once every tile (128 frames x 64 label positions) that a frame's cells lie in holds more
  // flagged cells than are redone one by one, maxplus_kernel redoes all of them over every
  // column whatever is found here: the workgroup then stops (the counters only grow).  An
  // utterance whose scores do not suit lists -- while the sample's did -- so costs a frame or
  // two per tile instead of the whole list pass.  One thread looks, a frame ahead; everybody
  // reads its answer after the barrier in between.
  auto tiles_lost = [&](int t) -> int {
    if (phase == 0) return 0;
    const int* tf = w.tile_fail + ((size_t)b * tiles_t + t / kCdTileT) * tiles_u;
    for (int k = 0; 64 * k < Ub; ++k)
      if (__hip_atomic_load(tf + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) <= kCdTileLimit)
        return 0;
    return 1;
  };
  if (tid == 0) {
    L->bad[0] = L->bad[1] = 0;
    L->quit[0] = tiles_lost(t_lo);
  }
  fetch_quarter<kVec, kPieces>(Eb + (size_t)t_lo * d.V, d.V, ahead);
  __syncthreads();
  int parity = 0;
  for (int t = t_lo; t < t_hi; ++t) {
    // this frame's row is in registers; the next one's is requested before the evaluation
    const int fp = (t - t_lo) & 1;
    if (L->quit[fp]) break;  // uniform
    // (asked before the next row is requested: loads return in order, and waiting for this
    // answer behind the row's loads would wait for the row)
    const int lost_next = (tid == 0 && t + 1 < t_hi) ? tiles_lost(t + 1) : 0;
    commit_quarter<kVec, kPieces>(ahead, d.V, d.blank, pitch, rank, fp, row, L);
    if (t + 1 < t_hi) fetch_quarter<kVec, kPieces>(Eb + (size_t)(t + 1) * d.V, d.V, ahead);
    if (tid == 0) L->quit[fp ^ 1] = lost_next;
    __syncthreads();
    if (tid == 0) L->bad[fp ^ 1] = 0;  // the next frame's flag: nobody sets it before the hand-over barrier
    const float tau = fmaxf(fmaxf(L->tau[0], L->tau[1]), fmaxf(L->tau[2], L->tau[3]));
    const bool bad = L->bad[fp] != 0;
    for (int ub = 0; ub < Ub; ub += 2 * 64, parity ^= 1) {
      const int u = ub + 64 * blk + lane;
      const bool live = ub + 64 * blk < Ub;  // uniform: some of this wavefront's positions exist
      const bool valid = u < Ub;
      const int uc = valid ? u : Ub - 1;
      float top = kNegInf;
      int at = kNone;
      if (live) {
        // ---- A_t against the transposed P
        const unsigned ubyte = 4u * (unsigned)uc;
        float topa = kNegInf;
        int wina = 0;  // first slot of the batch that reached topa
        struct ABatch {
          float p[kCdBatch], x[kCdBatch];
        };
        auto arequest = [&](int slot, ABatch& r) {
          unsigned o[kCdBatch];
#pragma unroll
          for (int j = 0; j < kCdBatch; j += 4) {
            const uint4 ov = *reinterpret_cast<const uint4*>(&L->off[slot + j]);
            const float4 xv = *reinterpret_cast<const float4*>(&L->val[slot + j]);
            o[j] = ov.x; o[j + 1] = ov.y; o[j + 2] = ov.z; o[j + 3] = ov.w;
            r.x[j] = xv.x; r.x[j + 1] = xv.y; r.x[j + 2] = xv.z; r.x[j + 3] = xv.w;
          }
#pragma unroll
          for (int j = 0; j < kCdBatch; ++j)
            r.p[j] = *reinterpret_cast<const float*>(ptb + (o[j] + ubyte));
        };
        auto avisit = [&](int slot, const ABatch& r) {
          float bm = kNegInf;
#pragma unroll
          for (int j = 0; j < kCdBatch; j += 2)
            bm = fmaxf(fmaxf(bm, r.x[j] + r.p[j]), r.x[j + 1] + r.p[j + 1]);
          if (bm > topa) { topa = bm; wina = slot; }
        };
        {
          // this wavefront's two quarters as one run of batches; two are in flight, and past the
          // last one the walk requests (and with an odd count also visits) padding
          const int n0 = __builtin_amdgcn_readfirstlane(L->n[2 * part]);
          const int n1 = __builtin_amdgcn_readfirstlane(L->n[2 * part + 1]);
          const int nb0 = (n0 + kCdBatch - 1) / kCdBatch, nb = nb0 + (n1 + kCdBatch - 1) / kCdBatch;
          const int base0 = 2 * part * kCdSeg, base1 = base0 + kCdSeg - nb0 * kCdBatch;
          auto slot_of = [&](int i) { return (i < nb0 ? base0 : base1) + i * kCdBatch; };
          if (nb > 0) {
            ABatch a0, a1;
            arequest(slot_of(0), a0);
#pragma unroll 1
            for (int i = 0; i < nb; i += 2) {
              arequest(slot_of(i + 1), a1);
              avisit(slot_of(i), a0);
              arequest(slot_of(i + 2), a0);
              avisit(slot_of(i + 1), a1);
            }
          }
        }
        int ata = kNone;
        if (topa > kNegInf) {  // the batch again, last candidate first
          float p[kCdBatch], x[kCdBatch];
          int c[kCdBatch];
#pragma unroll
          for (int j = 0; j < kCdBatch; ++j) {
            c[j] = L->idx[wina + j];
            x[j] = L->val[wina + j];
            p[j] = *reinterpret_cast<const float*>(ptb + (L->off[wina + j] + ubyte));
          }
#pragma unroll
          for (int j = kCdBatch - 1; j >= 0; --j)
            if (x[j] + p[j] == topa) ata = c[j];
        }

        // ---- C_u against the row in LDS
        float topc = kNegInf;
        int winc = 0;  // first list position of the batch that reached topc
        int nmax = nmax_first;
        if (ub > 0) {
          nmax = valid ? w.pcount[(size_t)b * d.U + u] : 0;
#pragma unroll
          for (int s = 1; s < 64; s <<= 1) nmax = max(nmax, __shfl_xor(nmax, s, 64));
          nmax = __builtin_amdgcn_readfirstlane(nmax);
        }
        const int cbatches = (nmax + kCdBatch - 1) / kCdBatch, chalf = (cbatches + 1) >> 1;
        const int c_lo = part * chalf * kCdBatch, c_hi = min(cbatches, (part + 1) * chalf) * kCdBatch;
        // {4 x column, score} of list position k for this lane: plk + 512 k
        const char* plblock = reinterpret_cast<const char*>(
            w.plist + (((size_t)b * blocks + ((ub >> 6) + blk)) * kCdStored) * 64);
        // (lanes past the utterance's last label position read the last one's entries: the same
        // cache lines, where their own would be lines nobody needs)
        const unsigned lane8 = 8u * (unsigned)(uc - ub - 64 * blk);
        struct CBatch {
          int2 e[kCdBatch];
        };
        auto crequest = [&](int k0, CBatch& r) {
          const char* kb = plblock + (size_t)k0 * 512;
#pragma unroll
          for (int j = 0; j < kCdBatch; ++j)
            r.e[j] = *reinterpret_cast<const int2*>((kb + j * 512) + lane8);
        };
        auto cvisit = [&](int k0, const CBatch& r) {
          float bm = kNegInf;
#pragma unroll
          for (int j = 0; j < kCdBatch; j += 2) {
            const float s0 =
                *reinterpret_cast<const float*>(rowb + r.e[j].x) + __int_as_float(r.e[j].y);
            const float s1 = *reinterpret_cast<const float*>(rowb + r.e[j + 1].x) +
                             __int_as_float(r.e[j + 1].y);
            bm = fmaxf(fmaxf(bm, s0), s1);
          }
          if (bm > topc) { topc = bm; winc = k0; }
        };
        if (c_lo < c_hi) {  // (an odd count of batches: one more, the other half's or padding)
          CBatch e0, e1;
          crequest(c_lo, e0);
#pragma unroll 1
          for (int k0 = c_lo; k0 < c_hi; k0 += 2 * kCdBatch) {
            crequest(k0 + kCdBatch, e1);
            cvisit(k0, e0);
            crequest(k0 + 2 * kCdBatch, e0);
            cvisit(k0 + kCdBatch, e1);
          }
        }
        int atc = kNone;
        if (topc > kNegInf) {
          const char* kb = plblock + (size_t)winc * 512 + lane8;  // per lane
          int2 e[kCdBatch];
#pragma unroll
          for (int j = 0; j < kCdBatch; ++j) e[j] = *reinterpret_cast<const int2*>(kb + j * 512);
#pragma unroll
          for (int j = kCdBatch - 1; j >= 0; --j)
            if (*reinterpret_cast<const float*>(rowb + e[j].x) + __int_as_float(e[j].y) == topc)
              atc = e[j].x >> 2;
        }
        top = topa;
        at = ata;
        if (topc > top || (topc == top && atc < at)) { top = topc; at = atc; }
        if (part == 1) {
          L->mtop[parity][blk][lane] = top;
          L->marg[parity][blk][lane] = at;
        }
      }
      __syncthreads();
      if (live && part == 0) {
        const float ot = L->mtop[parity][blk][lane];
        const int oa = L->marg[parity][blk][lane];
        if (ot > top || (ot == top && oa < at)) { top = ot; at = oa; }
        const float bound =
            tau + (ub == 0 ? ptau_first : (valid ? w.ptau[(size_t)b * d.U + u] : 0.0f));
        const bool ok = !bad && top > bound;
        if (gathered) {
          const int dd = t + u, ph = dd & 3;  // per lane
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            qtop[k] = ph == k ? top : qtop[k];
            qarg[k] = ph == k ? (ok ? at : -1) : qarg[k];
          }
          if (valid && (ph == 3 || t == t_hi - 1)) {
            const int held = min(ph, t - t_lo);  // earlier cells of this group the lane holds
            const size_t o = plane_at(d, b, u, dd - ph);  // the group's first anti-diagonal: 16-byte aligned
            if (held == 3) {
              *reinterpret_cast<float4*>(best + o) = make_float4(qtop[0], qtop[1], qtop[2], qtop[3]);
              *reinterpret_cast<int4*>(arg + o) = make_int4(qarg[0], qarg[1], qarg[2], qarg[3]);
            } else {
#pragma unroll
              for (int k = 0; k < 4; ++k)
                if (k <= ph && k >= ph - held) { best[o + k] = qtop[k]; arg[o + k] = qarg[k]; }
            }
          }
        } else if (valid) {
          const size_t o = plane_at(d, b, u, t + u);
          best[o] = top;
          arg[o] = ok ? at : -1;
        }
        const unsigned long long failed = __ballot(valid && !ok);
        const unsigned long long cells = __ballot(valid);
        if (phase == 0 && lane == 0) {
          atomicAdd(&w.stats[0], __builtin_popcountll(failed));
          atomicAdd(&w.stats[1], __builtin_popcountll(cells));
        }
        if (failed) {  // count them per tile and put them on the call's list
          const size_t tile = ((size_t)b * tiles_t + t / kCdTileT) * tiles_u + (ub >> 6) + blk;
          const int n = __builtin_popcountll(failed);
          int base = 0;
          if (lane == 0) {
            atomicAdd(&w.tile_fail[tile], n);
            base = atomicAdd(&w.stats[4], n);
          }
          base = __builtin_amdgcn_readfirstlane(base);
          const int slot = base + lanes_below(failed);
          if (valid && !ok) {
            if ((unsigned)slot < (unsigned)w.cell_cap) w.cells[slot] = make_int2(b * d.T + t, u);
            else atomicMax(&w.tile_fail[tile], kCdTileLimit + 1);  // no room: the tile is redone whole
          }
        }
      }
    }
    // (no barrier here: after the hand-over barrier nobody reads the row or the lists again,
    // and the hand-over arrays are next written two barriers further on)
  }
}

// ------------------------------------------------------------------ flagged cells, one by one
// The wavefronts of the grid share the call's list of flagged cells, one cell at a time each
// (cells of tiles that maxplus_kernel redoes whole are passed over): all columns, each lane
// keeping the lowest column of its own maximum; (larger sum, lower column) merges the lanes.
// Neighbours on the list were flagged together -- the same frame, mostly -- so the four
// wavefronts of a workgroup read the same row of E.
template <typename TIO>
__global__ __launch_bounds__(256) void cand_cells_kernel(const TIO* __restrict__ E,
                                                         const TIO* __restrict__ P,
                                                         float* __restrict__ best,
                                                         int* __restrict__ arg, CandScratch w,
                                                         Dims d) {
  if (w.stats[2] == 0) return;
  const int count = min(w.stats[4], w.cell_cap);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int tiles_t = (d.T + kCdTileT - 1) / kCdTileT, tiles_u = (d.U + kCdTileU - 1) / kCdTileU;
  for (int i = 4 * blockIdx.x + wave; i < count; i += 4 * gridDim.x) {
    const int2 c = w.cells[i];
    const int b = c.x / d.T, t = c.x - b * d.T, u = c.y;
    if (w.tile_fail[((size_t)b * tiles_t + t / kCdTileT) * tiles_u + u / kCdTileU] > kCdTileLimit)
      continue;
    const TIO* e = E + ((size_t)b * d.T + t) * d.V;
    const TIO* p = P + ((size_t)b * d.U + u) * d.V;
    float top = kNegInf;
    int at = kNone;
    // four columns at a time, ascending; eight such pieces of either row requested together
    for (int v0 = 4 * lane; v0 < d.V; v0 += 4 * 64 * 8) {
      float4 x[8], y[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int v = min(v0 + 4 * 64 * k, d.V - 1);
        x[k] = load4_any(e, v, d.V);
        y[k] = load4_any(p, v, d.V);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int v = v0 + 4 * 64 * k;
        const float s[4] = {x[k].x + y[k].x, x[k].y + y[k].y, x[k].z + y[k].z, x[k].w + y[k].w};
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (v + j < d.V && v + j != d.blank && s[j] > top) { top = s[j]; at = v + j; }
      }
    }
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) {
      const float ot = __shfl_xor(top, s, 64);
      const int oa = __shfl_xor(at, s, 64);
      if (ot > top || (ot == top && oa < at)) { top = ot; at = oa; }
    }
    if (lane == 0) {
      const size_t o = plane_at(d, b, u, t + u);
      best[o] = top;
      arg[o] = at == kNone ? 0 : at;  // :160 nothing beat -inf: index 0 stays
    }
  }
}

// After a sample: lists go on if few enough of its cells were flagged (one thread).  After the
// first sample a failure asks for the second, with the longer lists; after the second it sends
// the call to every column.
__global__ void cand_decide_kernel(int* stats, int force, int stage, int* tile_fail,
                                   int tiles_per_utterance, int first, int second) {
  const bool enough = stats[1] >= kCdSampleMin;
  const bool few = enough && (long long)stats[0] * kCdSampleOdds <= (long long)stats[1];
  if (stage == 1) {
    const bool ok = force || few;
    stats[2] = ok ? 1 : 0;
    // (a sample too small to judge by sends the call to every column at once: longer lists
    // would be judged by the same few cells)
    stats[3] = (ok || !enough) ? 0 : 1;
    if (!ok) {  // the second sample redoes and flags the same cells: their first entries go
      stats[0] = stats[1] = 0;
      stats[4] = 0;
      for (int i = 0; i < tiles_per_utterance; ++i) {
        tile_fail[(size_t)first * tiles_per_utterance + i] = 0;
        if (second >= 0) tile_fail[(size_t)second * tiles_per_utterance + i] = 0;
      }
    }
  } else if (stats[3] != 0) {
    stats[2] = few ? 2 : 0;
    stats[3] = 0;
  }
}

__global__ void cand_zero_kernel(int* x, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = 0;
}

// the skewed planes as plain [B][T][U] arrays (cells outside an utterance: -inf / -1)
__global__ __launch_bounds__(256) void table_out_kernel(const float* __restrict__ bestS,
                                                        const int* __restrict__ argS,
                                                        const int* __restrict__ inLen,
                                                        const int* __restrict__ labLen,
                                                        float* __restrict__ best,
                                                        int* __restrict__ arg, Dims d) {
  const int b = blockIdx.z, t = blockIdx.y, u = blockIdx.x * 256 + threadIdx.x;
  if (u >= d.U) return;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const bool cell = t < Tb && u < Ub;
  const size_t o = plane_at(d, b, u, t + u), q = ((size_t)b * d.T + t) * d.U + u;
  best[q] = cell ? bestS[o] : kNegInf;
  arg[q] = cell ? argS[o] : -1;
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
size_t min_size(size_t a, size_t b) { return a < b ? a : b; }
int cand_uq(const Dims& d) { return (d.U + 3) & ~3; }
size_t cand_tiles(const Dims& d) {
  return (size_t)d.B * ((d.T + kCdTileT - 1) / kCdTileT) * ((d.U + kCdTileU - 1) / kCdTileU);
}

void carve(void* base, const Dims& d, CandScratch* w) {
  char* p = static_cast<char*>(base);
  const int Uq = cand_uq(d);
  w->PT = reinterpret_cast<float*>(p);
  p += align256(sizeof(float) * (size_t)d.B * d.V * Uq);
  w->plist = reinterpret_cast<int2*>(p);
  p += align256(sizeof(int2) * (size_t)d.B * ((d.U + 63) / 64) * kCdStored * 64);
  w->pcount = reinterpret_cast<int*>(p);
  p += align256(sizeof(int) * (size_t)d.B * d.U);
  w->ptau = reinterpret_cast<float*>(p);
  p += align256(sizeof(float) * (size_t)d.B * d.U);
  w->tile_fail = reinterpret_cast<int*>(p);
  w->stats = w->tile_fail + cand_tiles(d);  // cleared together
  p += align256(sizeof(int) * (cand_tiles(d) + kCdStats));
  w->cells = reinterpret_cast<int2*>(p);
  w->cell_cap = (int)min_size(cand_tiles(d) * kCdTileLimit, (size_t)1 << 30);
}

// The rank (of 64 per-thread maxima of a wavefront) whose threshold leaves about
// length_in_sqrt_v * sqrt(V) of V independently drawn scores above it: a thread's maximum lies
// above a threshold that a share p of the scores exceeds with probability 1 - (1-p)^(V/256).
int list_rank(float length_in_sqrt_v, int V) {
  const double n = length_in_sqrt_v * std::sqrt((double)V);
  const double r = 64.0 * (1.0 - std::exp(-n / 256.0));
  return r < 8.0 ? 8 : (r > 56.0 ? 56 : (int)(r + 0.5));
}

template <typename K>
int allow_lds(K kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return kOk;
  RNNT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  return kOk;
}

template <typename TIO>
int cand_any(const TIO* E, const TIO* P, const int* inLen, const int* labLen, float* best,
             int* arg, const Dims& d, void* scratch, bool force, hipStream_t s) {
  CandScratch w;
  carve(scratch, d, &w);
  const int Uq = cand_uq(d);
  const bool vec = d.V % 4 == 0 &&
                   ((reinterpret_cast<uintptr_t>(E) | reinterpret_cast<uintptr_t>(P)) &
                    (4 * sizeof(TIO) - 1)) == 0;
  const size_t lds = cand_lds_bytes(d.V);
  const int tiles = (int)cand_tiles(d);
  hipLaunchKernelGGL(cand_zero_kernel, dim3((tiles + kCdStats + 255) / 256), dim3(256), 0, s,
                     w.tile_fail, tiles + kCdStats);
  RNNT_LAUNCH_CHECK("cand_zero_kernel");
  // The sample's utterances first (their lists, their transposed P, one frame in kCdSampleEvery),
  // then the decision; if it is a no, the same sample again with the longer lists, and the
  // decision between those and every column; then everything else -- whose launches return at
  // once if it is every column (as the second sample's do when the first one passed).
  const int first = 0, second = d.B > 1 ? d.B / 2 : -1;
  const Pass sample{0, first, second, 1}, again{0, first, second, 2}, rest{1, first, second, 0};
  const int nsample = d.B > 1 ? 2 : 1;
  const int4 ranks = make_int4(list_rank(kCdListE, d.V), list_rank(kCdListP, d.V),
                               list_rank(kCdLongE, d.V), list_rank(kCdLongP, d.V));
  const int pieces = (padded_row(d.V) / 4 + 255) / 256;  // 16-byte pieces per thread of a quarter of a row
  const int chunks = (d.T + kCdFrames - 1) / kCdFrames, ublocks64 = ((d.U + 63) / 64) * 64;
  const int sample_chunks = (d.T + kCdSampleEvery - 1) / kCdSampleEvery;
#define RNNT_CAND_PASS(VEC, PS, NB, CH, TRANSPOSE)                                               \
  do {                                                                                           \
    if (TRANSPOSE) {                                                                             \
      hipLaunchKernelGGL((cand_transpose_p_kernel<TIO>),                                         \
                         dim3((d.V + 31) / 32, (Uq + 31) / 32, NB), dim3(256), 0, s, P, w.PT, d, \
                         Uq, PS, w.stats);                                                       \
      RNNT_LAUNCH_CHECK("cand_transpose_p_kernel");                                              \
    }                                                                                            \
    hipLaunchKernelGGL((cand_lists_p_kernel<VEC, TIO>), dim3(ublocks64, NB), dim3(kCdThreads),  \
                       lds, s, P, w, d, PS, ranks);                                              \
    RNNT_LAUNCH_CHECK("cand_lists_p_kernel");                                                    \
    if (pieces <= kCdAheadShort)                                                                 \
      hipLaunchKernelGGL((cand_rows_kernel<VEC, kCdAheadShort, TIO>), dim3(CH, NB),              \
                         dim3(kCdThreads), lds, s, E, inLen, labLen, best, arg, w, d, Uq, PS,    \
                         ranks);                                                                 \
    else                                                                                         \
      hipLaunchKernelGGL((cand_rows_kernel<VEC, kCdAheadLong, TIO>), dim3(CH, NB),               \
                         dim3(kCdThreads), lds, s, E, inLen, labLen, best, arg, w, d, Uq, PS,    \
                         ranks);                                                                 \
    RNNT_LAUNCH_CHECK("cand_rows_kernel");                                                       \
  } while (0)
#define RNNT_CAND_DECIDE(STAGE)                                                                  \
  do {                                                                                           \
    hipLaunchKernelGGL(cand_decide_kernel, dim3(1), dim3(1), 0, s, w.stats, force ? 1 : 0,       \
                       STAGE, w.tile_fail, tiles / d.B, first, second);                          \
    RNNT_LAUNCH_CHECK("cand_decide_kernel");                                                     \
  } while (0)
#define RNNT_CAND_PASSES(VEC)                                                                    \
  do {                                                                                           \
    RNNT_TRY(allow_lds(cand_lists_p_kernel<VEC, TIO>, lds));                                     \
    RNNT_TRY(allow_lds(cand_rows_kernel<VEC, kCdAheadShort, TIO>, lds));                         \
    RNNT_TRY(allow_lds(cand_rows_kernel<VEC, kCdAheadLong, TIO>, lds));                          \
    RNNT_CAND_PASS(VEC, sample, nsample, sample_chunks, true);                                   \
    RNNT_CAND_DECIDE(1);                                                                         \
    RNNT_CAND_PASS(VEC, again, nsample, sample_chunks, false);                                   \
    RNNT_CAND_DECIDE(2);                                                                         \
    RNNT_CAND_PASS(VEC, rest, d.B, chunks, true);                                                \
  } while (0)
  if (vec) RNNT_CAND_PASSES(true);
  else RNNT_CAND_PASSES(false);
#undef RNNT_CAND_PASS
#undef RNNT_CAND_DECIDE
#undef RNNT_CAND_PASSES
  return kOk;
}

template <typename TIO>
int cells_any(const TIO* E, const TIO* P, const int* inLen, const int* labLen, float* best,
              int* arg, const Dims& d, void* scratch, hipStream_t s) {
  CandScratch w;
  carve(scratch, d, &w);
  const int groups = (int)min_size(kCdCellGroups, ((size_t)w.cell_cap + 3) / 4);
  hipLaunchKernelGGL((cand_cells_kernel<TIO>), dim3(groups), dim3(256), 0, s, E, P, best, arg, w,
                     d);
  RNNT_LAUNCH_CHECK("cand_cells_kernel");
  return kOk;
}

}  // namespace

int maxplus_tile_limit() { return kCdTileLimit; }

// Whether the list path can take this shape at all: a quarter of a row fits the registers a
// wavefront keeps for it (which also keeps a row and its lists inside a compute unit's LDS), an
// offset into one utterance's transposed P fits 31 bits, and so does a count of the cells.
bool maxplus_lists_possible(const Dims& d) {
  if (d.B == 0 || d.T == 0 || d.U == 0 || d.V < 4) return false;
  if (padded_row(d.V) > 4 * 256 * kCdAheadLong) return false;
  if ((size_t)d.V * cand_uq(d) >= ((size_t)1 << 29)) return false;
  if ((size_t)d.B * d.T * d.U >= ((size_t)1 << 31)) return false;  // cells are counted in an int
  return true;
}

// Where the list path is tried without being asked for (measured on normally distributed
// scores, B = 32, T = 2000).  Looking at every column costs time in proportion to U x V; the
// list path's time is mostly the staging of the rows of E, in proportion to V, and grows slowly
// with U.  The two are level at U = 101 with 2000 columns, at U = 33 with 4000-10000 and at
// U = 64 with 4000; lists are 10 % ahead at (U, V) = (33, 10000) and (64, 4000), 15 % at
// (101, 3000-4000), 22 % at (51-64, 10000), 30-47 % at U = 101 from 5000 columns up, and
// further ahead on small grids (B x T of a few thousand frames, where the all-columns kernel's
// tiles leave most of the device idle).  Two workgroups' rows and lists must fit a compute
// unit's LDS (about 17400 columns; with one workgroup nothing covers the staging of a row).
// Whether a call goes through with it is decided on its own scores (cand_decide_kernel).
bool maxplus_lists_pay(const Dims& d) {
  return maxplus_lists_possible(d) && d.V >= 3000 && (size_t)d.U * d.V >= 250000 &&
         2 * cand_lds_bytes(d.V) <= 160 * 1024;
}

size_t maxplus_lists_bytes(const Dims& d) {
  if (!maxplus_lists_possible(d)) return 0;
  const int Uq = cand_uq(d);
  return align256(sizeof(float) * (size_t)d.B * d.V * Uq) +
         align256(sizeof(int2) * (size_t)d.B * ((d.U + 63) / 64) * kCdStored * 64) +
         2 * align256(sizeof(int) * (size_t)d.B * d.U) +
         align256(sizeof(int) * (cand_tiles(d) + kCdStats)) +
         align256(sizeof(int2) * min_size(cand_tiles(d) * kCdTileLimit, (size_t)1 << 30));
}

void maxplus_lists_counters(void* scratch, const Dims& d, const int** tile_fail,
                            const int** lists_on) {
  CandScratch w;
  carve(scratch, d, &w);
  *tile_fail = w.tile_fail;
  *lists_on = w.stats + 2;
}

int launch_table_out(const float* bestS, const int* argS, const int* inLen, const int* labLen,
                     float* best, int* arg, const Dims& d, hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  hipLaunchKernelGGL(table_out_kernel, dim3((d.U + 255) / 256, d.T, d.B), dim3(256), 0, s, bestS,
                     argS, inLen, labLen, best, arg, d);
  RNNT_LAUNCH_CHECK("table_out_kernel");
  return kOk;
}

int launch_maxplus_lists(const float* E, const float* P, const int* inLen, const int* labLen,
                         float* best, int* arg, const Dims& d, void* scratch, bool force,
                         hipStream_t s) {
  return cand_any(E, P, inLen, labLen, best, arg, d, scratch, force, s);
}
int launch_maxplus_lists(const bf16_t* E, const bf16_t* P, const int* inLen, const int* labLen,
                         float* best, int* arg, const Dims& d, void* scratch, bool force,
                         hipStream_t s) {
  return cand_any(E, P, inLen, labLen, best, arg, d, scratch, force, s);
}
int launch_maxplus_lists(const f16_t* E, const f16_t* P, const int* inLen, const int* labLen,
                         float* best, int* arg, const Dims& d, void* scratch, bool force,
                         hipStream_t s) {
  return cand_any(E, P, inLen, labLen, best, arg, d, scratch, force, s);
}
int launch_maxplus_cells(const float* E, const float* P, const int* inLen, const int* labLen,
                         float* best, int* arg, const Dims& d, void* scratch, hipStream_t s) {
  return cells_any(E, P, inLen, labLen, best, arg, d, scratch, s);
}
int launch_maxplus_cells(const bf16_t* E, const bf16_t* P, const int* inLen, const int* labLen,
                         float* best, int* arg, const Dims& d, void* scratch, hipStream_t s) {
  return cells_any(E, P, inLen, labLen, best, arg, d, scratch, s);
}
int launch_maxplus_cells(const f16_t* E, const f16_t* P, const int* inLen, const int* labLen,
                         float* best, int* arg, const Dims& d, void* scratch, hipStream_t s) {
  return cells_any(E, P, inLen, labLen, best, arg, d, scratch, s);
}

}  // namespace rnnt

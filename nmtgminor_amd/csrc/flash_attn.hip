// Attention over packed variable-length sequences without the [heads, len_q, len_k] score tensor: what the reference
// gets from the third-party module flash_attn_cuda (onmt/modules/optimized/flash_mha.py:32-75: fwd / bwd over
// [total_tokens, heads, head_dim] tensors with cumulative sequence lengths).
//
// Forward, one block per (sequence, head, 128 queries), four wavefronts of 32 queries each:
//   the wavefront's query rows stay in registers as MFMA operands; keys and values arrive in tiles of 64 keys through
//   LDS (loaded into registers one tile ahead, two LDS buffers, one barrier per tile);
//   S^T = K Q^T on v_mfma_f32_32x32x16 puts one query per lane pair (l, l ^ 32) and 32 of the tile's 64 keys in each
//   lane's accumulators, so the running maximum and sum of the online softmax are per-lane scalars;
//   the probabilities are rounded to the 16-bit type, moved from accumulator to operand layout with two
//   v_permlane32_swap per 16 keys, and multiplied with V^T, read from LDS with the transposing read.
// Backward, two kernels with the same tiling, both recomputing S from Q, K and the saved log-sum-exp:
//   dQ kernel  (block = 128 queries, loop over key tiles): D = rowsum(dO * O), dP^T = V dO^T, dS = P (dP - D),
//              dQ^T += K^T dS^T;
//   dK/dV kernel (block = 128 keys, loop over query tiles of 64): the mirror image with one key per lane pair:
//              dV^T += dO^T P, dK^T += Q^T dS.
//   No atomics and no accumulation across blocks: results do not depend on scheduling.
// Dropout keeps element (query i, key j) of (sequence b, head h) when byte 4 (i % 4) + (j % 4) of the Philox block with
// index ((b H + h) ceil(max_q / 4) + i / 4) ceil(max_k / 4) + j / 4 is below round(256 (1 - p)); kept probabilities are
// scaled by 256 / that threshold, so the expectation is exact although p is quantised to 1/256. The three kernels do
// not run the generator (its ten rounds of quarter-rate integer multiplies cost more than the softmax): a small kernel
// ahead of them turns the decisions into one bit per element, one 32-bit word per (group of 32 queries, key). In the
// query-major kernels (forward, dQ) a lane pair is a query and an accumulator register a key, so the pair of words
// of the two keys that a register holds in the two halves of the wavefront IS the lane mask of a select: it is loaded
// into scalar registers and costs no vector instruction besides the select. The key-major kernel (dK / dV) loads its
// key's word per group of queries and tests bits. An explicit byte mask is turned into the same words.
#include "gemm.hip.h"

namespace nmtg {
namespace {

constexpr int FA_ROWS = 128;   // queries (forward, dQ) or keys (dK/dV) per block: 32 per wavefront
constexpr int FA_TILE = 64;    // rows of the streamed operand per LDS tile
constexpr int FA_THREADS = 256;
constexpr float FA_NEG = -1e30f;
constexpr float FA_LAZY = 8.f;   // log2 of the growth of a row maximum that moves the softmax's reference point
constexpr float FA_LOG2E = 1.4426950408889634f;

struct FaArgs {
  const void *q, *k, *v, *o, *d_o;
  void *out, *dq, *dk, *dv;
  float* lse;      // [B, H, max_q]
  float* delta;    // [B, H, max_q]
  const int32_t *cu_q, *cu_k;   // both null: batch-strided call, see seq_span()
  int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh, o_st, o_sh, do_st, do_sh, dq_st, dq_sh, dk_st, dk_sh, dv_st, dv_sh;
  int64_t q_sb, k_sb, v_sb, o_sb, do_sb, dq_sb, dk_sb, dv_sb;   // per sequence, 0 in packed calls
  const uint8_t* pad;    // batch-strided calls: key padding mask [B, max_k], 1 = masked, or null
  const int32_t* kinfo;  // with pad: [B, kinfo_pitch], see flash_key_info_kernel
  int kinfo_pitch;       // 1 + ceil(max_k / 64)
  const uint8_t* tmask;  // batch-strided calls: time mask [max_q, max_k] shared by every sequence and head, 1 = masked, or null
  const int32_t *qinfo, *kqinfo;   // with tmask: summaries by 32 queries x 64 keys and by 32 keys x 64 queries (flash_time_info_kernel)
  int qinfo_pitch, kqinfo_pitch;   // 1 + ceil(max_k / 64) and 2 + ceil(max_q / 64)
  // The mask itself, one bit per element in the order of a lane's 32 accumulator registers (tile_bit()): a lane reads ONE
  // word per masked tile. pad_bits [B][key tiles][2], tq_bits [max_q][key tiles][2] (a query's keys), tk_bits
  // [max_k][query tiles][2] (a key's queries); the last index is the lane's half of the wavefront.
  const uint32_t *pad_bits, *tq_bits, *tk_bits;
  int key_tiles, query_tiles;
  int heads, max_q, max_k;
  float scale, scale_log2;
  int causal;
  const uint8_t* mask;   // explicit keep-mask [B, H, max_q, max_k] (bit kernel, mode 1)
  uint8_t* mask_out;     // where the drawn mask is written as bytes, or null (bit kernel, mode 2)
  uint32_t thr;          // keep when byte < thr (bit kernel, mode 2)
  float drop_scale;
  uint64_t seed, offset;
  // keep bits [B H, q32 groups of 32 queries, kp keys]: bit (i % 32) of word bit_slot(j) of row (b H + h, i / 32)
  uint32_t* bits;
  int q32, kp;           // 4 ceil(max_q / 128) and 64 ceil(max_k / 64)
};

// Inside each group of eight keys the words are stored in the order 0, 4, 1, 5, 2, 6, 3, 7: the two keys that one
// accumulator register holds in the two halves of a wavefront (j and j + 4) lie side by side as one 64-bit lane mask.
__device__ __forceinline__ int bit_slot(int key) { return (key & ~7) | ((key & 3) << 1) | ((key >> 2) & 1); }

typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));

// lanes 32..63 of `a` change places with lanes 0..31 of `b`
__device__ __forceinline__ void swap_halves(uint32_t& a, uint32_t& b) {
  const u32x2_t r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  a = r[0];
  b = r[1];
}
// f(own value, value of lane ^ 32)
__device__ __forceinline__ float pair_max(float v) {
  uint32_t a = __float_as_uint(v), b = a;
  swap_halves(a, b);
  return fmaxf(__uint_as_float(a), __uint_as_float(b));
}
__device__ __forceinline__ float pair_sum(float v) {
  uint32_t a = __float_as_uint(v), b = a;
  swap_halves(a, b);
  return __uint_as_float(a) + __uint_as_float(b);
}

// two floats rounded (to nearest even) into one register of two 16-bit elements, one conversion instruction
typedef float f32x2_t __attribute__((ext_vector_type(2)));
template <typename T> struct pair_of;
template <> struct pair_of<f16_t> { typedef _Float16 type __attribute__((ext_vector_type(2))); };
template <> struct pair_of<bf16_t> { typedef __bf16 type __attribute__((ext_vector_type(2))); };
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, typename pair_of<T>::type));
}

// Accumulator registers r0 .. r0+7 of a 32 x 32 tile (lane (col, half) holds rows 8 (r / 4) + 4 half + r % 4) as the
// B operand of the next product: lane (col, half) holds rows 16 (r0 / 8) + 8 half .. + 7.
template <typename T>
__device__ __forceinline__ uint4 acc_to_operand(const float* p) {
  uint32_t g0a = pack2<T>(p[0], p[1]), g0b = pack2<T>(p[2], p[3]), g1a = pack2<T>(p[4], p[5]), g1b = pack2<T>(p[6], p[7]);
  swap_halves(g0a, g1a);
  swap_halves(g0b, g1b);
  return make_uint4(g0a, g0b, g1a, g1b);
}

// ---- LDS images of a [64 rows][D] tile, rows of D 16-bit elements = D / 8 chunks of 16 bytes ----
// "row image": chunk c of row r at position c ^ (r & 7); read as the A operand (lane = row, 8 consecutive columns).
// "transposed image": chunk c of row r at position c ^ 2 (r & 3); read with ds_read_b64_tr_b16 as the A operand of the
// transposed tile (lane = column, 8 consecutive rows).
template <int D>
__device__ __forceinline__ uint32_t row_image_at(int r, int c) { return static_cast<uint32_t>(r * (2 * D) + ((c ^ (r & 7)) * 16)); }
template <int D>
__device__ __forceinline__ uint32_t tr_image_at(int r, int c) { return static_cast<uint32_t>(r * (2 * D) + ((c ^ (2 * (r & 3))) * 16)); }

template <int D>
struct Staged {
  static constexpr int CH = D / 8;
  static constexpr int N = FA_TILE * CH / FA_THREADS;
  uint4 v[N];
  // rows row0 .. row0+63 of a sequence of `len` rows that starts at `base` (head offset applied); rows past the end are zeros
  template <typename T>
  __device__ __forceinline__ void load(const T* base, int64_t stride, int row0, int len) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int id = (static_cast<int>(threadIdx.x) & (FA_THREADS - 1)) + FA_THREADS * i;   // a block may hold several groups of FA_THREADS
      const int r = id / CH, c = id % CH;
      v[i] = make_uint4(0, 0, 0, 0);
      if (row0 + r < len) v[i] = *reinterpret_cast<const uint4*>(base + static_cast<int64_t>(row0 + r) * stride + 8 * c);
    }
  }
  __device__ __forceinline__ void store_rows(uint8_t* img) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int id = (static_cast<int>(threadIdx.x) & (FA_THREADS - 1)) + FA_THREADS * i;   // a block may hold several groups of FA_THREADS
      *reinterpret_cast<uint4*>(img + row_image_at<D>(id / CH, id % CH)) = v[i];
    }
  }
  __device__ __forceinline__ void store_transposed(uint8_t* img) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int id = (static_cast<int>(threadIdx.x) & (FA_THREADS - 1)) + FA_THREADS * i;   // a block may hold several groups of FA_THREADS
      *reinterpret_cast<uint4*>(img + tr_image_at<D>(id / CH, id % CH)) = v[i];
    }
  }
};

// A operand from the row image: rows 32 i + (lane & 31), columns 16 s + 8 (lane >> 5) .. + 7
template <int D>
__device__ __forceinline__ uint4 read_rows(const uint8_t* img, int i, int s, int lane) {
  return *reinterpret_cast<const uint4*>(img + row_image_at<D>(32 * i + (lane & 31), 2 * s + (lane >> 5)));
}
// A operand of the transposed tile: columns 32 i + (lane & 31), rows 16 kk + 8 (lane >> 5) .. + 7. Within 16 lanes the
// transposing read takes 4 rows x 16 columns and hands each lane the 4 rows of its own column.
template <int D>
__device__ __forceinline__ uint4 read_transposed(const uint8_t* img, int i, int kk, int lane) {
  const int r = 16 * kk + 8 * (lane >> 5) + ((lane >> 2) & 3);
  const int c = 4 * i + 2 * ((lane >> 4) & 1) + ((lane >> 1) & 1);
  const uint8_t* p = img + tr_image_at<D>(r, c) + (lane & 1) * 8;      // r + 4 has the same r & 3: same swizzle
  const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p));
  const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 4 * 2 * D));
  union { s16x4_t s[2]; uint4 u; } cv;
  cv.s[0] = lo;
  cv.s[1] = hi;
  return cv.u;
}

// The wavefront's 32 resident rows as the B operand: lane (row, half) holds columns 16 s + 8 half .. + 7
template <typename T, int D>
__device__ __forceinline__ void load_resident(uint4 (&f)[D / 16], const T* base, int64_t stride, int row, int len, int lane) {
  const T* p = base + static_cast<int64_t>(row) * stride + 8 * (lane >> 5);
#pragma unroll
  for (int s = 0; s < D / 16; ++s) f[s] = row < len ? *reinterpret_cast<const uint4*>(p + 16 * s) : make_uint4(0, 0, 0, 0);
}

// Touches the rows that stay in registers for a whole tile loop (the queries of the inference kernel), in front of the
// loop and outside any branch. They are loaded under conditions, and without a use that the compiler sees on every path
// it repeats the wait for them inside the loop, behind the loads of the next tile: every tile then waits for its own
// prefetch. Not for the training kernels: behind a statement like this one (or a wait instruction of our own) the
// compiler no longer reads wave-uniform values (tile classes, dropout bits) through the scalar cache but with vector
// loads, each waited for on the spot.
template <int N>
__device__ __forceinline__ void registers_landed(const uint4 (&f)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" ::"v"(f[i].x), "v"(f[i].y), "v"(f[i].z), "v"(f[i].w));
}

// Where sequence b lies and how long it is. Packed calls read the cumulative lengths. Batch-strided calls (no cumulative
// lengths) give every sequence max_q queries and max_k keys, b * *_sb elements into each tensor; a key padding mask cuts
// the keys at the last live one, and masked keys below that are handled tile by tile (pad_tile()).
struct SeqSpan { int qs, lq, ks, lk; };
__device__ __forceinline__ SeqSpan seq_span(const FaArgs& a, int b) {
  SeqSpan s;
  if (a.cu_q != nullptr) {
    s.qs = a.cu_q[b];
    s.lq = min(a.cu_q[b + 1] - s.qs, a.max_q);
    s.ks = a.cu_k[b];
    s.lk = min(a.cu_k[b + 1] - s.ks, a.max_k);
  } else {
    s.qs = 0;
    s.lq = a.max_q;
    s.ks = 0;
    s.lk = a.pad != nullptr ? a.kinfo[static_cast<int64_t>(b) * a.kinfo_pitch] : a.max_k;
  }
  return s;
}
// Whether key tile t holds masked keys that the sequence length does not already cut off, for the wavefront's group of
// 32 queries. MODE 1: key padding mask (the same for every query of sequence b). MODE 2: time mask (the same for every
// sequence). A tile of a time mask whose keys are all masked counts too (class 2; the blocks skip such tiles where they
// lie behind the last live one, see tile_bound()).
template <int MODE>
__device__ __forceinline__ bool masked_tile(const FaArgs& a, int b, int group, int t) {
  if constexpr (MODE == 1) return a.kinfo[static_cast<int64_t>(b) * a.kinfo_pitch + 1 + t] != 0;
  else return a.qinfo[static_cast<int64_t>(group) * a.qinfo_pitch + 1 + t] != 0;
}
// the packed mask of tile t for this lane's query qr (inside the mask): one load
template <int MODE>
__device__ __forceinline__ uint32_t tile_mask_bits(const FaArgs& a, int b, int qr, int t, int half) {
  if constexpr (MODE == 1) return a.pad_bits[(static_cast<int64_t>(b) * a.key_tiles + t) * 2 + half];
  else return a.tq_bits[(static_cast<int64_t>(qr) * a.key_tiles + t) * 2 + half];
}
// time mask: the number of key tiles that a block of 128 queries has to visit (behind it every key is masked for all of them)
__device__ __forceinline__ int tile_bound(const FaArgs& a, int block) {
  const int groups = (a.max_q + 31) / 32;
  int n = 0;
  for (int i = 0; i < FA_ROWS / 32; ++i) n = max(n, a.qinfo[static_cast<int64_t>(min(4 * block + i, groups - 1)) * a.qinfo_pitch]);
  return n;
}

// Bit i = 16 n + r of a packed mask word stands for element (n, r) of a lane's 32 accumulator registers of a tile:
// index 64 t + 32 n + 8 (r / 4) + 4 half + r % 4 along the tile's 64 keys (queries, in the key-major kernel).
__device__ __forceinline__ int tile_bit_index(int t, int i, int half) {
  const int n = i >> 4, r = i & 15;
  return FA_TILE * t + 32 * n + 8 * (r / 4) + 4 * half + r % 4;
}
// The packed word of one half from the tile's 64 bits in index order (a wavefront's ballot, lane = index within the tile).
__device__ __forceinline__ uint32_t tile_word_of(uint64_t in_order, int half) {
  uint32_t word = 0;
#pragma unroll
  for (int n = 0; n < 2; ++n)
#pragma unroll
    for (int g = 0; g < 4; ++g)
      word |= static_cast<uint32_t>((in_order >> (32 * n + 8 * g + 4 * half)) & 0xfu) << (16 * n + 4 * g);
  return word;
}

// Time mask [max_q, max_k] -> the two summaries. Blocks 0 .. ceil(max_q / 32) - 1 write qinfo: per group of 32 queries,
// word 0 = 1 + the last key tile with a live key (0: none), word 1 + t = class of tile t (0 no masked key, 1 some, 2 all).
// The other blocks write kqinfo: per group of 32 keys, word 0 = the first tile of 64 queries with a live element (the tile
// count if none), word 1 = 1 + the last one, word 2 + t = class of query tile t. Elements outside the mask do not count.
__global__ __launch_bounds__(256) void flash_time_info_kernel(const uint8_t* tmask, int max_q, int max_k, int32_t* qinfo,
                                                              int qpitch, int32_t* kqinfo, int kpitch, uint32_t* tq_bits,
                                                              uint32_t* tk_bits) {
  __shared__ int first[4], last[4];
  const int tid = static_cast<int>(threadIdx.x), wave = tid >> 6, lane = tid & 63;
  const int qgroups = (max_q + 31) / 32, kgroups = (max_k + 31) / 32;
  if (static_cast<int>(blockIdx.x) >= qgroups + kgroups) {
    // the blocks behind the summaries pack the mask: one thread per word, first the words by query, then those by key
    // (a wavefront per 64 x 64 patch with ballots was measured too: 22 us against 16 for the whole kernel at T = 512)
    const int nkt = qpitch - 1, nqt = kpitch - 2;
    const int64_t by_q = static_cast<int64_t>(max_q) * nkt * 2, by_k = static_cast<int64_t>(max_k) * nqt * 2;
    const int64_t w = (static_cast<int64_t>(blockIdx.x) - qgroups - kgroups) * 256 + tid;
    if (w < by_q) {
      const int half = static_cast<int>(w & 1), t = static_cast<int>((w >> 1) % nkt), q = static_cast<int>((w >> 1) / nkt);
      const uint8_t* row = tmask + static_cast<int64_t>(q) * max_k;
      // the 32 bytes first (independent loads, out together), then the word
      uint8_t byte[32];
#pragma unroll
      for (int i = 0; i < 32; ++i) byte[i] = row[min(tile_bit_index(t, i, half), max_k - 1)];
      uint32_t word = 0;
#pragma unroll
      for (int i = 0; i < 32; ++i) word |= (byte[i] != 0 ? 1u : 0u) << i;
      tq_bits[w] = word;
    } else if (w < by_q + by_k) {
      const int64_t u = w - by_q;
      const int half = static_cast<int>(u & 1), t = static_cast<int>((u >> 1) % nqt), k = static_cast<int>((u >> 1) / nqt);
      uint8_t byte[32];
#pragma unroll
      for (int i = 0; i < 32; ++i) byte[i] = tmask[static_cast<int64_t>(min(tile_bit_index(t, i, half), max_q - 1)) * max_k + k];
      uint32_t word = 0;
#pragma unroll
      for (int i = 0; i < 32; ++i) word |= (byte[i] != 0 ? 1u : 0u) << i;
      tk_bits[u] = word;
    }
    return;
  }
  const bool by_query = static_cast<int>(blockIdx.x) < qgroups;
  const int g = by_query ? static_cast<int>(blockIdx.x) : static_cast<int>(blockIdx.x) - qgroups;
  const int ntiles = by_query ? qpitch - 1 : kpitch - 2;
  int32_t* out = by_query ? qinfo + static_cast<int64_t>(g) * qpitch + 1 : kqinfo + static_cast<int64_t>(g) * kpitch + 2;
  int lo = ntiles, hi = 0;
  for (int t = wave; t < ntiles; t += 4) {
    // by_query: this lane's key against the group's 32 queries; otherwise this lane's query against the group's 32 keys
    const int mine = FA_TILE * t + lane;
    const bool valid = mine < (by_query ? max_k : max_q);
    // (no early exit and clamped addresses: the 32 loads are independent and go out together)
    bool any = false, all = true;
    const int mine_c = min(mine, (by_query ? max_k : max_q) - 1), others = by_query ? max_q : max_k;
#pragma unroll
    for (int r = 0; r < 32; ++r) {
      const int other = 32 * g + r, other_c = min(other, others - 1);
      const int q = by_query ? other_c : mine_c, k = by_query ? mine_c : other_c;
      const bool m = tmask[static_cast<int64_t>(q) * max_k + k] != 0;
      any |= m && other < others;
      all &= m || other >= others;
    }
    any = any && valid;
    const bool none_live = __builtin_amdgcn_ballot_w64(valid && !all) == 0;
    const bool some_masked = __builtin_amdgcn_ballot_w64(valid && any) != 0;
    const int cls = none_live ? 2 : some_masked ? 1 : 0;
    if (lane == 0) out[t] = cls;
    if (cls != 2) { lo = min(lo, t); hi = max(hi, t + 1); }
  }
  if (lane == 0) { first[wave] = lo; last[wave] = hi; }
  __syncthreads();
  if (tid == 0) {
    const int f = min(min(first[0], first[1]), min(first[2], first[3])), l = max(max(last[0], last[1]), max(last[2], last[3]));
    if (by_query) out[-1] = l;
    else { out[-2] = f; out[-1] = l; }
  }
}

// Key padding mask [B, max_k] -> key_info [B, 1 + ceil(max_k / 64)]: word 0 = 1 + the index of the last live key (0 when
// every key is masked), word 1 + t = whether tile t has a masked key below that. One block per sequence.
__global__ __launch_bounds__(256) void flash_key_info_kernel(const uint8_t* pad, int max_k, int32_t* kinfo, int pitch,
                                                             uint32_t* pad_bits) {
  __shared__ int part[4];
  const int b = blockIdx.x, tid = static_cast<int>(threadIdx.x);
  const uint8_t* row = pad + static_cast<int64_t>(b) * max_k;
  int last = 0;
  for (int j = tid; j < max_k; j += 256)
    if (row[j] == 0) last = j + 1;
  for (int off = 32; off > 0; off >>= 1) last = max(last, __shfl_xor(last, off, 64));
  if ((tid & 63) == 0) part[tid >> 6] = last;
  __syncthreads();
  const int lk = max(max(part[0], part[1]), max(part[2], part[3]));
  int32_t* out = kinfo + static_cast<int64_t>(b) * pitch;
  if (tid == 0) out[0] = lk;
  // one wavefront per tile: a key per lane
  for (int t = tid >> 6; t < pitch - 1; t += 4) {
    const int key = FA_TILE * t + (tid & 63);
    const bool masked = key < lk && row[key] != 0;
    const uint64_t keys = __builtin_amdgcn_ballot_w64(masked);
    if ((tid & 63) == 0) out[1 + t] = keys != 0 ? 1 : 0;
    // the mask below the last live key, packed: the tile's two words [tile][half]
    if ((tid & 63) < 2) pad_bits[(static_cast<int64_t>(b) * (pitch - 1) + t) * 2 + (tid & 63)] = tile_word_of(keys, tid & 63);
  }
}

// Keep bits from the generator: one thread per (head of a sequence, group of 32 queries, group of four keys) runs the
// eight generator calls of its 32 x 4 elements (one call per 4 x 4 patch) and writes the four keys' words.
__global__ __launch_bounds__(256) void flash_bits_rng_kernel(FaArgs a, int64_t total) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const int k4n = a.kp / 4;
  const int j4 = static_cast<int>(id % k4n);
  const int64_t row = id / k4n;                      // (b H + h) q32 + group
  const int grp = static_cast<int>(row % a.q32);
  const int bh = static_cast<int>(row / a.q32), b = bh / a.heads;
  const SeqSpan sp = seq_span(a, b);
  const int lq = sp.lq, lk = sp.lk;
  if (32 * grp >= lq || 4 * j4 >= lk) return;        // never read: every element there is masked or not stored
  const Philox gen(a.seed);
  const uint64_t q4 = static_cast<uint64_t>((a.max_q + 3) / 4), k4 = static_cast<uint64_t>((a.max_k + 3) / 4);
  uint32_t word[4] = {0, 0, 0, 0};
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const uint4 r = gen((static_cast<uint64_t>(bh) * q4 + static_cast<uint64_t>(8 * grp + u)) * k4 + static_cast<uint64_t>(j4), a.offset);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int qi = 0; qi < 4; ++qi)
#pragma unroll
      for (int kj = 0; kj < 4; ++kj)
        word[kj] |= (((w[qi] >> (8 * kj)) & 0xffu) < a.thr ? 1u : 0u) << (4 * u + qi);
  }
  uint32_t* out = a.bits + row * a.kp;
#pragma unroll
  for (int kj = 0; kj < 4; ++kj) out[bit_slot(4 * j4 + kj)] = word[kj];
  if (a.mask_out != nullptr) {
#pragma unroll
    for (int kj = 0; kj < 4; ++kj) {
      const int key = 4 * j4 + kj;
      if (key < lk)
        for (int i = 0; i < 32; ++i) {
          const int qi = 32 * grp + i;
          if (qi < lq) a.mask_out[(static_cast<int64_t>(bh) * a.max_q + qi) * a.max_k + key] = (word[kj] >> i) & 1u;
        }
    }
  }
}

// Keep bits from an explicit byte mask [B, H, max_q, max_k]: one thread per (head of a sequence, group of 32 queries, key).
__global__ __launch_bounds__(256) void flash_bits_mask_kernel(FaArgs a, int64_t total) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const int key = static_cast<int>(id % a.kp);
  const int64_t row = id / a.kp;
  const int grp = static_cast<int>(row % a.q32);
  const int bh = static_cast<int>(row / a.q32), b = bh / a.heads;
  const SeqSpan sp = seq_span(a, b);
  const int lq = sp.lq, lk = sp.lk;
  if (32 * grp >= lq || key >= lk) return;
  uint32_t word = 0;
  for (int i = 0; i < 32; ++i) {
    const int qi = 32 * grp + i;
    if (qi < lq && a.mask[(static_cast<int64_t>(bh) * a.max_q + qi) * a.max_k + key] != 0) word |= 1u << i;
  }
  a.bits[row * a.kp + bit_slot(key)] = word;
}

// The same for four keys per thread, read as one word per query (max_k a multiple of 4, mask 4-byte aligned).
__global__ __launch_bounds__(256) void flash_bits_mask4_kernel(FaArgs a, int64_t total) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const int k4n = a.kp / 4;
  const int key0 = 4 * static_cast<int>(id % k4n);
  const int64_t row = id / k4n;
  const int grp = static_cast<int>(row % a.q32);
  const int bh = static_cast<int>(row / a.q32), b = bh / a.heads;
  const SeqSpan sp = seq_span(a, b);
  if (32 * grp >= sp.lq || key0 >= sp.lk) return;     // key0 < lk <= max_k and max_k is a multiple of 4: key0 + 3 < max_k
  const uint8_t* src = a.mask + (static_cast<int64_t>(bh) * a.max_q + 32 * grp) * a.max_k + key0;
  const int nq = min(32, sp.lq - 32 * grp);
  uint32_t word[4] = {0, 0, 0, 0};
#pragma unroll 8
  for (int i = 0; i < nq; ++i) {
    const uint32_t m = *reinterpret_cast<const uint32_t*>(src + static_cast<int64_t>(i) * a.max_k);
#pragma unroll
    for (int kj = 0; kj < 4; ++kj) word[kj] |= (((m >> (8 * kj)) & 0xffu) != 0 ? 1u : 0u) << i;
  }
  uint32_t* out = a.bits + row * a.kp;
#pragma unroll
  for (int kj = 0; kj < 4; ++kj) out[bit_slot(key0 + kj)] = word[kj];
}

// The 32 lane masks of one 64-key tile for the wavefront's group of 32 queries: mask e belongs to accumulator register
// e % 16 of accumulator e / 16 (keys 32 (e / 16) + 8 ((e % 16) / 4) + e % 4 in lanes 0..31 and that + 4 in lanes 32..63).
__device__ __forceinline__ const uint64_t* tile_lane_masks(const FaArgs& a, int bh, int group, int tile) {
  return reinterpret_cast<const uint64_t*>(a.bits + (static_cast<int64_t>(bh) * a.q32 + group) * a.kp + FA_TILE * tile);
}

// Writes the wavefront's 32 rows x D accumulators (acc[i][r]: column 32 i + 8 (r / 4) + 4 half + r % 4 of row lane & 31)
// through its own LDS patch as whole 16-byte chunks, rows past `len` skipped.
template <typename T, int D>
__device__ __forceinline__ void store_rows_out(const acc16_t (&acc)[D / 32], float mul, uint8_t* patch, T* base, int64_t stride,
                                               int row0, int len, int lane) {
  const int half = lane >> 5, row = lane & 31;
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int col = 32 * i + 8 * g + 4 * half;
      uint2 w;
      w.x = pack2<T>(acc[i][4 * g + 0] * mul, acc[i][4 * g + 1] * mul);
      w.y = pack2<T>(acc[i][4 * g + 2] * mul, acc[i][4 * g + 3] * mul);
      *reinterpret_cast<uint2*>(patch + row_image_at<D>(row, col / 8) + (col % 8) * 2) = w;
    }
  __syncthreads();
  constexpr int CH = D / 8;
#pragma unroll
  for (int i = 0; i < 32 * CH / 64; ++i) {
    const int id = lane + 64 * i;
    const int r = id / CH, c = id % CH;
    if (row0 + r < len)
      *reinterpret_cast<uint4*>(base + static_cast<int64_t>(row0 + r) * stride + 8 * c) =
          *reinterpret_cast<const uint4*>(patch + row_image_at<D>(r, c));
  }
}

// -------------------------------------------------------------------------------------------------------------------
// forward
// -------------------------------------------------------------------------------------------------------------------
// PAD: the call has a key padding mask (batch-strided calls only); without it no mask code is compiled in.
template <typename T, int D, int DROP, int PAD>
__global__ __launch_bounds__(FA_THREADS, D == 64 ? 3 : 1) void flash_fwd_kernel(FaArgs a) {
  extern __shared__ __align__(16) uint8_t lds_raw[];
  constexpr int IMG = FA_TILE * D * 2;
  const int b = blockIdx.z, h = blockIdx.y, q0 = static_cast<int>(blockIdx.x) * FA_ROWS;
  const SeqSpan sp = seq_span(a, b);
  const int qs = sp.qs, lq = sp.lq, ks = sp.ks, lk = sp.lk;
  if (q0 >= lq) return;
  const int lane = static_cast<int>(threadIdx.x) & 63, wave = static_cast<int>(threadIdx.x) >> 6, half = lane >> 5;
  const int bh = b * a.heads + h;
  const int qrow = q0 + 32 * wave + (lane & 31);
  const T* qb = static_cast<const T*>(a.q) + static_cast<int64_t>(qs) * a.q_st + static_cast<int64_t>(b) * a.q_sb + static_cast<int64_t>(h) * a.q_sh;
  const T* kb = static_cast<const T*>(a.k) + static_cast<int64_t>(ks) * a.k_st + static_cast<int64_t>(b) * a.k_sb + static_cast<int64_t>(h) * a.k_sh;
  const T* vb = static_cast<const T*>(a.v) + static_cast<int64_t>(ks) * a.v_st + static_cast<int64_t>(b) * a.v_sb + static_cast<int64_t>(h) * a.v_sh;
  uint4 qf[D / 16];
  load_resident<T, D>(qf, qb, a.q_st, qrow, lq, lane);

  const int nkeys = a.causal ? min(lk, q0 + FA_ROWS) : lk;
  int ntiles = (nkeys + FA_TILE - 1) / FA_TILE;
  if constexpr (PAD == 2) ntiles = min(ntiles, tile_bound(a, static_cast<int>(blockIdx.x)));
  const int group = static_cast<int>(blockIdx.x) * (FA_ROWS / 32) + __builtin_amdgcn_readfirstlane(wave);   // of 32 queries

  acc16_t o[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  float m = FA_NEG, l = 0.f;
  const float dead_raw = FA_NEG / a.scale_log2;   // the raw score that the scale turns into -1e30
  [[maybe_unused]] const int qr = min(qrow, lq - 1);   // the row whose time-mask words this lane reads

  // The packed mask word of a tile is asked for one tile ahead, behind that tile's keys and values, and is there when the
  // wait for those ends the iteration; asked for at its own tile it would be waited for together with the next tile's loads.
  [[maybe_unused]] uint32_t mdead_next = 0;
  if constexpr (PAD != 0) {
    if (ntiles > 0) mdead_next = tile_mask_bits<PAD>(a, b, qr, 0, half);
  }
  Staged<D> sk, sv;
  // (not under `ntiles > 0`: rows past the end load nothing and store zeros, and a wait that lies on every path into
  // the loop lets the compiler know there that the resident rows above have landed; behind a branch it would repeat
  // their wait inside the loop, after the next tile's loads, and every tile would wait for its own prefetch)
  sk.load(kb, a.k_st, 0, lk);
  sv.load(vb, a.v_st, 0, lk);
  sk.store_rows(lds_raw);
  sv.store_transposed(lds_raw + IMG);
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const uint8_t* kimg = lds_raw + (t & 1) * 2 * IMG;
    const uint8_t* vimg = kimg + IMG;
    [[maybe_unused]] const uint32_t mdead = mdead_next;
    if (t + 1 < ntiles) {
      sk.load(kb, a.k_st, (t + 1) * FA_TILE, lk);
      sv.load(vb, a.v_st, (t + 1) * FA_TILE, lk);
      if constexpr (PAD != 0) mdead_next = tile_mask_bits<PAD>(a, b, qr, t + 1, half);
    }
    acc16_t s[2];
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[n][r] = 0.f;
#pragma unroll
    for (int ss = 0; ss < D / 16; ++ss)
#pragma unroll
      for (int n = 0; n < 2; ++n) mfma<T>::run(read_rows<D>(kimg, n, ss, lane), qf[ss], s[n]);
    // Masking only where the tile crosses the end of the keys or the causal diagonal (the same for the whole wavefront).
    // A masked raw score is the value that the scale turns into -1e30 or beyond: its probability is exp2 of that, 0.
    // bit 16 n + r of mdead: the mask hides key (n, r) of the tile from this lane's query. One word, packed by the mask's
    // summary kernel (as byte loads, 32 per tile, the compiler waited for each in turn).
    bool padt = false;
    if constexpr (PAD != 0) {
      // With the causal flag on top of a mask, a row whose keys up to the diagonal are all masked meets the diagonal's
      // dead keys in tiles without a masked key and still has the initial m there: every tile takes the masked-tile route
      // then (the combination is rare; the reference's decoder passes its causal mask as a time mask).
      padt = masked_tile<PAD>(a, b, min(group, (a.max_q + 31) / 32 - 1), t) || a.causal != 0;
    }
    const bool edge = (t + 1) * FA_TILE > lk || (a.causal && t * FA_TILE + FA_TILE - 1 > q0 + 32 * wave) || padt;
    if (edge) {
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = t * FA_TILE + 32 * n + 8 * (r / 4) + 4 * half + r % 4;
          bool dead = key >= lk || (a.causal && key > qrow);
          if constexpr (PAD != 0) dead = dead || ((mdead >> (16 * n + r)) & 1u) != 0;
          if (dead) s[n][r] = dead_raw;
        }
    }
    // tile maximum of the scaled scores from the extreme raw score (one multiplication instead of 32)
    float ext = s[0][0];
    if (a.scale_log2 >= 0.f) {
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) ext = fmaxf(ext, s[n][r]);
    } else {
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) ext = fminf(ext, s[n][r]);
    }
    const float mx = pair_max(ext * a.scale_log2);
    // The reference point m follows the running maximum lazily: it moves (and the accumulators are rescaled) only when a
    // row's maximum has grown by more than 2^8, so probabilities relative to m stay below 256, inside every type here,
    // and most tiles skip the rescaling. out = O / l does not depend on m. Every row sees a live key in its first tile
    // (key 0), so m leaves its initial value there.
    const bool grow = mx > m + FA_LAZY;
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
      const float m_new = grow ? mx : m;
      const float alpha = fast_exp2(m - m_new);
      m = m_new;
      l *= alpha;
#pragma unroll
      for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
    }
    float lsum = 0.f;
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pr = fast_exp2(__builtin_fmaf(s[n][r], a.scale_log2, -m));
        s[n][r] = pr;
        lsum += pr;
      }
    if constexpr (PAD != 0) if (padt) {
      // A row that has met no live key yet still has the initial m, against which a dead score is not small: such
      // probabilities are set to 0 by hand. (Without masked keys inside the sequence, key 0 is live for every row. Under
      // the causal flag every tile counts as one with masked keys, see padt above.)
      lsum = 0.f;
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = t * FA_TILE + 32 * n + 8 * (r / 4) + 4 * half + r % 4;
          if (key >= lk || (a.causal && key > qrow) || ((mdead >> (16 * n + r)) & 1u) != 0) s[n][r] = 0.f;
          lsum += s[n][r];
        }
    }
    l += lsum;
    if constexpr (DROP != 0) {
      const uint64_t* lane_mask = tile_lane_masks(a, bh, group, t);
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          s[n][r] = __builtin_amdgcn_inverse_ballot_w64(lane_mask[16 * n + r]) ? s[n][r] : 0.f;   // the scale waits for the end
    }
#pragma unroll
    for (int kk = 0; kk < FA_TILE / 16; ++kk) {
      float pv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) pv[e] = s[kk / 2][8 * (kk % 2) + e];
      const uint4 pf = acc_to_operand<T>(pv);
#pragma unroll
      for (int i = 0; i < D / 32; ++i) mfma<T>::run(read_transposed<D>(vimg, i, kk, lane), pf, o[i]);
    }
    if (t + 1 < ntiles) {
      uint8_t* nk = lds_raw + ((t + 1) & 1) * 2 * IMG;
      sk.store_rows(nk);
      sv.store_transposed(nk + IMG);
    }
    __syncthreads();
  }
  l = pair_sum(l);
  const float inv = l > 0.f ? a.drop_scale / l : 0.f;
  if (half == 0 && qrow < lq)
    a.lse[static_cast<int64_t>(bh) * a.max_q + qrow] = l > 0.f ? (m + log2f(l)) * (1.0f / FA_LOG2E) : -INFINITY;
  T* ob = static_cast<T*>(a.out) + static_cast<int64_t>(qs) * a.o_st + static_cast<int64_t>(b) * a.o_sb + static_cast<int64_t>(h) * a.o_sh;
  store_rows_out<T, D>(o, inv, lds_raw + wave * (32 * D * 2), ob, a.o_st, q0 + 32 * wave, lq, lane);
}

// -------------------------------------------------------------------------------------------------------------------
// backward, dQ and D = rowsum(dO * O)
// -------------------------------------------------------------------------------------------------------------------
template <typename T, int D, int DROP, int PAD>
__global__ __launch_bounds__(FA_THREADS, D == 64 ? 2 : 1) void flash_bwd_dq_kernel(FaArgs a) {
  extern __shared__ __align__(16) uint8_t lds_raw[];
  constexpr int IMG = FA_TILE * D * 2;
  const int b = blockIdx.z, h = blockIdx.y, q0 = static_cast<int>(blockIdx.x) * FA_ROWS;
  const SeqSpan sp = seq_span(a, b);
  const int qs = sp.qs, lq = sp.lq, ks = sp.ks, lk = sp.lk;
  if (q0 >= lq) return;
  const int lane = static_cast<int>(threadIdx.x) & 63, wave = static_cast<int>(threadIdx.x) >> 6, half = lane >> 5;
  const int bh = b * a.heads + h;
  const int qrow = q0 + 32 * wave + (lane & 31);
  const T* qb = static_cast<const T*>(a.q) + static_cast<int64_t>(qs) * a.q_st + static_cast<int64_t>(b) * a.q_sb + static_cast<int64_t>(h) * a.q_sh;
  const T* kb = static_cast<const T*>(a.k) + static_cast<int64_t>(ks) * a.k_st + static_cast<int64_t>(b) * a.k_sb + static_cast<int64_t>(h) * a.k_sh;
  const T* vb = static_cast<const T*>(a.v) + static_cast<int64_t>(ks) * a.v_st + static_cast<int64_t>(b) * a.v_sb + static_cast<int64_t>(h) * a.v_sh;
  const T* ob = static_cast<const T*>(a.o) + static_cast<int64_t>(qs) * a.o_st + static_cast<int64_t>(b) * a.o_sb + static_cast<int64_t>(h) * a.o_sh;
  const T* gb = static_cast<const T*>(a.d_o) + static_cast<int64_t>(qs) * a.do_st + static_cast<int64_t>(b) * a.do_sb + static_cast<int64_t>(h) * a.do_sh;
  uint4 qf[D / 16], gf[D / 16];
  load_resident<T, D>(qf, qb, a.q_st, qrow, lq, lane);
  load_resident<T, D>(gf, gb, a.do_st, qrow, lq, lane);
  float delta = 0.f;
  {
    uint4 of[D / 16];
    load_resident<T, D>(of, ob, a.o_st, qrow, lq, lane);
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      const T* x = reinterpret_cast<const T*>(&of[s]);
      const T* y = reinterpret_cast<const T*>(&gf[s]);
#pragma unroll
      for (int e = 0; e < 8; ++e) delta += elem<T>::to_float(x[e]) * elem<T>::to_float(y[e]);
    }
    delta = pair_sum(delta);
  }
  const int64_t stat = static_cast<int64_t>(bh) * a.max_q + qrow;
  float lse2 = -FA_NEG;   // rows past the sequence: probability 0
  if (qrow < lq) {
    const float v = a.lse[stat];
    lse2 = v == -INFINITY ? -FA_NEG : v * FA_LOG2E;
    if (half == 0) a.delta[stat] = delta;
  }

  const int nkeys = a.causal ? min(lk, q0 + FA_ROWS) : lk;
  int ntiles = (nkeys + FA_TILE - 1) / FA_TILE;
  if constexpr (PAD == 2) ntiles = min(ntiles, tile_bound(a, static_cast<int>(blockIdx.x)));
  const int group = static_cast<int>(blockIdx.x) * (FA_ROWS / 32) + __builtin_amdgcn_readfirstlane(wave);   // of 32 queries
  const float dead_raw = FA_NEG / a.scale_log2;   // the raw score that the scale turns into -1e30
  [[maybe_unused]] const int qr = min(qrow, lq - 1);   // the row whose time-mask words this lane reads
  acc16_t dq[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[i][r] = 0.f;

  [[maybe_unused]] uint32_t mdead_next = 0;      // the packed mask word, one tile ahead, as in the forward kernel
  if constexpr (PAD != 0) {
    if (ntiles > 0) mdead_next = tile_mask_bits<PAD>(a, b, qr, 0, half);
  }
  // per buffer: K row image, K transposed image, V row image
  Staged<D> sk, sv;
  sk.load(kb, a.k_st, 0, lk);          // on every path, as in the forward kernel
  sv.load(vb, a.v_st, 0, lk);
  sk.store_rows(lds_raw);
  sk.store_transposed(lds_raw + IMG);
  sv.store_rows(lds_raw + 2 * IMG);
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const uint8_t* kimg = lds_raw + (t & 1) * 3 * IMG;
    const uint8_t* ktimg = kimg + IMG;
    const uint8_t* vimg = kimg + 2 * IMG;
    [[maybe_unused]] const uint32_t mdead = mdead_next;
    if (t + 1 < ntiles) {
      sk.load(kb, a.k_st, (t + 1) * FA_TILE, lk);
      sv.load(vb, a.v_st, (t + 1) * FA_TILE, lk);
      if constexpr (PAD != 0) mdead_next = tile_mask_bits<PAD>(a, b, qr, t + 1, half);
    }
    // the lane masks of the tile's first 32 keys: asked for ahead of the products, which cover the scalar cache's latency
    [[maybe_unused]] uint64_t first_masks[16];
    if constexpr (DROP != 0) {
      const uint64_t* lm = tile_lane_masks(a, bh, group, t);
#pragma unroll
      for (int r = 0; r < 16; ++r) first_masks[r] = lm[r];
    }
    acc16_t s[2], dp[2];
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[n][r] = 0.f; dp[n][r] = 0.f; }
#pragma unroll
    for (int ss = 0; ss < D / 16; ++ss)
#pragma unroll
      for (int n = 0; n < 2; ++n) {
        mfma<T>::run(read_rows<D>(kimg, n, ss, lane), qf[ss], s[n]);
        mfma<T>::run(read_rows<D>(vimg, n, ss, lane), gf[ss], dp[n]);
      }
    // masking as in the forward: only where the tile crosses the end of the keys or the causal diagonal
    // bit 16 n + r of mdead: the mask hides key (n, r) of the tile from this lane's query. One word, packed by the mask's
    // summary kernel (as byte loads, 32 per tile, the compiler waited for each in turn).
    bool padt = false;
    if constexpr (PAD != 0) padt = masked_tile<PAD>(a, b, min(group, (a.max_q + 31) / 32 - 1), t);
    if ((t + 1) * FA_TILE > lk || (a.causal && t * FA_TILE + FA_TILE - 1 > q0 + 32 * wave) || padt) {
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = t * FA_TILE + 32 * n + 8 * (r / 4) + 4 * half + r % 4;
          bool dead = key >= lk || (a.causal && key > qrow);
          if constexpr (PAD != 0) dead = dead || ((mdead >> (16 * n + r)) & 1u) != 0;
          if (dead) s[n][r] = dead_raw;
        }
    }
    [[maybe_unused]] const uint64_t* lane_mask = DROP != 0 ? tile_lane_masks(a, bh, group, t) : nullptr;
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pr = fast_exp2(__builtin_fmaf(s[n][r], a.scale_log2, -lse2));
        float kscale = 1.f;
        if constexpr (DROP != 0)
          kscale = __builtin_amdgcn_inverse_ballot_w64(n == 0 ? first_masks[r] : lane_mask[16 + r]) ? a.drop_scale : 0.f;
        s[n][r] = pr * __builtin_fmaf(dp[n][r], kscale, -delta);     // dS
      }
#pragma unroll
    for (int kk = 0; kk < FA_TILE / 16; ++kk) {
      float dsv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) dsv[e] = s[kk / 2][8 * (kk % 2) + e];
      const uint4 df = acc_to_operand<T>(dsv);
#pragma unroll
      for (int i = 0; i < D / 32; ++i) mfma<T>::run(read_transposed<D>(ktimg, i, kk, lane), df, dq[i]);
    }
    if (t + 1 < ntiles) {
      uint8_t* nk = lds_raw + ((t + 1) & 1) * 3 * IMG;
      sk.store_rows(nk);
      sk.store_transposed(nk + IMG);
      sv.store_rows(nk + 2 * IMG);
    }
    __syncthreads();
  }
  T* dqb = static_cast<T*>(a.dq) + static_cast<int64_t>(qs) * a.dq_st + static_cast<int64_t>(b) * a.dq_sb + static_cast<int64_t>(h) * a.dq_sh;
  store_rows_out<T, D>(dq, a.scale, lds_raw + wave * (32 * D * 2), dqb, a.dq_st, q0 + 32 * wave, lq, lane);
}

// -------------------------------------------------------------------------------------------------------------------
// backward, dK and dV: one key per lane pair, query tiles of 64 streamed through LDS
// -------------------------------------------------------------------------------------------------------------------
// TM: the call has a time mask; without it none of that code is compiled in.
template <typename T, int D, int DROP, int TM>
__global__ __launch_bounds__(FA_THREADS, D == 64 ? 2 : 1) void flash_bwd_dkv_kernel(FaArgs a) {
  extern __shared__ __align__(16) uint8_t lds_raw[];
  constexpr int IMG = FA_TILE * D * 2;
  constexpr int BUF = 4 * IMG + 2 * FA_TILE * 4;   // Q rows, Q transposed, dO rows, dO transposed, lse2[64], delta[64]
  const int b = blockIdx.z, h = blockIdx.y, k0 = static_cast<int>(blockIdx.x) * FA_ROWS;
  const SeqSpan sp = seq_span(a, b);
  const int qs = sp.qs, lq = sp.lq, ks = sp.ks, lk = sp.lk;
  // Packed calls write the rows of the sequence's keys; batch-strided calls write all max_k rows (zeros past the last
  // live key: the gradient of the projection reads every row).
  const int lk_out = a.cu_q != nullptr ? lk : a.max_k;
  if (k0 >= lk) {
    if (k0 < lk_out) {
      T* dkz = static_cast<T*>(a.dk) + static_cast<int64_t>(b) * a.dk_sb + static_cast<int64_t>(h) * a.dk_sh;
      T* dvz = static_cast<T*>(a.dv) + static_cast<int64_t>(b) * a.dv_sb + static_cast<int64_t>(h) * a.dv_sh;
      constexpr int CH = D / 8;
      for (int id = static_cast<int>(threadIdx.x); id < FA_ROWS * CH; id += FA_THREADS) {
        const int row = k0 + id / CH, c = id % CH;
        if (row < lk_out) {
          *reinterpret_cast<uint4*>(dkz + static_cast<int64_t>(row) * a.dk_st + 8 * c) = make_uint4(0, 0, 0, 0);
          *reinterpret_cast<uint4*>(dvz + static_cast<int64_t>(row) * a.dv_st + 8 * c) = make_uint4(0, 0, 0, 0);
        }
      }
    }
    return;
  }
  const int lane = static_cast<int>(threadIdx.x) & 63, wave = static_cast<int>(threadIdx.x) >> 6, half = lane >> 5;
  const int bh = b * a.heads + h;
  const int krow = k0 + 32 * wave + (lane & 31);
  // this lane's key is masked (past the end, or padded), and whether any key of the wavefront is
  const bool kdead = krow >= lk || (a.pad != nullptr && a.pad[static_cast<int64_t>(b) * a.max_k + krow] != 0);
  const bool wave_dead = __builtin_amdgcn_ballot_w64(kdead) != 0;
  const T* qb = static_cast<const T*>(a.q) + static_cast<int64_t>(qs) * a.q_st + static_cast<int64_t>(b) * a.q_sb + static_cast<int64_t>(h) * a.q_sh;
  const T* kb = static_cast<const T*>(a.k) + static_cast<int64_t>(ks) * a.k_st + static_cast<int64_t>(b) * a.k_sb + static_cast<int64_t>(h) * a.k_sh;
  const T* vb = static_cast<const T*>(a.v) + static_cast<int64_t>(ks) * a.v_st + static_cast<int64_t>(b) * a.v_sb + static_cast<int64_t>(h) * a.v_sh;
  const T* gb = static_cast<const T*>(a.d_o) + static_cast<int64_t>(qs) * a.do_st + static_cast<int64_t>(b) * a.do_sb + static_cast<int64_t>(h) * a.do_sh;
  uint4 kf[D / 16], vf[D / 16];
  load_resident<T, D>(kf, kb, a.k_st, krow, lk, lane);
  load_resident<T, D>(vf, vb, a.v_st, krow, lk, lane);

  // causal: queries before the block's first key see none of its keys
  int t0 = a.causal ? k0 / FA_TILE : 0;
  int ntiles = (lq + FA_TILE - 1) / FA_TILE;
  // time mask: the block's four groups of 32 keys know the first and the last query tile with a live element
  const int kgroups = (a.max_k + 31) / 32;
  const int kgroup = min(static_cast<int>(blockIdx.x) * (FA_ROWS / 32) + __builtin_amdgcn_readfirstlane(wave), kgroups - 1);
  if constexpr (TM != 0) {
    int lo = ntiles, hi = 0;
    for (int i = 0; i < FA_ROWS / 32; ++i) {
      const int32_t* row = a.kqinfo + static_cast<int64_t>(min(static_cast<int>(blockIdx.x) * (FA_ROWS / 32) + i, kgroups - 1)) * a.kqinfo_pitch;
      lo = min(lo, row[0]);
      hi = max(hi, row[1]);
    }
    t0 = max(t0, lo);
    ntiles = min(ntiles, hi);
  }
  const int krow_c = min(krow, a.max_k - 1);   // the column whose time-mask words this lane reads
  const float dead_raw = FA_NEG / a.scale_log2;   // the raw score that the scale turns into -1e30
  acc16_t dk[D / 32], dv[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dk[i][r] = 0.f; dv[i][r] = 0.f; }

  Staged<D> sq, sg;
  // threads 0..63: the log-sum-exp of the tile's query (-inf past the end), 64..127: its D. As loaded: the value is only
  // looked at when the tile is stored (a comparison or a product right behind the load would be a wait right behind the
  // tile loads issued before it, every tile).
  float st_raw = 0.f;
  auto load_stats = [&](int t) {
    const int tid = static_cast<int>(threadIdx.x);
    if (tid < 2 * FA_TILE) {
      const int qi = t * FA_TILE + (tid & (FA_TILE - 1));
      const float* src = tid < FA_TILE ? a.lse : a.delta;
      st_raw = tid < FA_TILE ? -INFINITY : 0.f;
      if (qi < lq) st_raw = src[static_cast<int64_t>(bh) * a.max_q + qi];
    }
  };
  auto store_tile = [&](uint8_t* buf) {
    sq.store_rows(buf);
    sq.store_transposed(buf + IMG);
    sg.store_rows(buf + 2 * IMG);
    sg.store_transposed(buf + 3 * IMG);
    if (threadIdx.x < 2 * FA_TILE) {
      // lse in units of log2; a row without a live key (or past the end) gets the large positive value that turns its
      // probabilities into zeros
      const float lse2 = st_raw == -INFINITY ? -FA_NEG : st_raw * FA_LOG2E;
      reinterpret_cast<float*>(buf + 4 * IMG)[threadIdx.x] = threadIdx.x < FA_TILE ? lse2 : st_raw;
    }
  };
  // keep bits of this lane's key for a tile's two groups of 32 queries, requested one tile ahead like the tile itself
  [[maybe_unused]] uint32_t kraw_next[2] = {0, 0};
  auto load_keep_bits = [&](int t) {
    if constexpr (DROP != 0) {
      if (krow < lk) {
        const uint32_t* w = a.bits + (static_cast<int64_t>(bh) * a.q32 + 2 * t) * a.kp + bit_slot(krow);
        kraw_next[0] = w[0];
        kraw_next[1] = w[a.kp];
      }
    }
  };
  uint32_t tdead_next = 0;                        // the packed time-mask word, one tile ahead, as in the forward kernel
  if (TM != 0 && t0 < ntiles) tdead_next = a.tk_bits[(static_cast<int64_t>(krow_c) * a.query_tiles + t0) * 2 + half];
  sq.load(qb, a.q_st, t0 * FA_TILE, lq);          // on every path, as in the forward kernel
  sg.load(gb, a.do_st, t0 * FA_TILE, lq);
  load_stats(t0);
  if (t0 < ntiles) load_keep_bits(t0);
  store_tile(lds_raw + (t0 & 1) * BUF);
  __syncthreads();
  for (int t = t0; t < ntiles; ++t) {
    const uint8_t* qimg = lds_raw + (t & 1) * BUF;
    const uint8_t* qtimg = qimg + IMG;
    const uint8_t* gimg = qimg + 2 * IMG;
    const uint8_t* gtimg = qimg + 3 * IMG;
    const float* stats = reinterpret_cast<const float*>(qimg + 4 * IMG);
    const uint32_t tdead = tdead_next;
    [[maybe_unused]] const uint32_t kraw[2] = {kraw_next[0], kraw_next[1]};
    if (t + 1 < ntiles) {
      sq.load(qb, a.q_st, (t + 1) * FA_TILE, lq);
      sg.load(gb, a.do_st, (t + 1) * FA_TILE, lq);
      load_stats(t + 1);
      load_keep_bits(t + 1);
      if (TM != 0) tdead_next = a.tk_bits[(static_cast<int64_t>(krow_c) * a.query_tiles + t + 1) * 2 + half];
    }
    acc16_t s[2], dp[2];
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[n][r] = 0.f; dp[n][r] = 0.f; }
#pragma unroll
    for (int ss = 0; ss < D / 16; ++ss)
#pragma unroll
      for (int n = 0; n < 2; ++n) {
        mfma<T>::run(read_rows<D>(qimg, n, ss, lane), kf[ss], s[n]);
        mfma<T>::run(read_rows<D>(gimg, n, ss, lane), vf[ss], dp[n]);
      }
    // s[n][r]: query 32 n + 8 (r / 4) + 4 half + r % 4 of the tile, key krow. P (dropped, scaled) stays in dp's place
    // for dV, dS goes to s for dK.
    // time mask: bit 16 n + r of tdead = the mask hides query (n, r) of the tile from this lane's key; one word, packed
    // by the mask's summary kernel.
    bool tmt = false;
    if constexpr (TM != 0) tmt = a.kqinfo[static_cast<int64_t>(kgroup) * a.kqinfo_pitch + 2 + t] != 0;
    if (wave_dead || (a.causal && t * FA_TILE < k0 + 32 * wave + 31) || tmt) {
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int qi = t * FA_TILE + 32 * n + 8 * (r / 4) + 4 * half + r % 4;
          if (kdead || (a.causal && krow > qi) || ((tdead >> (16 * n + r)) & 1u) != 0) s[n][r] = dead_raw;
        }
    }
    // keep bits of this lane's key for the tile's two groups of 32 queries, shifted so that bit 8 g + c is register 4 g + c
    uint32_t kbits[2] = {0, 0};
    if constexpr (DROP != 0) {
      kbits[0] = kraw[0] >> (4 * half);
      kbits[1] = kraw[1] >> (4 * half);
    }
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int ql = 32 * n + 8 * g + 4 * half;          // first of four consecutive queries, within the tile
        const float4 l4 = *reinterpret_cast<const float4*>(stats + ql);
        const float4 d4 = *reinterpret_cast<const float4*>(stats + FA_TILE + ql);
        const float lse2[4] = {l4.x, l4.y, l4.z, l4.w}, dl[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * g + e;
          const float pr = fast_exp2(__builtin_fmaf(s[n][r], a.scale_log2, -lse2[e]));
          const bool keep = DROP == 0 || ((kbits[n] >> (8 * g + e)) & 1u) != 0;
          const float kscale = DROP != 0 ? (keep ? a.drop_scale : 0.f) : 1.f;
          s[n][r] = pr * __builtin_fmaf(dp[n][r], kscale, -dl[e]);   // dS
          dp[n][r] = keep ? pr : 0.f;                                // kept probabilities; their scale waits for the end
        }
      }
#pragma unroll
    for (int kk = 0; kk < FA_TILE / 16; ++kk) {
      float pv[8], dsv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) { pv[e] = dp[kk / 2][8 * (kk % 2) + e]; dsv[e] = s[kk / 2][8 * (kk % 2) + e]; }
      const uint4 pf = acc_to_operand<T>(pv), df = acc_to_operand<T>(dsv);
#pragma unroll
      for (int i = 0; i < D / 32; ++i) {
        mfma<T>::run(read_transposed<D>(gtimg, i, kk, lane), pf, dv[i]);
        mfma<T>::run(read_transposed<D>(qtimg, i, kk, lane), df, dk[i]);
      }
    }
    if (t + 1 < ntiles) store_tile(lds_raw + ((t + 1) & 1) * BUF);
    __syncthreads();
  }
  T* dkb = static_cast<T*>(a.dk) + static_cast<int64_t>(ks) * a.dk_st + static_cast<int64_t>(b) * a.dk_sb + static_cast<int64_t>(h) * a.dk_sh;
  T* dvb = static_cast<T*>(a.dv) + static_cast<int64_t>(ks) * a.dv_st + static_cast<int64_t>(b) * a.dv_sb + static_cast<int64_t>(h) * a.dv_sh;
  uint8_t* patch = lds_raw + wave * (32 * D * 2);
  store_rows_out<T, D>(dk, a.scale, patch, dkb, a.dk_st, k0 + 32 * wave, lk_out, lane);
  __syncthreads();
  store_rows_out<T, D>(dv, a.drop_scale, patch, dvb, a.dv_st, k0 + 32 * wave, lk_out, lane);
}

// -------------------------------------------------------------------------------------------------------------------
// inference: probabilities and context in one kernel, two passes over the keys
// -------------------------------------------------------------------------------------------------------------------
// The reference's inference calls return the probabilities (its coverage), so they have to be written once; the scores
// do not, and with them goes a write, a read and two launches of the [heads, tq, tk] tensor. The tiling is the
// forward's above. Pass 1 streams the key tiles and keeps the running maximum and sum of each row; pass 2 streams keys
// and values, recomputes the scores, writes the normalised probabilities (through a strip of LDS per wavefront, so that a
// row's 64 keys leave as 128 contiguous bytes) and multiplies them with the values. The scores are rounded to the
// tensors' 16-bit type before the softmax, as a stored score tensor would round them.
constexpr int PA_PITCH = FA_TILE * 2 + 8;    // bytes per row of a wavefront's probability strip
// The score of a masked key, and the running maximum before any key: a power of two, so that its product with log2(e)
// is exact and exp2(fma(dead, log2e, -(dead * log2e))) is exactly 1 for a row that has seen no live key yet (any other
// constant leaves the fma a rounding residue of 1e22, whose exp2 overflows).
constexpr float PA_DEAD = -0x1p100f;

// the two 16-bit elements of a register as floats
template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t w);
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t w);
template <> __device__ __forceinline__ float unpack_lo<bf16_t>(uint32_t w) { return __uint_as_float(w << 16); }
template <> __device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
template <> __device__ __forceinline__ float unpack_lo<f16_t>(uint32_t w) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w & 0xffffu)));
}
template <> __device__ __forceinline__ float unpack_hi<f16_t>(uint32_t w) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w >> 16)));
}

// mask bytes (1 = masked) of the four keys key0 .. key0 + 3 for this lane's query, keys past the end count as masked.
// The load is unconditional (from a clamped address) and the eight words of a tile are requested together. Two steps,
// so that a caller can ask for a tile's words early and touch them (which is where the wait for the load lands) late:
// the load from the clamped address, then the words of keys past the end.
template <int MASK>
__device__ __forceinline__ uint32_t mask_word_load(const AttnProbsCall& a, int b, int qrow, int key0) {
  if constexpr (MASK == 0) return 0u;
  const int kc = min(key0, a.tk - 4);                 // tk is a positive multiple of 4
  const int64_t row = MASK == 1 ? b : min(qrow, a.tq - 1);
  return *reinterpret_cast<const uint32_t*>(a.mask + row * a.tk + kc);
}
template <int MASK>
__device__ __forceinline__ void tile_mask_load(const AttnProbsCall& a, int b, int qrow, int t, int half, uint32_t (&mw)[2][4]) {
#pragma unroll
  for (int n = 0; n < 2; ++n)
#pragma unroll
    for (int g = 0; g < 4; ++g) mw[n][g] = mask_word_load<MASK>(a, b, qrow, t * FA_TILE + 32 * n + 8 * g + 4 * half);
}
__device__ __forceinline__ void tile_mask_finish(const AttnProbsCall& a, int t, int half, const uint32_t (&raw)[2][4], uint32_t (&mw)[2][4]) {
#pragma unroll
  for (int n = 0; n < 2; ++n)
#pragma unroll
    for (int g = 0; g < 4; ++g) mw[n][g] = t * FA_TILE + 32 * n + 8 * g + 4 * half < a.tk ? raw[n][g] : 0x01010101u;
}

// G groups of four wavefronts share the block's 128 queries and take the key tiles in turn (tile t goes to group
// t % G); each group has its own tile buffers, the row statistics after pass 1 and the context accumulators after pass 2
// are combined through LDS. G = 2 is for calls with so few blocks (a decoder's 128 positions: one block per head and
// sentence) that four wavefronts per compute unit would leave the vector units waiting on every dependency.
template <typename T, int D, int MASK, int G>
__global__ __launch_bounds__(FA_THREADS * G, (D == 64 && G == 1) ? 2 : 1) void attn_probs_kernel(AttnProbsCall a) {
  extern __shared__ __align__(16) uint8_t lds_raw[];
  constexpr int IMG = FA_TILE * D * 2, NWAVE = 4 * G;
  const int b = blockIdx.z, h = blockIdx.y, q0 = static_cast<int>(blockIdx.x) * FA_ROWS;
  const int lane = static_cast<int>(threadIdx.x) & 63, half = lane >> 5;
  const int wave_all = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
  const int group = wave_all / 4, wave = wave_all % 4;
  const int qrow = q0 + 32 * wave + (lane & 31);
  const T* qb = static_cast<const T*>(a.q) + b * a.q_sb + h * a.q_sh;
  const T* kb = static_cast<const T*>(a.k) + b * a.k_sb + h * a.k_sh;
  const T* vb = static_cast<const T*>(a.v) + b * a.v_sb + h * a.v_sh;
  uint4 qf[D / 16];
  load_resident<T, D>(qf, qb, a.q_st, qrow, a.tq, lane);
  const int ntiles = (a.tk + FA_TILE - 1) / FA_TILE;
  uint8_t* tiles = lds_raw + group * (4 * IMG);
  uint8_t* strip = lds_raw + G * (4 * IMG) + wave_all * (32 * PA_PITCH);
  float* stats = reinterpret_cast<float*>(lds_raw + G * (4 * IMG) + NWAVE * (32 * PA_PITCH));   // [G][128][2]
  // With a key-padding mask the sentence's keys end somewhere before tk (padding sits at the end of a batch's shorter
  // sentences): the tiles behind the last live key are not computed, their probabilities are written as the zeros they are.
  int live_tiles = ntiles;
  if constexpr (MASK == 1) {
    int last = -1;
    const uint8_t* mrow = a.mask + static_cast<int64_t>(b) * a.tk;
    for (int j = 4 * static_cast<int>(threadIdx.x); j < a.tk; j += 4 * FA_THREADS * G) {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(mrow + j);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (((w >> (8 * e)) & 0xffu) == 0) last = j + e;
    }
    const float wl = wave_max(static_cast<float>(last));     // key indices are far below 2^24: exact in fp32
    if (lane == 0) stats[wave_all] = wl;
    __syncthreads();
    float bl = stats[0];
#pragma unroll
    for (int w = 1; w < NWAVE; ++w) bl = fmaxf(bl, stats[w]);
    live_tiles = (static_cast<int>(bl) + 1 + FA_TILE - 1) / FA_TILE;
    __syncthreads();                                        // stats is written again after pass 1
  }

  // the tile's 32 scores of this lane, rounded and masked. The mask words of a tile are requested one round ahead, behind
  // the loads of that tile's keys (values): vector loads return in order, so a mask word asked for at its tile would be
  // waited for together with the next tile's keys, and every round would last a whole memory latency.
  auto tile_scores = [&](const uint8_t* kimg, const uint32_t (&mw)[2][4], acc16_t (&s)[2]) {
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[n][r] = 0.f;
#pragma unroll
    for (int ss = 0; ss < D / 16; ++ss)
#pragma unroll
      for (int n = 0; n < 2; ++n) mfma<T>::run(read_rows<D>(kimg, n, ss, lane), qf[ss], s[n]);
    // scaled, rounded to the 16-bit type two at a time (one packed conversion, two unpacking shifts), masked; natural units
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          const uint32_t pr = pack2<T>(s[n][4 * g + e] * a.scale, s[n][4 * g + e + 1] * a.scale);
          const float lo = unpack_lo<T>(pr), hi = unpack_hi<T>(pr);
          s[n][4 * g + e] = ((mw[n][g] >> (8 * e)) & 0xffu) != 0 ? PA_DEAD : lo;
          s[n][4 * g + e + 1] = ((mw[n][g] >> (8 * e + 8)) & 0xffu) != 0 ? PA_DEAD : hi;
        }
      }
  };

  // ---- pass 1: row maximum and sum over this group's tiles ----
  float m = PA_DEAD, l = 0.f;
  Staged<D> sk, sv;
  const int live_rounds = (live_tiles + G - 1) / G;
  uint32_t mw[2][4], mw_next[2][4];
  // (the empty statement keeps the compiler from working on the words, and so from waiting for them, any earlier)
  auto take_next_mask = [&](int t) {
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int g = 0; g < 4; ++g) asm volatile("" : "+v"(mw_next[n][g]));
    tile_mask_finish(a, t, half, mw_next, mw);
  };
  tile_mask_load<MASK>(a, b, qrow, group, half, mw_next);   // clamped addresses: any tile index may be asked for
  tile_mask_finish(a, group, half, mw_next, mw);
  if (group < live_tiles) {
    sk.load(kb, a.k_st, group * FA_TILE, a.tk);
    sk.store_rows(tiles);
  }
  registers_landed(qf);
  __syncthreads();
  for (int it = 0; it < live_rounds; ++it) {
    const int t = it * G + group;
    const uint8_t* kimg = tiles + (it & 1) * 2 * IMG;
    if (t + G < live_tiles) {
      sk.load(kb, a.k_st, (t + G) * FA_TILE, a.tk);
      tile_mask_load<MASK>(a, b, qrow, t + G, half, mw_next);
    }
    if (t < live_tiles) {
      acc16_t s[2];
      tile_scores(kimg, mw, s);
      float mx = s[0][0];
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[n][r]);
      const float m_new = fmaxf(m, pair_max(mx));
      const float m2 = m_new * FA_LOG2E;
      float sum = 0.f;
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) sum += fast_exp2(__builtin_fmaf(s[n][r], FA_LOG2E, -m2));
      l = l * fast_exp2((m - m_new) * FA_LOG2E) + sum;
      m = m_new;
    }
    if (t + G < live_tiles) {
      sk.store_rows(tiles + ((it + 1) & 1) * 2 * IMG);
      take_next_mask(t + G);
    }
    __syncthreads();
  }
  l = pair_sum(l);
  if constexpr (G > 1) {
    if (half == 0) {
      stats[((group * 4 + wave) * 32 + lane) * 2] = m;
      stats[((group * 4 + wave) * 32 + lane) * 2 + 1] = l;
    }
    __syncthreads();
    float mm = PA_DEAD, ll = 0.f;
#pragma unroll
    for (int gg = 0; gg < G; ++gg) mm = fmaxf(mm, stats[((gg * 4 + wave) * 32 + (lane & 31)) * 2]);
#pragma unroll
    for (int gg = 0; gg < G; ++gg) {
      const float* st2 = stats + ((gg * 4 + wave) * 32 + (lane & 31)) * 2;
      ll += st2[1] * fast_exp2((st2[0] - mm) * FA_LOG2E);
    }
    m = mm;
    l = ll;
  }
  // a row without a live key keeps the initial maximum: its probabilities are zeros (the reference turns the NaN into 0)
  const float inv = (m > 0.5f * PA_DEAD && l > 0.f) ? 1.f / l : 0.f;

  // ---- pass 2: probabilities out, context accumulated ----
  const float m2 = m * FA_LOG2E;
  acc16_t o[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  tile_mask_load<MASK>(a, b, qrow, group, half, mw_next);
  tile_mask_finish(a, group, half, mw_next, mw);
  if (group < live_tiles) {
    sk.load(kb, a.k_st, group * FA_TILE, a.tk);
    sv.load(vb, a.v_st, group * FA_TILE, a.tk);
    sk.store_rows(tiles);
    sv.store_transposed(tiles + IMG);
  }
  registers_landed(qf);
  __syncthreads();
  T* prow = static_cast<T*>(a.probs) + (static_cast<int64_t>(b) * a.heads + h) * a.tq * a.tk;
  // the tiles behind the last live key: zeros, no arithmetic (every wavefront of the block takes its share of them)
  for (int t = live_tiles + group; a.probs != nullptr && t < ntiles; t += G) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = q0 + 32 * wave + 4 * j + (lane >> 4), key = t * FA_TILE + 4 * (lane & 15);
      if (row < a.tq && key < a.tk) *reinterpret_cast<uint2*>(prow + static_cast<int64_t>(row) * a.tk + key) = make_uint2(0, 0);
    }
  }
  for (int it = 0; it < live_rounds; ++it) {
    const int t = it * G + group;
    const uint8_t* kimg = tiles + (it & 1) * 2 * IMG;
    const uint8_t* vimg = kimg + IMG;
    if (t + G < live_tiles) {
      sk.load(kb, a.k_st, (t + G) * FA_TILE, a.tk);
      sv.load(vb, a.v_st, (t + G) * FA_TILE, a.tk);
      tile_mask_load<MASK>(a, b, qrow, t + G, half, mw_next);
    }
    if (t < live_tiles) {
      acc16_t s[2];
      tile_scores(kimg, mw, s);
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[n][r] = fast_exp2(__builtin_fmaf(s[n][r], FA_LOG2E, -m2)) * inv;
      // this lane's 4-key groups into the wavefront's strip: row = its query, 8 bytes per group (a caller that does not
      // want the probabilities passes no buffer for them)
      if (a.probs != nullptr) {
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            uint2 w;
            w.x = pack2<T>(s[n][4 * g + 0], s[n][4 * g + 1]);
            w.y = pack2<T>(s[n][4 * g + 2], s[n][4 * g + 3]);
            *reinterpret_cast<uint2*>(strip + (lane & 31) * PA_PITCH + (32 * n + 8 * g + 4 * half) * 2) = w;
          }
      }
#pragma unroll
      for (int kk = 0; kk < FA_TILE / 16; ++kk) {
        float pv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) pv[e] = s[kk / 2][8 * (kk % 2) + e];
        const uint4 pf = acc_to_operand<T>(pv);
#pragma unroll
        for (int i = 0; i < D / 32; ++i) mfma<T>::run(read_transposed<D>(vimg, i, kk, lane), pf, o[i]);
      }
      if (a.probs != nullptr) {
        wave_lds_fence();
        // 16 lanes take one row's 64 keys (8 bytes each), four rows per step
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int r = 4 * j + (lane >> 4), key = t * FA_TILE + 4 * (lane & 15);
          const int row = q0 + 32 * wave + r;
          if (row < a.tq && key < a.tk)
            *reinterpret_cast<uint2*>(prow + static_cast<int64_t>(row) * a.tk + key) =
                *reinterpret_cast<const uint2*>(strip + r * PA_PITCH + 8 * (lane & 15));
        }
        wave_lds_fence();
      }
    }
    if (t + G < live_tiles) {
      uint8_t* nk = tiles + ((it + 1) & 1) * 2 * IMG;
      sk.store_rows(nk);
      sv.store_transposed(nk + IMG);
      take_next_mask(t + G);
    }
    __syncthreads();
  }
  if constexpr (G > 1) {
    // the other groups' partial contexts through LDS (over the tile buffers, which nobody reads any more)
    float4* part = reinterpret_cast<float4*>(lds_raw);
    if (group != 0) {
#pragma unroll
      for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          part[((((group - 1) * 4 + wave) * (D / 32) + i) * 4 + g) * 64 + lane] =
              make_float4(o[i][4 * g], o[i][4 * g + 1], o[i][4 * g + 2], o[i][4 * g + 3]);
    }
    __syncthreads();
    if (group == 0) {
#pragma unroll
      for (int gg = 0; gg < G - 1; ++gg)
#pragma unroll
        for (int i = 0; i < D / 32; ++i)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float4 x = part[(((gg * 4 + wave) * (D / 32) + i) * 4 + g) * 64 + lane];
            o[i][4 * g] += x.x; o[i][4 * g + 1] += x.y; o[i][4 * g + 2] += x.z; o[i][4 * g + 3] += x.w;
          }
    }
    __syncthreads();
  }
  T* cb = static_cast<T*>(a.ctx) + b * a.c_sb + h * a.c_sh;
  // every wavefront takes part in the store's barrier; only group 0 holds rows to store
  store_rows_out<T, D>(o, 1.f, lds_raw + wave_all * (32 * D * 2), cb, a.c_st, q0 + 32 * wave, group == 0 ? a.tq : 0, lane);
}

template <int D, int G> constexpr int probs_lds() { return G * (4 * FA_TILE * D * 2 + 4 * 32 * PA_PITCH + 128 * 2 * 4); }

template <int D> constexpr int fwd_lds() { return 2 * 2 * FA_TILE * D * 2; }
template <int D> constexpr int dq_lds() { return 2 * 3 * FA_TILE * D * 2; }
template <int D> constexpr int dkv_lds() { return 2 * (4 * FA_TILE * D * 2 + 2 * FA_TILE * 4); }

template <typename K>
int launch(K kern, const char* what, dim3 grid, int lds, hipStream_t st, const FaArgs& a) {
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, lds, hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kern, grid, dim3(FA_THREADS), lds, st, a);
  return 0;
}

template <typename T, int D>
int fwd_launch(const FaArgs& a, int drop, dim3 grid, hipStream_t st) {
  TraceScope trace("flash_attn_fwd", st);
  if (a.tmask != nullptr)
    return drop == 0 ? launch(flash_fwd_kernel<T, D, 0, 2>, "flash_attn_fwd", grid, fwd_lds<D>(), st, a)
                     : launch(flash_fwd_kernel<T, D, 1, 2>, "flash_attn_fwd", grid, fwd_lds<D>(), st, a);
  if (a.pad != nullptr)
    return drop == 0 ? launch(flash_fwd_kernel<T, D, 0, 1>, "flash_attn_fwd", grid, fwd_lds<D>(), st, a)
                     : launch(flash_fwd_kernel<T, D, 1, 1>, "flash_attn_fwd", grid, fwd_lds<D>(), st, a);
  return drop == 0 ? launch(flash_fwd_kernel<T, D, 0, 0>, "flash_attn_fwd", grid, fwd_lds<D>(), st, a)
                   : launch(flash_fwd_kernel<T, D, 1, 0>, "flash_attn_fwd", grid, fwd_lds<D>(), st, a);
}
template <typename T, int D>
int bwd_launch(const FaArgs& a, int drop, dim3 grid_q, dim3 grid_k, hipStream_t st) {
  int rc = 0;
  if (grid_q.x > 0) {
    TraceScope trace("flash_attn_bwd_dq", st);
    if (a.tmask != nullptr)
      rc = drop == 0 ? launch(flash_bwd_dq_kernel<T, D, 0, 2>, "flash_attn_bwd", grid_q, dq_lds<D>(), st, a)
                     : launch(flash_bwd_dq_kernel<T, D, 1, 2>, "flash_attn_bwd", grid_q, dq_lds<D>(), st, a);
    else if (a.pad != nullptr)
      rc = drop == 0 ? launch(flash_bwd_dq_kernel<T, D, 0, 1>, "flash_attn_bwd", grid_q, dq_lds<D>(), st, a)
                     : launch(flash_bwd_dq_kernel<T, D, 1, 1>, "flash_attn_bwd", grid_q, dq_lds<D>(), st, a);
    else
      rc = drop == 0 ? launch(flash_bwd_dq_kernel<T, D, 0, 0>, "flash_attn_bwd", grid_q, dq_lds<D>(), st, a)
                     : launch(flash_bwd_dq_kernel<T, D, 1, 0>, "flash_attn_bwd", grid_q, dq_lds<D>(), st, a);
  }
  if (rc || grid_k.x == 0) return rc;
  TraceScope trace("flash_attn_bwd_dkv", st);
  if (a.tmask != nullptr)
    return drop == 0 ? launch(flash_bwd_dkv_kernel<T, D, 0, 1>, "flash_attn_bwd", grid_k, dkv_lds<D>(), st, a)
                     : launch(flash_bwd_dkv_kernel<T, D, 1, 1>, "flash_attn_bwd", grid_k, dkv_lds<D>(), st, a);
  return drop == 0 ? launch(flash_bwd_dkv_kernel<T, D, 0, 0>, "flash_attn_bwd", grid_k, dkv_lds<D>(), st, a)
                   : launch(flash_bwd_dkv_kernel<T, D, 1, 0>, "flash_attn_bwd", grid_k, dkv_lds<D>(), st, a);
}

int64_t bits_q32(int64_t max_q) { return 4 * ((max_q + FA_ROWS - 1) / FA_ROWS); }
int64_t bits_kp(int64_t max_k) { return FA_TILE * ((max_k + FA_TILE - 1) / FA_TILE); }

// The keep bits of a call with dropout: drawn from the generator (mode 2) or taken from the byte mask (mode 1).
int bits_launch(const char* what, FaArgs& a, int drop_mode, int64_t batch, void* bits, bool ready, hipStream_t st) {
  if (drop_mode == 0) return 0;
  NMTG_REQUIRE(bits != nullptr && aligned16(bits), "%s: dropout needs the 16-byte aligned keep-bit workspace (nmtg_flash_attn_dropout_bits_bytes)", what);
  a.bits = static_cast<uint32_t*>(bits);
  a.q32 = static_cast<int>(bits_q32(a.max_q));
  a.kp = static_cast<int>(bits_kp(a.max_k));
  if (ready || a.max_q == 0 || a.max_k == 0) return 0;
  const int64_t rows = batch * a.heads * a.q32;
  const bool words = drop_mode == 1 && a.max_k % 4 == 0 && reinterpret_cast<uintptr_t>(a.mask) % 4 == 0;   // four keys per thread
  const int64_t total = rows * (drop_mode == 2 || words ? a.kp / 4 : a.kp);
  NMTG_REQUIRE((total + 255) / 256 <= 0x7fffffff, "%s: keep-bit workspace beyond one launch", what);
  TraceScope trace("flash_attn_keep_bits", st);
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (drop_mode == 2) hipLaunchKernelGGL(flash_bits_rng_kernel, grid, dim3(256), 0, st, a, total);
  else if (words) hipLaunchKernelGGL(flash_bits_mask4_kernel, grid, dim3(256), 0, st, a, total);
  else hipLaunchKernelGGL(flash_bits_mask_kernel, grid, dim3(256), 0, st, a, total);
  return 0;
}

bool view_ok(const void* p, int64_t st, int64_t sh, int64_t heads, int64_t d) {
  return aligned16(p) && st % 8 == 0 && sh % 8 == 0 && sh >= d && st >= (heads - 1) * sh + d;
}

int check_common(const char* what, int64_t batch, int64_t heads, int64_t d, int64_t max_q, int64_t max_k, int drop_mode, float p,
                 float scale, int dtype) {
  NMTG_REQUIRE(fabsf(scale) >= 1e-6f && fabsf(scale) <= 1e6f, "%s: softmax_scale %g (magnitudes from 1e-6 to 1e6 are handled)", what,
               (double)scale);
  NMTG_REQUIRE(batch >= 0 && heads >= 1 && max_q >= 0 && max_k >= 0, "%s: bad shape batch=%lld heads=%lld max_q=%lld max_k=%lld",
               what, (long long)batch, (long long)heads, (long long)max_q, (long long)max_k);
  NMTG_REQUIRE(d == 64 || d == 128, "%s: head dimension %lld (64 and 128 are built)", what, (long long)d);
  NMTG_REQUIRE(dtype == NMTG_F16 || dtype == NMTG_BF16, "%s: fp16 or bf16 tensors required (matrix-core kernel)", what);
  NMTG_REQUIRE(drop_mode >= 0 && drop_mode <= 2, "%s: dropout mode %d", what, drop_mode);
  NMTG_REQUIRE(drop_mode == 0 || (p >= 0.f && p < 1.f), "%s: dropout probability %g outside [0, 1)", what, (double)p);
  NMTG_REQUIRE(heads <= 65535 && batch <= 65535, "%s: more than 65535 heads or sequences in one launch", what);
  NMTG_REQUIRE(batch * heads * (max_q + 3) / 4 * ((max_k + 3) / 4) < (1ll << 62) && max_q <= (1 << 24) && max_k <= (1 << 24),
               "%s: sequence lengths too large", what);
  return 0;
}

void set_dropout(FaArgs& a, int drop_mode, float p, uint64_t seed, uint64_t offset) {
  a.thr = 256;
  a.drop_scale = 1.f;
  if (drop_mode == 1) a.drop_scale = 1.f / (1.f - p);
  if (drop_mode == 2) {
    long thr = lroundf(256.f * (1.f - p));
    a.thr = static_cast<uint32_t>(thr < 1 ? 1 : thr > 256 ? 256 : thr);
    a.drop_scale = 256.f / static_cast<float>(a.thr);
  }
  a.seed = seed;
  a.offset = offset;
}

// the launches of a forward call whose arguments are in place: keep bits, then the attention kernel
int fwd_run(const char* what, FaArgs& a, int64_t batch, int64_t d, int drop_mode, void* bits, int dtype, hipStream_t st) {
  const dim3 grid(static_cast<unsigned>((a.max_q + FA_ROWS - 1) / FA_ROWS), static_cast<unsigned>(a.heads), static_cast<unsigned>(batch));
  int rc = bits_launch(what, a, drop_mode, batch, bits, false, st);
  if (rc) return rc;
  if (dtype == NMTG_F16) rc = d == 64 ? fwd_launch<f16_t, 64>(a, drop_mode, grid, st) : fwd_launch<f16_t, 128>(a, drop_mode, grid, st);
  else rc = d == 64 ? fwd_launch<bf16_t, 64>(a, drop_mode, grid, st) : fwd_launch<bf16_t, 128>(a, drop_mode, grid, st);
  if (rc) return rc;
  NMTG_CHECK_LAUNCH(what);
  return 0;
}

int bwd_run(const char* what, FaArgs& a, int64_t batch, int64_t d, int drop_mode, void* bits, bool bits_ready, int dtype, hipStream_t st) {
  const dim3 grid_q(static_cast<unsigned>((a.max_q + FA_ROWS - 1) / FA_ROWS), static_cast<unsigned>(a.heads), static_cast<unsigned>(batch));
  const dim3 grid_k(static_cast<unsigned>((a.max_k + FA_ROWS - 1) / FA_ROWS), static_cast<unsigned>(a.heads), static_cast<unsigned>(batch));
  int rc = bits_launch(what, a, drop_mode, batch, bits, bits_ready, st);
  if (rc) return rc;
  if (dtype == NMTG_F16) rc = d == 64 ? bwd_launch<f16_t, 64>(a, drop_mode, grid_q, grid_k, st) : bwd_launch<f16_t, 128>(a, drop_mode, grid_q, grid_k, st);
  else rc = d == 64 ? bwd_launch<bf16_t, 64>(a, drop_mode, grid_q, grid_k, st) : bwd_launch<bf16_t, 128>(a, drop_mode, grid_q, grid_k, st);
  if (rc) return rc;
  NMTG_CHECK_LAUNCH(what);
  return 0;
}

// a [len, batch, heads, head_dim] view: as view_ok, and a batch stride that keeps the alignment
bool batched_view_ok(const void* p, int64_t st, int64_t sb, int64_t sh, int64_t heads, int64_t d) {
  return aligned16(p) && st % 8 == 0 && sb % 8 == 0 && sh % 8 == 0 && sh >= d && sb >= 0 && st >= 0;
}

// the key padding mask of a batch-strided call: fills key_info ahead of every kernel that reads it
int key_info_launch(const char* what, FaArgs& a, int64_t batch, const uint8_t* pad, void* key_info, hipStream_t st) {
  if (pad == nullptr) return 0;
  NMTG_REQUIRE(key_info != nullptr && reinterpret_cast<uintptr_t>(key_info) % 4 == 0,
               "%s: a key padding mask needs the key_info workspace (nmtg_flash_attn_key_info_bytes)", what);
  a.pad = pad;
  a.kinfo = static_cast<const int32_t*>(key_info);
  a.kinfo_pitch = 1 + (a.max_k + FA_TILE - 1) / FA_TILE;
  a.key_tiles = a.kinfo_pitch - 1;
  uint32_t* bits = static_cast<uint32_t*>(key_info) + batch * a.kinfo_pitch;      // behind the summaries
  a.pad_bits = bits;
  if (a.max_k == 0) return 0;
  TraceScope trace("flash_attn_key_info", st);
  hipLaunchKernelGGL(flash_key_info_kernel, dim3(static_cast<unsigned>(batch)), dim3(256), 0, st, pad, a.max_k,
                     static_cast<int32_t*>(key_info), a.kinfo_pitch, bits);
  return 0;
}

// the time mask of a batch-strided call: fills time_info (the two summaries, one behind the other) ahead of every kernel
int64_t time_summary_words(int64_t len_q, int64_t len_k) {
  return (len_q + 31) / 32 * (1 + (len_k + FA_TILE - 1) / FA_TILE) + (len_k + 31) / 32 * (2 + (len_q + FA_TILE - 1) / FA_TILE);
}
int64_t time_info_words(int64_t len_q, int64_t len_k) {   // + the packed mask, by query and by key
  return time_summary_words(len_q, len_k) + 2 * len_q * ((len_k + FA_TILE - 1) / FA_TILE) + 2 * len_k * ((len_q + FA_TILE - 1) / FA_TILE);
}
int time_info_launch(const char* what, FaArgs& a, const uint8_t* time_mask, void* time_info, hipStream_t st) {
  if (time_mask == nullptr) return 0;
  NMTG_REQUIRE(a.pad == nullptr, "%s: a key padding mask or a time mask, not both", what);
  NMTG_REQUIRE(time_info != nullptr && reinterpret_cast<uintptr_t>(time_info) % 4 == 0,
               "%s: a time mask needs the time_info workspace (nmtg_flash_attn_time_info_bytes)", what);
  if (a.max_q == 0 || a.max_k == 0) return 0;
  const int qgroups = (a.max_q + 31) / 32, kgroups = (a.max_k + 31) / 32;
  a.tmask = time_mask;
  a.qinfo_pitch = 1 + (a.max_k + FA_TILE - 1) / FA_TILE;
  a.kqinfo_pitch = 2 + (a.max_q + FA_TILE - 1) / FA_TILE;
  int32_t* base = static_cast<int32_t*>(time_info);
  a.qinfo = base;
  a.kqinfo = base + static_cast<int64_t>(qgroups) * a.qinfo_pitch;
  a.key_tiles = a.qinfo_pitch - 1;
  a.query_tiles = a.kqinfo_pitch - 2;
  uint32_t* tq = reinterpret_cast<uint32_t*>(base + time_summary_words(a.max_q, a.max_k));
  uint32_t* tk = tq + static_cast<int64_t>(a.max_q) * a.key_tiles * 2;
  a.tq_bits = tq;
  a.tk_bits = tk;
  const int64_t words = 2 * (static_cast<int64_t>(a.max_q) * a.key_tiles + static_cast<int64_t>(a.max_k) * a.query_tiles);
  const int64_t blocks = qgroups + kgroups + (words + 255) / 256;
  NMTG_REQUIRE(blocks <= 0x7fffffff, "%s: time mask too large", what);
  TraceScope trace("flash_attn_time_info", st);
  hipLaunchKernelGGL(flash_time_info_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, time_mask, a.max_q,
                     a.max_k, base, a.qinfo_pitch, base + static_cast<int64_t>(qgroups) * a.qinfo_pitch, a.kqinfo_pitch, tq, tk);
  return 0;
}

template <typename T, int D, int G>
int probs_launch(const AttnProbsCall& c, dim3 grid, hipStream_t st) {
  auto go = [&](auto kern) {
    constexpr int lds = probs_lds<D, G>();
    if (lds > 64 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "attn_probs: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, grid, dim3(FA_THREADS * G), lds, st, c);
    return 0;
  };
  if (c.mask == nullptr || c.mask_kind == 0) return go(attn_probs_kernel<T, D, 0, G>);
  if (c.mask_kind == 1) return go(attn_probs_kernel<T, D, 1, G>);
  return go(attn_probs_kernel<T, D, 2, G>);
}

}  // namespace

bool attn_probs_ok(const AttnProbsCall& c) {
  if (switched_off("NMTG_ATTN_PROBS")) return false;
  auto view = [&](const void* p, int64_t st, int64_t sb, int64_t sh) {
    return aligned16(p) && st % 8 == 0 && sb % 8 == 0 && sh % 8 == 0 && st >= 0 && sb >= 0 && sh >= 0;
  };
  return (c.dtype == NMTG_F16 || c.dtype == NMTG_BF16) && (c.d == 64 || c.d == 128) && c.tk >= 1 && c.tk % 4 == 0 && c.tq >= 1 &&
         c.batch >= 1 && c.batch <= 65535 && c.heads >= 1 && c.heads <= 65535 && view(c.q, c.q_st, c.q_sb, c.q_sh) &&
         view(c.k, c.k_st, c.k_sb, c.k_sh) && view(c.v, c.v_st, c.v_sb, c.v_sh) && view(c.ctx, c.c_st, c.c_sb, c.c_sh) &&
         reinterpret_cast<uintptr_t>(c.probs) % 8 == 0 &&
         (c.mask == nullptr || c.mask_kind == 0 || reinterpret_cast<uintptr_t>(c.mask) % 4 == 0) && fabsf(c.scale) <= 1e6f;
}

int attn_probs_run(const AttnProbsCall& c, hipStream_t st) {
  // Two groups of wavefronts per block when the blocks alone would not give every SIMD two wavefronts and there are
  // key tiles to share out. NMTG_ATTN_PROBS_SPLIT=0 / =1 forces one form or the other.
  const dim3 grid(static_cast<unsigned>((c.tq + FA_ROWS - 1) / FA_ROWS), static_cast<unsigned>(c.heads), static_cast<unsigned>(c.batch));
  const int64_t blocks = static_cast<int64_t>(grid.x) * grid.y * grid.z;
  const char* forced = getenv("NMTG_ATTN_PROBS_SPLIT");
  // (head dimension 64 only: at 128 the tile buffers of two groups do not fit the LDS)
  const bool split = c.d == 64 && (forced != nullptr && (forced[0] == '0' || forced[0] == '1') ? forced[0] == '1'
                                                                                               : blocks < 2 * 256 && c.tk > 2 * FA_TILE);
  TraceScope trace(split ? "attn_probs_2groups" : "attn_probs", st);
  int rc;
  if (split) {
    rc = c.dtype == NMTG_F16 ? probs_launch<f16_t, 64, 2>(c, grid, st) : probs_launch<bf16_t, 64, 2>(c, grid, st);
  } else {
    if (c.dtype == NMTG_F16) rc = c.d == 64 ? probs_launch<f16_t, 64, 1>(c, grid, st) : probs_launch<f16_t, 128, 1>(c, grid, st);
    else rc = c.d == 64 ? probs_launch<bf16_t, 64, 1>(c, grid, st) : probs_launch<bf16_t, 128, 1>(c, grid, st);
  }
  if (rc) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "attn_probs: launch failed: %s", hipGetErrorString(e));
  return 0;
}

}  // namespace nmtg

using namespace nmtg;

extern "C" int64_t nmtg_flash_attn_dropout_bits_bytes(int64_t batch, int64_t heads, int64_t max_seqlen_q, int64_t max_seqlen_k) {
  if (batch <= 0 || heads <= 0 || max_seqlen_q <= 0 || max_seqlen_k <= 0) return 0;
  return batch * heads * bits_q32(max_seqlen_q) * bits_kp(max_seqlen_k) * 4;
}

extern "C" int nmtg_flash_attn_fwd(const void* q, const void* k, const void* v, void* out, const int32_t* cu_seqlens_q,
                                   const int32_t* cu_seqlens_k, float* softmax_lse, int64_t batch, int64_t heads,
                                   int64_t head_dim, int64_t max_seqlen_q, int64_t max_seqlen_k, int64_t q_stride_t,
                                   int64_t q_stride_h, int64_t k_stride_t, int64_t k_stride_h, int64_t v_stride_t,
                                   int64_t v_stride_h, int64_t out_stride_t, int64_t out_stride_h, float softmax_scale,
                                   int causal, int dropout_mode, float dropout_p, const uint8_t* dropout_mask,
                                   uint8_t* dropout_mask_out, void* dropout_bits, uint64_t seed, uint64_t offset, int dtype,
                                   void* stream) {
  if (int rc = check_common("flash_attn_fwd", batch, heads, head_dim, max_seqlen_q, max_seqlen_k, dropout_mode, dropout_p, softmax_scale, dtype)) return rc;
  if (batch == 0 || max_seqlen_q == 0) return 0;
  NMTG_REQUIRE(q && k && v && out && cu_seqlens_q && cu_seqlens_k && softmax_lse, "flash_attn_fwd: null pointer argument");
  NMTG_REQUIRE(dropout_mode != 1 || dropout_mask, "flash_attn_fwd: dropout mode 1 replays a keep-mask and none was given");
  NMTG_REQUIRE(view_ok(q, q_stride_t, q_stride_h, heads, head_dim) && view_ok(k, k_stride_t, k_stride_h, heads, head_dim) &&
                   view_ok(v, v_stride_t, v_stride_h, heads, head_dim) && view_ok(out, out_stride_t, out_stride_h, heads, head_dim),
               "flash_attn_fwd: q, k, v and out must be 16-byte aligned [tokens, heads, head_dim] views with a contiguous "
               "head_dim and strides that are multiples of 8 elements");
  FaArgs a = {};
  a.q = q; a.k = k; a.v = v; a.out = out; a.lse = softmax_lse; a.cu_q = cu_seqlens_q; a.cu_k = cu_seqlens_k;
  a.q_st = q_stride_t; a.q_sh = q_stride_h; a.k_st = k_stride_t; a.k_sh = k_stride_h; a.v_st = v_stride_t; a.v_sh = v_stride_h;
  a.o_st = out_stride_t; a.o_sh = out_stride_h;
  a.heads = static_cast<int>(heads); a.max_q = static_cast<int>(max_seqlen_q); a.max_k = static_cast<int>(max_seqlen_k);
  a.scale = softmax_scale; a.scale_log2 = softmax_scale * FA_LOG2E; a.causal = causal != 0;
  a.mask = dropout_mask; a.mask_out = dropout_mask_out;
  set_dropout(a, dropout_mode, dropout_p, seed, offset);
  return fwd_run("flash_attn_fwd", a, batch, head_dim, dropout_mode, dropout_bits, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int nmtg_flash_attn_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out,
                                   const float* softmax_lse, void* dq, void* dk, void* dv, float* softmax_d,
                                   const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int64_t batch, int64_t heads,
                                   int64_t head_dim, int64_t max_seqlen_q, int64_t max_seqlen_k, int64_t dout_stride_t,
                                   int64_t dout_stride_h, int64_t q_stride_t, int64_t q_stride_h, int64_t k_stride_t,
                                   int64_t k_stride_h, int64_t v_stride_t, int64_t v_stride_h, int64_t out_stride_t,
                                   int64_t out_stride_h, int64_t dq_stride_t, int64_t dq_stride_h, int64_t dk_stride_t,
                                   int64_t dk_stride_h, int64_t dv_stride_t, int64_t dv_stride_h, float softmax_scale,
                                   int causal, int dropout_mode, float dropout_p, const uint8_t* dropout_mask,
                                   void* dropout_bits, int dropout_bits_ready, uint64_t seed, uint64_t offset, int dtype,
                                   void* stream) {
  if (int rc = check_common("flash_attn_bwd", batch, heads, head_dim, max_seqlen_q, max_seqlen_k, dropout_mode, dropout_p, softmax_scale, dtype)) return rc;
  if (batch == 0) return 0;
  NMTG_REQUIRE(dout && q && k && v && out && softmax_lse && dq && dk && dv && softmax_d && cu_seqlens_q && cu_seqlens_k,
               "flash_attn_bwd: null pointer argument");
  NMTG_REQUIRE(dropout_mode != 1 || dropout_mask || dropout_bits_ready,
               "flash_attn_bwd: dropout mode 1 replays a keep-mask and none was given");
  NMTG_REQUIRE(view_ok(q, q_stride_t, q_stride_h, heads, head_dim) && view_ok(k, k_stride_t, k_stride_h, heads, head_dim) &&
                   view_ok(v, v_stride_t, v_stride_h, heads, head_dim) && view_ok(out, out_stride_t, out_stride_h, heads, head_dim) &&
                   view_ok(dout, dout_stride_t, dout_stride_h, heads, head_dim) && view_ok(dq, dq_stride_t, dq_stride_h, heads, head_dim) &&
                   view_ok(dk, dk_stride_t, dk_stride_h, heads, head_dim) && view_ok(dv, dv_stride_t, dv_stride_h, heads, head_dim),
               "flash_attn_bwd: every tensor must be a 16-byte aligned [tokens, heads, head_dim] view with a contiguous "
               "head_dim and strides that are multiples of 8 elements");
  FaArgs a = {};
  a.q = q; a.k = k; a.v = v; a.o = out; a.d_o = dout; a.dq = dq; a.dk = dk; a.dv = dv;
  a.lse = const_cast<float*>(softmax_lse); a.delta = softmax_d; a.cu_q = cu_seqlens_q; a.cu_k = cu_seqlens_k;
  a.q_st = q_stride_t; a.q_sh = q_stride_h; a.k_st = k_stride_t; a.k_sh = k_stride_h; a.v_st = v_stride_t; a.v_sh = v_stride_h;
  a.o_st = out_stride_t; a.o_sh = out_stride_h; a.do_st = dout_stride_t; a.do_sh = dout_stride_h;
  a.dq_st = dq_stride_t; a.dq_sh = dq_stride_h; a.dk_st = dk_stride_t; a.dk_sh = dk_stride_h; a.dv_st = dv_stride_t; a.dv_sh = dv_stride_h;
  a.heads = static_cast<int>(heads); a.max_q = static_cast<int>(max_seqlen_q); a.max_k = static_cast<int>(max_seqlen_k);
  a.scale = softmax_scale; a.scale_log2 = softmax_scale * FA_LOG2E; a.causal = causal != 0;
  a.mask = dropout_mask; a.mask_out = nullptr;
  set_dropout(a, dropout_mode, dropout_p, seed, offset);
  return bwd_run("flash_attn_bwd", a, batch, head_dim, dropout_mode, dropout_bits, dropout_bits_ready != 0, dtype,
                 static_cast<hipStream_t>(stream));
}

extern "C" int64_t nmtg_flash_attn_key_info_bytes(int64_t batch, int64_t len_k) {
  if (batch <= 0 || len_k < 0) return 0;
  return batch * (1 + 3 * ((len_k + FA_TILE - 1) / FA_TILE)) * 4;      // summaries + two packed words per tile
}

extern "C" int64_t nmtg_flash_attn_time_info_bytes(int64_t len_q, int64_t len_k) {
  if (len_q <= 0 || len_k <= 0) return 0;
  return time_info_words(len_q, len_k) * 4;
}

extern "C" int nmtg_flash_attn_batched_fwd(const void* q, const void* k, const void* v, void* out, const uint8_t* key_padding_mask,
                                           void* key_info, const uint8_t* time_mask, void* time_info, float* softmax_lse, int64_t batch, int64_t heads, int64_t head_dim,
                                           int64_t len_q, int64_t len_k, int64_t q_stride_t, int64_t q_stride_b, int64_t q_stride_h,
                                           int64_t k_stride_t, int64_t k_stride_b, int64_t k_stride_h, int64_t v_stride_t,
                                           int64_t v_stride_b, int64_t v_stride_h, int64_t out_stride_t, int64_t out_stride_b,
                                           int64_t out_stride_h, float softmax_scale, int causal, int dropout_mode, float dropout_p,
                                           const uint8_t* dropout_mask, uint8_t* dropout_mask_out, void* dropout_bits,
                                           uint64_t seed, uint64_t offset, int dtype, void* stream) {
  const char* what = "flash_attn_batched_fwd";
  if (int rc = check_common(what, batch, heads, head_dim, len_q, len_k, dropout_mode, dropout_p, softmax_scale, dtype)) return rc;
  if (batch == 0 || len_q == 0) return 0;
  NMTG_REQUIRE(q && k && v && out && softmax_lse, "%s: null pointer argument", what);
  NMTG_REQUIRE(dropout_mode != 1 || dropout_mask, "%s: dropout mode 1 replays a keep-mask and none was given", what);
  NMTG_REQUIRE(batched_view_ok(q, q_stride_t, q_stride_b, q_stride_h, heads, head_dim) &&
                   batched_view_ok(k, k_stride_t, k_stride_b, k_stride_h, heads, head_dim) &&
                   batched_view_ok(v, v_stride_t, v_stride_b, v_stride_h, heads, head_dim) &&
                   batched_view_ok(out, out_stride_t, out_stride_b, out_stride_h, heads, head_dim),
               "%s: q, k, v and out must be 16-byte aligned [len, batch, heads, head_dim] views with a contiguous head_dim and "
               "strides that are multiples of 8 elements", what);
  FaArgs a = {};
  a.q = q; a.k = k; a.v = v; a.out = out; a.lse = softmax_lse;
  a.q_st = q_stride_t; a.q_sb = q_stride_b; a.q_sh = q_stride_h; a.k_st = k_stride_t; a.k_sb = k_stride_b; a.k_sh = k_stride_h;
  a.v_st = v_stride_t; a.v_sb = v_stride_b; a.v_sh = v_stride_h; a.o_st = out_stride_t; a.o_sb = out_stride_b; a.o_sh = out_stride_h;
  a.heads = static_cast<int>(heads); a.max_q = static_cast<int>(len_q); a.max_k = static_cast<int>(len_k);
  a.scale = softmax_scale; a.scale_log2 = softmax_scale * FA_LOG2E; a.causal = causal != 0;
  a.mask = dropout_mask; a.mask_out = dropout_mask_out;
  set_dropout(a, dropout_mode, dropout_p, seed, offset);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = key_info_launch(what, a, batch, key_padding_mask, key_info, st)) return rc;
  if (int rc = time_info_launch(what, a, time_mask, time_info, st)) return rc;
  return fwd_run(what, a, batch, head_dim, dropout_mode, dropout_bits, dtype, st);
}

extern "C" int nmtg_flash_attn_batched_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out,
                                           const float* softmax_lse, void* dq, void* dk, void* dv, float* softmax_d,
                                           const uint8_t* key_padding_mask, void* key_info, const uint8_t* time_mask,
                                           void* time_info, int64_t batch, int64_t heads,
                                           int64_t head_dim, int64_t len_q, int64_t len_k, int64_t q_stride_t, int64_t q_stride_b,
                                           int64_t q_stride_h, int64_t k_stride_t, int64_t k_stride_b, int64_t k_stride_h,
                                           int64_t v_stride_t, int64_t v_stride_b, int64_t v_stride_h, int64_t out_stride_t,
                                           int64_t out_stride_b, int64_t out_stride_h, float softmax_scale, int causal,
                                           int dropout_mode, float dropout_p, const uint8_t* dropout_mask, void* dropout_bits,
                                           int dropout_bits_ready, uint64_t seed, uint64_t offset, int dtype, void* stream) {
  const char* what = "flash_attn_batched_bwd";
  if (int rc = check_common(what, batch, heads, head_dim, len_q, len_k, dropout_mode, dropout_p, softmax_scale, dtype)) return rc;
  if (batch == 0) return 0;
  NMTG_REQUIRE(dout && q && k && v && out && softmax_lse && dq && dk && dv && softmax_d, "%s: null pointer argument", what);
  NMTG_REQUIRE(dropout_mode != 1 || dropout_mask || dropout_bits_ready, "%s: dropout mode 1 replays a keep-mask and none was given", what);
  NMTG_REQUIRE(batched_view_ok(q, q_stride_t, q_stride_b, q_stride_h, heads, head_dim) &&
                   batched_view_ok(k, k_stride_t, k_stride_b, k_stride_h, heads, head_dim) &&
                   batched_view_ok(v, v_stride_t, v_stride_b, v_stride_h, heads, head_dim) &&
                   batched_view_ok(out, out_stride_t, out_stride_b, out_stride_h, heads, head_dim) && aligned16(dout) &&
                   aligned16(dq) && aligned16(dk) && aligned16(dv),
               "%s: every tensor must be a 16-byte aligned [len, batch, heads, head_dim] view with a contiguous head_dim and "
               "strides that are multiples of 8 elements", what);
  FaArgs a = {};
  a.q = q; a.k = k; a.v = v; a.o = out; a.d_o = dout; a.dq = dq; a.dk = dk; a.dv = dv;
  a.lse = const_cast<float*>(softmax_lse); a.delta = softmax_d;
  a.q_st = a.dq_st = q_stride_t; a.q_sb = a.dq_sb = q_stride_b; a.q_sh = a.dq_sh = q_stride_h;
  a.k_st = a.dk_st = k_stride_t; a.k_sb = a.dk_sb = k_stride_b; a.k_sh = a.dk_sh = k_stride_h;
  a.v_st = a.dv_st = v_stride_t; a.v_sb = a.dv_sb = v_stride_b; a.v_sh = a.dv_sh = v_stride_h;
  a.o_st = a.do_st = out_stride_t; a.o_sb = a.do_sb = out_stride_b; a.o_sh = a.do_sh = out_stride_h;
  a.heads = static_cast<int>(heads); a.max_q = static_cast<int>(len_q); a.max_k = static_cast<int>(len_k);
  a.scale = softmax_scale; a.scale_log2 = softmax_scale * FA_LOG2E; a.causal = causal != 0;
  a.mask = dropout_mask; a.mask_out = nullptr;
  set_dropout(a, dropout_mode, dropout_p, seed, offset);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = key_info_launch(what, a, batch, key_padding_mask, key_info, st)) return rc;
  if (int rc = time_info_launch(what, a, time_mask, time_info, st)) return rc;
  return bwd_run(what, a, batch, head_dim, dropout_mode, dropout_bits, dropout_bits_ready != 0, dtype, st);
}

// Paged causal attention on the matrix cores (bf16 in, fp32 accumulate) for
// gfx950.  Compiled once per head size: -DFG_HD=<multiple of 16, at most 256>.
//
// Both kernels work on *items*: an item is a run of consecutive query tokens
// of one sequence; its rows are (token, query head of one kv head's group),
// token-major.  Per 64-key tile a wave computes, with v_mfma_f32_16x16x32_bf16,
//   S^T = K Q^T      (A = 16 keys x 32 head dims, B = Q^T, 16 query rows)
//   O^T += V^T P^T   (A = 16 head dims x 32 keys of the transposed V page)
// so that every lane keeps ONE query row (lane % 16) in both results: the
// running maximum, the sum and the rescaling need no exchange but two
// shuffles across the four lane groups.  The 64 keys of a tile are assigned
// to S's rows so that the probabilities a lane group ends up holding are 8
// consecutive key *slots* of the value page (kv_layout.h), which makes V's
// operand one 16-byte read and lets P stay in registers.  With the chunked
// page layout every operand load of a wave is 1 KB of contiguous memory.
//
//  * fg_attn_split (decode and very short portions, <= 16 rows an item): the
//    key ranges of the items are cut into chunks of equal size (fg_attn_plan,
//    on the device), a chunk is a workgroup whose tiles are dealt to its 4
//    waves, which stream K and V straight from the pages; the chunks' partial
//    (max, sum, O) go to scratch and a combine kernel merges them.
//  * fg_attn_tile (prompt portions, up to 128 rows an item): K and V tiles are
//    staged in LDS and shared by the workgroup's waves.
//
// Semantics as in attention.hip (fastgen/forward.py:176-258).
#include "common.h"
#include "kv_layout.h"
#include "attention_static.h"

#include <stdio.h>

#ifndef FG_HD
#error "compile with -DFG_HD=<head size>"
#endif
static_assert(FG_HD % 16 == 0 && FG_HD >= 16 && FG_HD <= 256, "head size: multiple of 16 up to 256");

constexpr int HD = FG_HD;
constexpr int NKS = (HD + 31) / 32;  // 32-wide steps over the head dimension (last may be half)
constexpr int NDB = HD / 16;         // 16-wide blocks of the head dimension
constexpr int TILE = 64;             // keys per tile

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Bit masks that zero the value slots of keys outside [lo, hi]; slot e of a
// chunk is key ka + (e & 3) + 16 * (e >> 2).  Branch-free, so that it can sit
// between loads without splitting them up.
__device__ __forceinline__ u32x4 slot_mask(int ka, int lo, int hi) {
  u32x4 m;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int k_even = ka + ((2 * w) & 3) + 16 * ((2 * w) >> 2), k_odd = k_even + 1;
    m[w] = ((k_even >= lo && k_even <= hi) ? 0x0000ffffu : 0u) | ((k_odd >= lo && k_odd <= hi) ? 0xffff0000u : 0u);
  }
  return m;
}
__device__ __forceinline__ bf16x8 and_mask(bf16x8 v, u32x4 m) {
  return __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, v) & m);
}

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

#define LOG2E 1.4426950408889634f

// Maximum over the four lanes that hold one query row (lane % 16 in each group of 16), in every one
// of them.  gfx950 swaps rows of 16 and halves of 32 lanes between two registers in the vector unit
// (no trip through the LDS crossbar, whose latency a wave with one or two row blocks cannot hide).
__device__ __forceinline__ float max_over_groups(float v) {
  const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));  // rows 0|1 and 2|3
  const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));  // halves
}

// key (within a tile) of S^T row `row` (0..15) of key block kb (0..3)
__device__ __forceinline__ int key_of(int kb, int row) { return 16 * kb + row; }

// An item: a run of consecutive query tokens of one sequence.
struct Item {
  int seq, tok0, n_tok, pos0;  // sequence, flat index and position of its first token
};
__device__ __forceinline__ Item load_item(const int* items, int i) {
  const int4 v = *(const int4*)(items + 4 * i);
  return Item{v.x, v.y, v.z, v.w};
}

// page lookup without a division when the page size is a power of two
struct Pager {
  const int* table;
  int page_size, shift;
  __device__ __forceinline__ int page_of(int key) const {
    return table[shift >= 0 ? key >> shift : key / page_size];
  }
  __device__ __forceinline__ int in_page(int key) const {
    return shift >= 0 ? key & (page_size - 1) : key % page_size;
  }
};

struct ItemRows {
  int pos;    // position of this lane's query row, -1 for a padding row
  int first;  // first key the row sees
};

// One 64-key tile for one wave, operands given by loader functors.
//   load_k(kb, ks) -> bf16x8 : K[16*kb + lane%16][32*ks + 8*(lane/16) ..+7]
//   load_v(db, ks) -> bf16x8 : V^T[16*db + lane%16][the 8 keys 32*ks + 4g + i, 32*ks + 16 + 4g + i]
//                              with g = lane/16, i = 0..3: the keys of pop[ks]
// PREFETCH: operands come from memory; all of K and half of V are requested
// before anything is computed (more registers).  Otherwise (operands in LDS)
// each is read where it is used.  RB: blocks of 16 query rows a wave holds;
// every K and V operand it reads serves all of them.
// ALLVIS: every row of the wave sees every key of the tile (no mask is computed).
// scale_log2 = scale * log2(e): scores, running maxima and exponents are kept in base 2.
template <bool PREFETCH, int RB, bool ALLVIS, class LK, class LV>
__device__ __forceinline__ void attend_tile(int k0, const ItemRows (&me)[RB], const bf16x8 (&qop)[RB][NKS],
                                            float scale_log2, float (&m)[RB], float (&l)[RB], f32x4 (&o)[RB][NDB],
                                            LK load_k, LV load_v) {
  const int g = (threadIdx.x % FG_WAVE) >> 4;
  // The order of the loads in the source is the order in which they are issued: all of K, then the
  // first half of V, are in flight before the first MFMA waits for anything; the second half of V is
  // issued when K's registers are free and flies during the softmax.
  bf16x8 kop[PREFETCH ? 4 : 1][NKS];
  bf16x8 vop0[PREFETCH ? NDB : 1], vop1[PREFETCH ? NDB : 1];
  if (PREFETCH) {
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) kop[kb][ks] = load_k(kb, ks);
#pragma unroll
    for (int db = 0; db < NDB; ++db) vop0[db] = load_v(db, 0);
  }
  f32x4 s[RB][4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) s[rb][kb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const bf16x8 k = PREFETCH ? kop[kb][ks] : load_k(kb, ks);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        s[rb][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k, qop[rb][ks], s[rb][kb], 0, 0, 0);
    }
  }
  if (PREFETCH) {
#pragma unroll
    for (int db = 0; db < NDB; ++db) vop1[db] = load_v(db, 1);
  }
  bf16x8 pop[RB][2];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = s[rb][kb][i];  // unscaled: the scale is positive, so it commutes with the maximum
        if (!ALLVIS) {
          const int key = k0 + key_of(kb, 4 * g + i);
          // bitwise, not short-circuit: a select, no branch
          v = ((key >= me[rb].first) & (key <= me[rb].pos)) ? v : -INFINITY;
        }
        s[rb][kb][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = max_over_groups(mx);
    const float m_new = fmaxf(m[rb], mx * scale_log2);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
    const float alpha = __builtin_amdgcn_exp2f(m[rb] - m_use);  // m = -inf: 0
    float sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[rb][kb][i], scale_log2, -m_use));
        sum += p;
        pop[rb][kb >> 1][4 * (kb & 1) + i] = (__bf16)p;
      }
    l[rb] = l[rb] * alpha + sum;  // this lane's share of the row's sum; the groups are added at the end
    // once the maxima have settled no row of the wave changes its maximum: nothing to rescale then
    if (__builtin_amdgcn_ballot_w64(m_new != m[rb]) != 0) {
#pragma unroll
      for (int db = 0; db < NDB; ++db) o[rb][db] *= alpha;
    }
    m[rb] = m_new;
  }
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      const bf16x8 v = PREFETCH ? (ks == 0 ? vop0[db] : vop1[db]) : load_v(db, ks);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        o[rb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pop[rb][ks], o[rb][db], 0, 0, 0);
    }
}

// qrow is always a readable row; `valid` says whether it is this lane's
__device__ __forceinline__ void load_q(bf16x8 (&qop)[NKS], const bf16_t* qrow, bool valid) {
  const int g = (threadIdx.x % FG_WAVE) >> 4;
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    const int d = 32 * ks + 8 * g;
    const bf16x8 v = *(const bf16x8*)(qrow + (d < HD ? d : 0));  // loads are never conditional
    qop[ks] = (valid && d < HD) ? v : zero8();
  }
}

// ------------------------------------------------------------------ split
// The key ranges of the items are cut into chunks of the same number of tiles for every item, so that
// a long sequence gives many workgroups and a short one few, each with about the same work; a plan
// kernel does the cutting on the device from the items alone, so that a captured step cuts anew
// for the lengths of every replay.
//
// plan: int32 [4 + 8 * max_chunks]
//   [0] tiles per chunk, [1] chunks in use;
//   from [4] on, 8 ints a chunk, the chunks of an item one after the other: the item's record
//   (sequence, first flat token, tokens, first position), first tile, end tile, chunks of the item
//   (0: this chunk is not in use), number of this chunk among its item's.
#define COMBINE_MAX_SPLITS 256
#define COMBINE_ROWS_MAX_GROUPS 8192  // up to this many workgroups the combine takes a workgroup a row
constexpr int PLAN_HEAD = 4;

// tiles an item's rows see: [t_lo, t_hi]
__device__ __forceinline__ void item_tiles(const Item& it, int window, int& t_lo, int& t_hi) {
  const int pos_last = it.pos0 + it.n_tok - 1;
  const int first_min = window > 0 && it.pos0 - window + 1 > 0 ? it.pos0 - window + 1 : 0;
  t_lo = first_min / TILE;
  t_hi = pos_last / TILE;
}

// One workgroup.  Tiles per chunk: the smallest multiple of min_tiles (at least min_tiles) with which
// all chunks fit into max_chunks (> n_items) whatever the items' lengths are (total / (max_chunks -
// n_items), rounded up) and no item has more than COMBINE_MAX_SPLITS; then, with the number of chunks
// that this gives the longest item, as even as they can be (33 tiles in chunks of 12, 12, 9, not 16,
// 16, 1: sequences of one length are the common case), if the chunks of all items still fit.
__global__ __launch_bounds__(256) void attn_plan_kernel(const int* __restrict__ items, int n_items, int window,
                                                        int max_chunks, int min_tiles, int* __restrict__ plan) {
  __shared__ int red_s[256], red_m[256];
  __shared__ int carry;
  const int tid = threadIdx.x;
  int tot = 0, mx = 0;
  for (int i = tid; i < n_items; i += 256) {
    int lo, hi;
    item_tiles(load_item(items, i), window, lo, hi);
    tot += hi - lo + 1;
    mx = max(mx, hi - lo + 1);
  }
  red_s[tid] = tot;
  red_m[tid] = mx;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (tid < w) {
      red_s[tid] += red_s[tid + w];
      red_m[tid] = max(red_m[tid], red_m[tid + w]);
    }
    __syncthreads();
  }
  tot = red_s[0];
  mx = red_m[0];
  __syncthreads();
  // sum over items of ceil(tiles / ts) <= tot / ts + n_items <= max_chunks
  const int room = max_chunks - n_items;
  int ts = max((tot + room - 1) / room, (mx + COMBINE_MAX_SPLITS - 1) / COMBINE_MAX_SPLITS);
  ts = max(1, (ts + min_tiles - 1) / min_tiles) * min_tiles;
  const int longest_chunks = max(1, (mx + ts - 1) / ts);  // chunks of the longest item
  const int even = max(1, ((mx + longest_chunks - 1) / longest_chunks + min_tiles - 1) / min_tiles) * min_tiles;
  if (even < ts) {  // uniform
    int cnt = 0;
    for (int i = tid; i < n_items; i += 256) {
      int lo, hi;
      item_tiles(load_item(items, i), window, lo, hi);
      cnt += (hi - lo + even) / even;
    }
    red_s[tid] = cnt;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
      if (tid < w) red_s[tid] += red_s[tid + w];
      __syncthreads();
    }
    if (red_s[0] <= max_chunks) ts = even;
    __syncthreads();
  }
  int* chunks = plan + PLAN_HEAD;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int i0 = 0; i0 < n_items; i0 += 256) {
    const int i = i0 + tid;
    Item it{0, 0, 0, 0};
    int lo = 0, hi = -1, c = 0;
    if (i < n_items) {
      it = load_item(items, i);
      item_tiles(it, window, lo, hi);
      c = (hi - lo + ts) / ts;
    }
    // inclusive scan of c over the workgroup
    red_s[tid] = c;
    __syncthreads();
    for (int w = 1; w < 256; w <<= 1) {
      const int add = tid >= w ? red_s[tid - w] : 0;
      __syncthreads();
      red_s[tid] += add;
      __syncthreads();
    }
    const int first = carry + red_s[tid] - c;
    for (int sp = 0; sp < c; ++sp) {
      int* rec = chunks + (size_t)(first + sp) * 8;
      *(int4*)rec = int4{it.seq, it.tok0, it.n_tok, it.pos0};
      *(int4*)(rec + 4) = int4{lo + sp * ts, min(hi + 1, lo + (sp + 1) * ts), c, sp};
    }
    __syncthreads();
    if (tid == 255) carry += red_s[255];
    __syncthreads();
  }
  const int used = carry;
  for (int j = used + tid; j < max_chunks; j += 256) {
    int* rec = chunks + (size_t)j * 8;
    *(int4*)rec = int4{0, 0, 0, 0};
    *(int4*)(rec + 4) = int4{0, 0, 0, 0};
  }
  if (tid == 0) {
    plan[0] = ts;
    plan[1] = used;
  }
}

// grid (n_kv, max_chunks), 256 threads: one chunk of one item (a run of at most 16 rows:
// n_tok * (H / KV) <= 16) for one kv head.  An item of one chunk writes its output rows; of more, the
// chunk's (max, sum, O) go to part_o / part_ml at row (chunk * n_kv + kv head) * 16 + row.
template <bool PERM /* the page's value slots are permuted: page_size % 32 == 0 */>
__global__ __launch_bounds__(256) void attn_split_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_table, int bt_stride, const int* __restrict__ plan,
    float* __restrict__ part_o, float* __restrict__ part_ml, int n_heads, int n_kv, int page_size,
    int page_shift, float scale, int window) {
  __shared__ float o_s[2][16][HD + 1];
  __shared__ float ml_s[2][16][2];
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int r16 = lane & 15, g = lane >> 4;
  const int kvh = blockIdx.x, chunk = blockIdx.y;
  const int G = n_heads / n_kv;
  const int* rec = plan + PLAN_HEAD + (size_t)chunk * 8;
  const int4 rec_a = *(const int4*)rec, rec_b = *(const int4*)(rec + 4);
  if (rec_b.z == 0) return;  // uniform: a chunk that is not in use
  const Item it{rec_a.x, rec_a.y, rec_a.z, rec_a.w};
  const int t_begin = rec_b.x, t_end = rec_b.y;
  const bool alone = rec_b.z == 1;  // the item's only chunk
  const Pager pager{block_table + (size_t)it.seq * bt_stride, page_size, page_shift};
  const KvLayout lay(page_size, HD);

  const int pos_last = it.pos0 + it.n_tok - 1;
  const int first_min = window > 0 && it.pos0 - window + 1 > 0 ? it.pos0 - window + 1 : 0;
  ItemRows me[1] = {{-1, 0}};
  const bool my_row = r16 < it.n_tok * G;
  const int my_tok = my_row ? r16 / G : 0, my_head = my_row ? r16 % G : 0;
  if (my_row) {
    me[0].pos = it.pos0 + my_tok;
    me[0].first = window > 0 && me[0].pos - window + 1 > 0 ? me[0].pos - window + 1 : 0;
  }
  bf16x8 qop[1][NKS];
  load_q(qop[0], q + (size_t)(it.tok0 + my_tok) * q_stride + (size_t)(kvh * G + my_head) * HD, my_row);

  float m_[1] = {-INFINITY}, l_[1] = {0.f};
  f32x4 o_[1][NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) o_[0][db] = f32x4{0.f, 0.f, 0.f, 0.f};

  const size_t head_elems = (size_t)page_size * HD;  // elements of one kv head in a page
  for (int t = t_begin + wave; t < t_end; t += 4) {
    const int k0 = t * TILE;
    // Loads are never conditional (a branch around a load keeps the compiler from issuing the
    // tile's loads together): addresses are clamped into the item's key range and what lies
    // outside is masked afterwards.
    // K chunks of this lane: key 16*kb + r16 of the tile, head dims 32*ks + 8*g
    const bf16_t* kptr[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const int key = min(max(k0 + 16 * kb + r16, first_min), pos_last);  // masked by the scores' select
      kptr[kb] = k_pages + ((size_t)pager.page_of(key) * n_kv + kvh) * head_elems +
                 lay.k_off(pager.in_page(key), 8 * g);
    }
    // V chunks of this lane: keys 32*ks + 4*g + (0..3) and 16 more on; head dim 16*db + r16
    const bf16_t* vptr[2][2];
    u32x4 vmask[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int ka = k0 + 32 * ks + 4 * g, kb2 = ka + 16;
      vmask[ks] = slot_mask(ka, first_min, pos_last);  // what lies outside may hold anything, NaN included
      const bool in_a = ka + 3 >= first_min && ka <= pos_last;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        // a key of the wanted run if it has one in range, else any key in range
        const int want = (half == 0 && (in_a || !PERM)) ? ka : kb2;
        const int x = min(max(want, first_min), pos_last);
        const int xin = pager.in_page(x);
        const int back = PERM ? (lay.v_slot(xin) & 7) : (xin & 3);  // to the start of the chunk / run of 4
        vptr[ks][half] = v_pages + ((size_t)pager.page_of(x) * n_kv + kvh) * head_elems + lay.v_off(xin, r16) - back;
      }
    }
    const size_t k_step = lay.k_step32(), v_step = lay.v_step_block();
    auto load_k = [&](int kb, int ks) -> bf16x8 {
      const bool in = 32 * ks + 8 * g < HD;
      const bf16x8 v = *(const bf16x8*)(kptr[kb] + (in ? ks * k_step : 0));
      return in ? v : zero8();
    };
    auto load_v = [&](int db, int ks) -> bf16x8 {
      bf16x8 v;
      if (PERM) {
        v = *(const bf16x8*)(vptr[ks][0] + db * v_step);
      } else {
        const bf16x4 lo = *(const bf16x4*)(vptr[ks][0] + db * v_step);
        const bf16x4 hi = *(const bf16x4*)(vptr[ks][1] + db * v_step);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = lo[e];
          v[4 + e] = hi[e];
        }
      }
      return and_mask(v, vmask[ks]);
    };
    attend_tile<true, 1, false>(k0, me, qop, scale * LOG2E, m_, l_, o_, load_k, load_v);
  }
  float m = m_[0], l = l_[0];
  f32x4(&o)[NDB] = o_[0];
  l += __shfl_xor(l, 16, FG_WAVE);
  l += __shfl_xor(l, 32, FG_WAVE);

  // ---- merge the 4 waves pairwise in registers: 2,3 -> 0,1 then 1 -> 0
  auto put = [&](int slot) {
    if (g == 0) {
      ml_s[slot][r16][0] = m;
      ml_s[slot][r16][1] = l;
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) o_s[slot][r16][16 * db + 4 * g + i] = o[db][i];
  };
  auto take = [&](int slot) {
    const float mo = ml_s[slot][r16][0], lo = ml_s[slot][r16][1];
    const float M = fmaxf(m, mo);
    const float fs = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - M);  // maxima are in base 2
    const float fo = mo == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mo - M);
    l = fs * l + fo * lo;
    m = M;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[db][i] = fs * o[db][i] + fo * o_s[slot][r16][16 * db + 4 * g + i];
  };
  if (wave >= 2) put(wave - 2);
  __syncthreads();
  if (wave < 2) take(wave);
  __syncthreads();
  if (wave == 1) put(0);
  __syncthreads();
  if (wave != 0) return;
  take(0);
  if (r16 >= it.n_tok * G) return;
  const int t_out = it.tok0 + r16 / G, h_out = kvh * G + r16 % G;
  if (alone) {
    bf16_t* orow = out + (size_t)t_out * out_stride + (size_t)h_out * HD;
    const float inv = 1.f / l;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      bf16x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = (__bf16)(o[db][i] * inv);
      *(bf16x4*)(orow + 16 * db + 4 * g) = v;
    }
  } else {
    const size_t row = ((size_t)chunk * n_kv + kvh) * 16 + r16;
#pragma unroll
    for (int db = 0; db < NDB; ++db) *(f32x4*)(part_o + row * HD + 16 * db + 4 * g) = o[db];
    if (g == 0) {
      part_ml[row * 2] = m;
      part_ml[row * 2 + 1] = l;
    }
  }
}

// Two kernels add up the chunks of the items that have several, in chunk order: the workgroups of an
// item's first chunk do it, all others leave as soon as they have their chunk's record (a wave that
// has asked for more has to wait for it before it can end, and most workgroups of a step of
// sequences of one length are of this kind).  Both are chains of dependent reads, so what they cost
// is how long that chain is and how many workgroups there are to start.
//
// For short chunk lists (a few sequences): grid (16 rows, n_kv, max_chunks), one thread per head
// dimension (at least one wave), a workgroup a row.  The chunks' maxima and sums are read by the first
// wave, one chunk a lane, together with the first eight partial outputs.
__global__ void attn_combine_rows_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                    const int* __restrict__ plan, bf16_t* __restrict__ out, int out_stride,
                                    int n_heads, int n_kv) {
  __shared__ float f_s[COMBINE_MAX_SPLITS];  // weight of each chunk's partial output: 2^(m_s - M) / L
  const int r = blockIdx.x, kvh = blockIdx.y, chunk = blockIdx.z, d = threadIdx.x;
  const int G = n_heads / n_kv;
  const int* rec = plan + PLAN_HEAD + (size_t)chunk * 8;
  const int4 rec_a = *(const int4*)rec, rec_b = *(const int4*)(rec + 4);
  const int n_splits = rec_b.z;
  if (n_splits <= 1 || rec_b.w != 0) return;  // uniform: not in use, or written by the split kernel, or not the first
  const Item it{rec_a.x, rec_a.y, rec_a.z, rec_a.w};
  if (r >= it.n_tok * G) return;  // uniform: a row beyond the item, its partial results are never written
  const size_t row0 = ((size_t)chunk * n_kv + kvh) * 16 + r, step = (size_t)n_kv * 16;  // rows from chunk to chunk
  const int dc = min(d, HD - 1);
  float first_o[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) first_o[u] = part_o[(row0 + (size_t)min(u, n_splits - 1) * step) * HD + dc];
  if (threadIdx.x < FG_WAVE) {
    constexpr int PER = COMBINE_MAX_SPLITS / FG_WAVE;
    float ms[PER], ls[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int sp = threadIdx.x + j * FG_WAVE;
      const float2 ml = *(const float2*)(part_ml + (row0 + (size_t)min(sp, n_splits - 1) * step) * 2);
      ms[j] = sp < n_splits ? ml.x : -INFINITY;  // maxima are in base 2
      ls[j] = ml.y;
    }
    float M = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; ++j) M = fmaxf(M, ms[j]);
    M = wave_max(M);
    float L = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      ms[j] = ms[j] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms[j] - M);
      L += ms[j] * ls[j];
    }
    L = wave_sum(L);
    const float inv = 1.f / L;
#pragma unroll
    for (int j = 0; j < PER; ++j) f_s[threadIdx.x + j * FG_WAVE] = ms[j] * inv;
  }
  __syncthreads();
  if (d >= HD) return;
  float O = 0.f;
#pragma unroll
  for (int u = 0; u < 8; ++u) O += u < n_splits ? f_s[u] * first_o[u] : 0.f;
  for (int s0 = 8; s0 < n_splits; s0 += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = part_o[(row0 + (size_t)min(s0 + u, n_splits - 1) * step) * HD + d];
#pragma unroll
    for (int u = 0; u < 8; ++u) O += s0 + u < n_splits ? f_s[s0 + u] * v[u] : 0.f;
  }
  const int t = it.tok0 + r / G, h = kvh * G + r % G;
  out[(size_t)t * out_stride + (size_t)h * HD + d] = (bf16_t)O;
}

// For long chunk lists (many sequences; sixteen times fewer workgroups): grid (n_kv, max_chunks), 256
// threads, a workgroup for the 16 rows x HD of a kv head.  Wave w weighs rows 4w .. 4w+3, one chunk a
// lane; then every thread adds up four neighbouring head dimensions of a row (or of several rows).
__global__ __launch_bounds__(256) void attn_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ plan,
    bf16_t* __restrict__ out, int out_stride, int n_heads, int n_kv) {
  __shared__ float f_s[16][COMBINE_MAX_SPLITS];  // weight of each chunk's partial output: 2^(m_s - M) / L
  const int kvh = blockIdx.x, chunk = blockIdx.y, tid = threadIdx.x;
  const int lane = tid % FG_WAVE, wave = tid / FG_WAVE;
  const int G = n_heads / n_kv;
  const int* rec = plan + PLAN_HEAD + (size_t)chunk * 8;
  const int4 rec_a = *(const int4*)rec, rec_b = *(const int4*)(rec + 4);
  const int n_splits = rec_b.z;
  if (n_splits <= 1 || rec_b.w != 0) return;  // uniform: not in use, or written by the split kernel, or not the first
  const Item it{rec_a.x, rec_a.y, rec_a.z, rec_a.w};
  constexpr int V4 = 4 * HD;             // float4s of one chunk's 16 x HD partial output
  constexpr int NV = (V4 + 255) / 256;   // of them a thread adds up
  constexpr int AHEAD = 4;               // chunks whose partial outputs are requested together with the statistics
  const size_t rows0 = ((size_t)chunk * n_kv + kvh) * 16, step = (size_t)n_kv * 16;  // rows from chunk to chunk
  f32x4 first_o[AHEAD][NV];
#pragma unroll
  for (int u = 0; u < AHEAD; ++u)
#pragma unroll
    for (int j = 0; j < NV; ++j)
      first_o[u][j] = *(const f32x4*)(part_o + (rows0 + (size_t)min(u, n_splits - 1) * step) * HD +
                                      (size_t)min(tid + 256 * j, V4 - 1) * 4);
  constexpr int PER = COMBINE_MAX_SPLITS / FG_WAVE;
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    float ms[PER], ls[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int sp = lane + j * FG_WAVE;
      const float2 ml = *(const float2*)(part_ml + (rows0 + 4 * wave + rr + (size_t)min(sp, n_splits - 1) * step) * 2);
      ms[j] = sp < n_splits ? ml.x : -INFINITY;  // maxima are in base 2
      ls[j] = ml.y;
    }
    float M = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; ++j) M = fmaxf(M, ms[j]);
    M = wave_max(M);
    float L = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      ms[j] = ms[j] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms[j] - M);
      L += ms[j] * ls[j];
    }
    L = wave_sum(L);
    const float inv = 1.f / L;  // (a row beyond the item's: never stored)
#pragma unroll
    for (int j = 0; j < PER; ++j) f_s[4 * wave + rr][lane + j * FG_WAVE] = ms[j] * inv;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = tid + 256 * j;
    if (idx >= V4) break;
    const int r = (4 * idx) / HD, d = (4 * idx) % HD;
    if (r >= it.n_tok * G) continue;  // a row beyond the item: its partial results are never written
    f32x4 O = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < AHEAD; ++u)
      if (u < n_splits) O += f_s[r][u] * first_o[u][j];
    for (int s0 = AHEAD; s0 < n_splits; s0 += 8) {
      f32x4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        v[u] = *(const f32x4*)(part_o + (rows0 + (size_t)min(s0 + u, n_splits - 1) * step) * HD + (size_t)idx * 4);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < n_splits) O += f_s[r][s0 + u] * v[u];
    }
    const int t = it.tok0 + r / G, h = kvh * G + r % G;
    bf16x4 o4;
#pragma unroll
    for (int i = 0; i < 4; ++i) o4[i] = (__bf16)O[i];
    *(bf16x4*)(out + (size_t)t * out_stride + (size_t)h * HD + d) = o4;
  }
}

static int page_shift_of(int page_size) {
  for (int s = 3; s < 31; ++s)
    if ((1 << s) == page_size) return s;
  return -1;
}

// ints of a plan of max_chunks chunks
extern "C" long long fg_attn_plan_ints(int max_chunks) { return PLAN_HEAD + 8LL * max_chunks; }

// Cuts the items (int32 [n_items][4], 16-byte aligned) into chunks: see the layout of `plan` above.
// max_chunks >= 2 * n_items; min_tiles: a chunk's tiles are a multiple of it (4: one tile a wave).
extern "C" int fg_attn_plan(const int* items, int n_items, int window, int max_chunks, int min_tiles, int* plan,
                            hipStream_t stream) {
  if (n_items <= 0) return FG_OK;
  if (!items || !plan || max_chunks < 2 * n_items || min_tiles < 1 || window < 0) return FG_ERR_ARG;
  attn_plan_kernel<<<1, 256, 0, stream>>>(items, n_items, window, max_chunks, min_tiles, plan);
  return fg_launch_status();
}

// plan: what fg_attn_plan made of the items, with the same n_items, max_chunks and window.
// max_rows: no item has more rows (tokens x heads of a kv head's group) than this, at most 16.
// part_o: fp32 [max_chunks * n_kv * 16 * HD], part_ml: the same rows x 2.
extern "C" int fg_attn_split(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                             const void* v_pages, const int* block_table, int bt_stride, const int* plan,
                             int n_items, int max_chunks, int max_rows, float* part_o, float* part_ml,
                             int n_heads, int n_kv, int hd, int page_size, float scale, int window,
                             hipStream_t stream) {
  if (n_items <= 0) return FG_OK;
  if (hd != HD || n_kv <= 0 || n_heads % n_kv || n_heads / n_kv > 16 || page_size < 8 || page_size % 8 ||
      !(scale > 0.f) || max_chunks < 2 * n_items || max_chunks > 65535 || n_kv > 65535 || window < 0 ||
      q_stride % 8 || out_stride % 4 || !plan || !part_o || !part_ml || max_rows < 1 || max_rows > 16)
    return FG_ERR_ARG;
#define LAUNCH(PERM)                                                                                           \
  attn_split_kernel<PERM><<<dim3(n_kv, max_chunks), 256, 0, stream>>>(                                         \
      (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,    \
      block_table, bt_stride, plan, part_o, part_ml, n_heads, n_kv, page_size,                                 \
      page_shift_of(page_size), scale, window)
  if (page_size % 32 == 0) LAUNCH(true); else LAUNCH(false);
#undef LAUNCH
  if ((long long)max_chunks * n_kv * max_rows <= COMBINE_ROWS_MAX_GROUPS)
    attn_combine_rows_kernel<<<dim3(max_rows, n_kv, max_chunks), HD < 64 ? 64 : HD, 0, stream>>>(
        part_o, part_ml, plan, (bf16_t*)out, out_stride, n_heads, n_kv);
  else
    attn_combine_kernel<<<dim3(n_kv, max_chunks), 256, 0, stream>>>(
        part_o, part_ml, plan, (bf16_t*)out, out_stride, n_heads, n_kv);
  return fg_launch_status();
}

// ----------------------------------------------------------- without allocation
// The plan, part_o and part_ml of a call live in this array (see attention_static.h).  In host code
// the array's name is only a handle for hipGetSymbolAddress: each GPU has its own copy at its own
// address, looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[FG_ATTN_STATIC_BYTES];

constexpr int STATIC_MAX_DEVICES = 64;
static unsigned char* scratch_ptr[STATIC_MAX_DEVICES];  // the array's address on each device, once known
static thread_local char static_error[256] = "";

extern "C" const char* fg_attn_decode_static_error() { return static_error; }

// bytes of scratch for max_chunks chunks: the plan (rounded up to 256 bytes), then part_o, then part_ml
static size_t static_plan_bytes(int max_chunks) {
  return (((size_t)(PLAN_HEAD + 8LL * max_chunks) * sizeof(int)) + 255) / 256 * 256;
}
static size_t static_bytes(int max_chunks, int n_kv) {
  return static_plan_bytes(max_chunks) + (size_t)max_chunks * n_kv * 16 * (HD + 2) * sizeof(float);
}

extern "C" int fg_attn_decode_static_max_chunks(int n_kv) {
  if (n_kv <= 0) return 0;
  int lo = 0, hi = 65535;  // the largest count whose scratch fits
  while (lo < hi) {
    const int mid = (lo + hi + 1) / 2;
    if (static_bytes(mid, n_kv) <= FG_ATTN_STATIC_BYTES) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// The address of `scratch` on the current device (nullptr, with the reason in static_error, if it
// cannot be had).
static unsigned char* static_scratch() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) {
    snprintf(static_error, sizeof static_error, "fg_attn_decode_static: no current device (%s, device %d)",
             hipGetErrorString(e), dev);
    return nullptr;
  }
  unsigned char* p = __atomic_load_n(&scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (p) return p;
  e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p) {
    snprintf(static_error, sizeof static_error, "fg_attn_decode_static: hipGetSymbolAddress failed on device %d: %s",
             dev, hipGetErrorString(e));
    return nullptr;
  }
  __atomic_store_n(&scratch_ptr[dev], p, __ATOMIC_RELEASE);  // every thread finds the same address
  return p;
}

extern "C" int fg_attn_decode_static(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                                     const void* v_pages, const int* block_table, int bt_stride, const int* items,
                                     int n_items, int max_chunks, int min_tiles, int max_rows, int n_heads,
                                     int n_kv, int hd, int page_size, float scale, int window,
                                     hipStream_t stream) {
  static_error[0] = 0;
  if (n_items <= 0) return FG_OK;
  if (n_kv <= 0 || max_chunks < 2 * n_items || static_bytes(max_chunks, n_kv) > FG_ATTN_STATIC_BYTES) {
    snprintf(static_error, sizeof static_error,
             "fg_attn_decode_static: %d items in %d chunks for %d kv heads of size %d need %zu bytes of scratch, "
             "the static array holds %u (at most %d chunks, half as many items)",
             n_items, max_chunks, n_kv, HD, n_kv > 0 ? static_bytes(max_chunks, n_kv) : (size_t)0,
             FG_ATTN_STATIC_BYTES, fg_attn_decode_static_max_chunks(n_kv));
    return n_kv > 0 && max_chunks >= 2 * n_items ? FG_ERR_SCRATCH : FG_ERR_ARG;
  }
  unsigned char* base = static_scratch();
  if (!base) return FG_ERR_SCRATCH;
  int* plan = (int*)base;
  float* part_o = (float*)(base + static_plan_bytes(max_chunks));
  float* part_ml = part_o + (size_t)max_chunks * n_kv * 16 * HD;
  int st = fg_attn_plan(items, n_items, window, max_chunks, min_tiles, plan, stream);
  if (st == FG_OK)
    st = fg_attn_split(q, q_stride, out, out_stride, k_pages, v_pages, block_table, bt_stride, plan, n_items,
                       max_chunks, max_rows, part_o, part_ml, n_heads, n_kv, hd, page_size, scale, window, stream);
  if (st != FG_OK)
    snprintf(static_error, sizeof static_error, "fg_attn_decode_static: %s",
             st == FG_ERR_ARG ? "an argument that the kernels cannot take" : "a kernel launch failed");
  return st;
}

// ------------------------------------------------------------------- tile
// One workgroup per (item, kv head); an item has at most TILE_ROWS / (H / KV) tokens.  The K and
// V tiles go through LDS in the order the operands are read: K [4 key blocks][HD/8 chunks]
// [16 keys][8], V [HD/16 dim blocks][8 key chunks][16 dims][8 slots] (slots as in the permuted page).
//
// Up to head size 128: 8 waves and two tiles at a time.  Four row groups of 32 rows (two blocks of
// 16 a wave, every K and V operand read serves both); the two waves of a row group take the even
// and the odd tiles and merge their (max, sum, O) at the end.  The last rows of a long prompt see
// every tile, one after the other: with two waves on them that chain is half as long, and a
// compute unit holds one workgroup whose eight waves all work until its end.  Workgroups are
// launched in the order of the items (most keys first), so short ones fill in behind long ones.
// Above 128: 4 waves of 16 rows, one tile at a time (two tiles would not fit the 64 KB of LDS).
// The second form also serves head sizes up to 128 when a step has few items ("small" items of 64 rows:
// twice as many workgroups of half the size, several to a compute unit, out of step with one another).
constexpr bool TILE_PAIR_OK = HD <= 128;
constexpr int TILE_ROWS = TILE_PAIR_OK ? 128 : 64;   // query rows of an item of the first form that this head size has
constexpr int TILE_ROWS_SMALL = 64;                // of the second form

template <bool PERM, bool TILE_PAIR>
__global__ __launch_bounds__(TILE_PAIR ? 512 : 256, TILE_PAIR ? 1 : 2) void attn_tile_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_table, int bt_stride, const int* __restrict__ items, int n_heads, int n_kv,
    int page_size, int page_shift, float scale, int window) {
  constexpr int TILE_RB = TILE_PAIR ? 2 : 1;  // row blocks a wave holds
  constexpr int TILE_THREADS = TILE_PAIR ? 512 : 256;
  constexpr int NT = TILE_THREADS;
  constexpr int NPT = TILE_PAIR ? 2 : 1;    // tiles a pass of the loop takes
  // tiles in LDS: with pairs, one pair is read while the next is written (128 KB at head size 128, of
  // the CU's 160 KB: the workgroup has the CU to itself anyway; measured 4 % faster than two slots)
  constexpr int NSLOT = TILE_PAIR ? 4 : 1;
  __shared__ __attribute__((aligned(16))) bf16_t k_lds[NSLOT][TILE * HD];
  __shared__ __attribute__((aligned(16))) bf16_t v_lds[NSLOT][TILE * HD];
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int r16 = lane & 15, g = lane >> 4;
  const int rg = wave & 3;    // row group
  const int par = wave >> 2;  // which tile of a pair this wave takes (0 when tiles come one at a time)
  const int item = blockIdx.x / n_kv, kvh = blockIdx.x % n_kv;
  const int G = n_heads / n_kv;
  const Item it = load_item(items, item);
  const Pager pager{block_table + (size_t)it.seq * bt_stride, page_size, page_shift};
  const KvLayout lay(page_size, HD);
  const int pos_last = it.pos0 + it.n_tok - 1;
  const int first_min = window > 0 && it.pos0 - window + 1 > 0 ? it.pos0 - window + 1 : 0;

  constexpr int RB = TILE_RB;
  ItemRows me[RB];
  bf16x8 qop[RB][NKS];
  int w_hi = -1, w_lo = 0x7fffffff;  // the keys this wave's rows can see: tiles outside are skipped by the wave
  int w_all_hi = 0x7fffffff, w_all_lo = 0;  // keys in [w_all_lo, w_all_hi] are seen by all rows of the wave
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = (rg * RB + rb) * 16 + r16;
    const bool my_row = row < it.n_tok * G;
    const int my_tok = my_row ? row / G : 0, my_head = my_row ? row % G : 0;
    me[rb] = ItemRows{-1, 0};
    if (my_row) {
      me[rb].pos = it.pos0 + my_tok;
      me[rb].first = window > 0 && me[rb].pos - window + 1 > 0 ? me[rb].pos - window + 1 : 0;
      w_hi = max(w_hi, me[rb].pos);
      w_lo = min(w_lo, me[rb].first);
      w_all_hi = min(w_all_hi, me[rb].pos);
      w_all_lo = max(w_all_lo, me[rb].first);
    } else {
      w_all_hi = -1;  // a padding row sees nothing: no tile is all visible
    }
    load_q(qop[rb], q + (size_t)(it.tok0 + my_tok) * q_stride + (size_t)(kvh * G + my_head) * HD, my_row);
  }
#pragma unroll
  for (int msk = 1; msk < 16; msk <<= 1) {
    w_hi = max(w_hi, __shfl_xor(w_hi, msk, FG_WAVE));
    w_lo = min(w_lo, __shfl_xor(w_lo, msk, FG_WAVE));
    w_all_hi = min(w_all_hi, __shfl_xor(w_all_hi, msk, FG_WAVE));
    w_all_lo = max(w_all_lo, __shfl_xor(w_all_lo, msk, FG_WAVE));
  }

  float m[RB], l[RB];
  f32x4 o[RB][NDB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    m[rb] = -INFINITY;
    l[rb] = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[rb][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const size_t head_elems = (size_t)page_size * HD;
  constexpr int KCH = HD / 8;                  // 16-byte chunks in a key
  constexpr int KTOT = TILE * KCH, VTOT = NDB * 8 * 16;  // chunks of a K tile, of a V tile
  constexpr int KN = (KTOT + NT - 1) / NT;     // K chunks a thread copies per tile
  constexpr int VN = (VTOT + NT - 1) / NT;     // V chunks a thread copies per tile
  bf16x8 kreg[KN], vreg[VN];
  // A tile's chunks on their way through registers.  Loads are never conditional within a tile:
  // addresses are clamped into the item's key range, value slots outside it are masked, keys
  // outside it give scores that the select discards.
  auto fetch = [&](int k0, bf16x8(&kr)[KN], bf16x8(&vr)[VN]) {
    if (PERM && (page_size & 63) == 0 && k0 >= first_min && k0 + TILE - 1 <= pos_last) {
      // The whole tile lies in one page and inside the key range: K's four 16-key blocks are 64*HD
      // contiguous elements in the order LDS wants them, V's eight key chunks are a contiguous run
      // per block of 16 head dims.  No masks, one page lookup.
      const int kin = pager.in_page(k0);
      const bf16_t* base_k = k_pages + ((size_t)pager.page_of(k0) * n_kv + kvh) * head_elems + (size_t)kin * HD;
      const bf16_t* base_v = v_pages + ((size_t)pager.page_of(k0) * n_kv + kvh) * head_elems + (size_t)(kin >> 3) * 128;
      const size_t v_block = (size_t)(page_size >> 3) * 128;  // elements of one block of 16 head dims
#pragma unroll
      for (int j = 0; j < KN; ++j) {
        const int w = min((int)threadIdx.x + NT * j, KTOT - 1);
        kr[j] = *(const bf16x8*)(base_k + (size_t)w * 8);
      }
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        const int w = min((int)threadIdx.x + NT * j, VTOT - 1);
        vr[j] = *(const bf16x8*)(base_v + (size_t)(w >> 7) * v_block + (size_t)(w & 127) * 8);
      }
      return;
    }
    // K: chunk (block kb, dims 8c.., key r) -> k_s[((kb*KCH + c)*16 + r)*8]; r fastest over threads
#pragma unroll
    for (int j = 0; j < KN; ++j) {
      const int w = min((int)threadIdx.x + NT * j, KTOT - 1);  // beyond the tile: a copy that is not stored
      const int r = w & 15, c = (w >> 4) % KCH, kb = (w >> 4) / KCH;
      const int key = min(max(k0 + 16 * kb + r, first_min), pos_last);
      kr[j] = *(const bf16x8*)(k_pages + ((size_t)pager.page_of(key) * n_kv + kvh) * head_elems +
                               lay.k_off(pager.in_page(key), 8 * c));
    }
    // V: chunk (dim block db, key chunk kc = 4*ks + gg, dim r) -> v_s[((db*8 + kc)*16 + r)*8];
    // its slots are keys 32*ks + 4*gg + (0..3) and 16 more on
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      const int w = min((int)threadIdx.x + NT * j, VTOT - 1);
      const int r = w & 15, kc = (w >> 4) & 7, db = w >> 7;
      const int ka = k0 + 32 * (kc >> 2) + 4 * (kc & 3), kb2 = ka + 16;
      const bool in_a = ka + 3 >= first_min && ka <= pos_last;
      const bf16_t* src[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int want = (half == 0 && (in_a || !PERM)) ? ka : kb2;
        const int x = min(max(want, first_min), pos_last);
        const int xin = pager.in_page(x);
        const int back = PERM ? (lay.v_slot(xin) & 7) : (xin & 3);
        src[half] = v_pages + ((size_t)pager.page_of(x) * n_kv + kvh) * head_elems + lay.v_off(xin, 16 * db + r) - back;
      }
      bf16x8 v;
      if (PERM) {
        v = *(const bf16x8*)src[0];
      } else {
        const bf16x4 lo = *(const bf16x4*)src[0], hi = *(const bf16x4*)src[1];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = lo[e];
          v[4 + e] = hi[e];
        }
      }
      vr[j] = and_mask(v, slot_mask(ka, first_min, pos_last));
    }
  };
  auto stash = [&](int b, const bf16x8(&kr)[KN], const bf16x8(&vr)[VN]) {
#pragma unroll
    for (int j = 0; j < KN; ++j)
      if (threadIdx.x + NT * j < KTOT) *(bf16x8*)(k_lds[b] + (size_t)(threadIdx.x + NT * j) * 8) = kr[j];
#pragma unroll
    for (int j = 0; j < VN; ++j)
      if (threadIdx.x + NT * j < VTOT) *(bf16x8*)(v_lds[b] + (size_t)(threadIdx.x + NT * j) * 8) = vr[j];
  };
  auto compute = [&](int k0, int b) {
    if (k0 > w_hi || k0 + TILE <= w_lo) return;  // nothing in this tile for this wave's rows
    const bf16_t* k_s = k_lds[b];
    const bf16_t* v_s = v_lds[b];
    auto load_k = [&](int kb, int ks) -> bf16x8 {
      const int c = 4 * ks + g;
      return c < KCH ? *(const bf16x8*)(k_s + ((kb * KCH + c) * 16 + r16) * 8) : zero8();
    };
    auto load_v = [&](int db, int ks) -> bf16x8 {
      return *(const bf16x8*)(v_s + ((db * 8 + 4 * ks + g) * 16 + r16) * 8);
    };
    if (k0 >= w_all_lo && k0 + TILE - 1 <= w_all_hi)  // uniform over the wave
      attend_tile<false, RB, true>(k0, me, qop, scale * LOG2E, m, l, o, load_k, load_v);
    else
      attend_tile<false, RB, false>(k0, me, qop, scale * LOG2E, m, l, o, load_k, load_v);
  };
  const int k_first = (first_min / TILE) * TILE;
  constexpr int STEP = NPT * TILE;  // keys per pass of the loop
  if (NSLOT == 2 * NPT) {
    // Pass i is read from its slots while pass i+1 arrives in the other slots: one barrier a pass.
    // A tile that is one whole page inside the key range goes from memory straight into LDS (a
    // lane's 16 bytes land at the wave's base + 16 * lane: the order the copy through registers
    // stores them in, too) and costs neither registers nor instructions; the tiles at the edges
    // of the range go through registers, where they are masked.
    // page: the page of key k0, looked up a pass earlier so that nobody waits for the table here
    auto page_ahead = [&](int k0) { return pager.page_of(min(k0, pos_last)); };
    auto bring = [&](int k0, int slot, int page) {
      if (k0 > pos_last) return;  // uniform
      if (PERM && (page_size & 63) == 0 && k0 >= first_min && k0 + TILE - 1 <= pos_last) {
        const int kin = pager.in_page(k0);
        const bf16_t* base_k = k_pages + ((size_t)page * n_kv + kvh) * head_elems + (size_t)kin * HD;
        const bf16_t* base_v = v_pages + ((size_t)page * n_kv + kvh) * head_elems + (size_t)(kin >> 3) * 128;
        const size_t v_block = (size_t)(page_size >> 3) * 128;
#pragma unroll
        for (int j = 0; j < KN; ++j) {
          const int w = threadIdx.x + NT * j;
          if (w < KTOT)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base_k + (size_t)w * 8),
                                             (__attribute__((address_space(3))) void*)(k_lds[slot] + (size_t)(w - lane) * 8),
                                             16, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < VN; ++j) {
          const int w = threadIdx.x + NT * j;
          if (w < VTOT)
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(base_v + (size_t)(w >> 7) * v_block + (size_t)(w & 127) * 8),
                (__attribute__((address_space(3))) void*)(v_lds[slot] + (size_t)(w - lane) * 8), 16, 0, 0);
        }
      } else {
        fetch(k0, kreg, vreg);
        stash(slot, kreg, vreg);
      }
    };
    int page_a = page_ahead(k_first + STEP), page_b = page_ahead(k_first + STEP + TILE);
    bring(k_first, 0, page_ahead(k_first));
    bring(k_first + TILE, 1, page_ahead(k_first + TILE));
    int s0 = 0;
    for (int k0 = k_first; k0 <= pos_last; k0 += STEP, s0 ^= NPT) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of pass k0 has landed in LDS
      __syncthreads();  // pass k0 is complete in its slots; nobody reads the other slots any more
      bring(k0 + STEP, s0 ^ NPT, page_a);
      bring(k0 + STEP + TILE, (s0 ^ NPT) + 1, page_b);
      page_a = page_ahead(k0 + 2 * STEP);
      page_b = page_ahead(k0 + 2 * STEP + TILE);
      const int mine = k0 + par * TILE;
      if (mine <= pos_last) compute(mine, s0 + par);
    }
  } else {
    // one tile at a time: the next tile's chunks fly into registers during this tile's MFMAs
    fetch(k_first, kreg, vreg);
    for (int k0 = k_first; k0 <= pos_last; k0 += STEP) {
      __syncthreads();  // the previous tile is no longer read
      stash(0, kreg, vreg);
      __syncthreads();
      if (k0 + STEP <= pos_last) fetch(k0 + STEP, kreg, vreg);
      compute(k0, 0);
    }
  }
  if (TILE_PAIR) {
    // the odd tiles' wave hands its (max, sum, O) to the even tiles' wave of the same rows, one row
    // block at a time, through the tiles' LDS; both waves hold the same rows in the same lanes
    float* o_x = (float*)&k_lds[0][0];   // [4 row groups][NDB][64 lanes][4]
    float* ml_x = (float*)&v_lds[0][0];  // [4 row groups][64 lanes][2]
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      __syncthreads();  // the tiles (or the previous row block) are no longer read
      if (par == 1) {
#pragma unroll
        for (int db = 0; db < NDB; ++db) *(f32x4*)(o_x + ((size_t)(rg * NDB + db) * FG_WAVE + lane) * 4) = o[rb][db];
        ml_x[(rg * FG_WAVE + lane) * 2] = m[rb];
        ml_x[(rg * FG_WAVE + lane) * 2 + 1] = l[rb];
      }
      __syncthreads();
      if (par == 0) {
        const float mo = ml_x[(rg * FG_WAVE + lane) * 2], lo = ml_x[(rg * FG_WAVE + lane) * 2 + 1];
        const float M = fmaxf(m[rb], mo);
        const float fs = m[rb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[rb] - M);
        const float fo = mo == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mo - M);
        l[rb] = fs * l[rb] + fo * lo;
        m[rb] = M;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          const f32x4 other = *(const f32x4*)(o_x + ((size_t)(rg * NDB + db) * FG_WAVE + lane) * 4);
          o[rb][db] = fs * o[rb][db] + fo * other;
        }
      }
    }
    if (par == 1) return;
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float lsum = l[rb];
    lsum += __shfl_xor(lsum, 16, FG_WAVE);
    lsum += __shfl_xor(lsum, 32, FG_WAVE);
    const int row = (rg * RB + rb) * 16 + r16;
    if (row < it.n_tok * G) {
      bf16_t* orow = out + (size_t)(it.tok0 + row / G) * out_stride + (size_t)(kvh * G + row % G) * HD;
      const float inv = 1.f / lsum;
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (__bf16)(o[rb][db][i] * inv);
        *(bf16x4*)(orow + 16 * db + 4 * g) = v;
      }
    }
  }
}

struct TileArgs {
  const bf16_t* q; int q_stride; bf16_t* out; int out_stride; const bf16_t* k_pages; const bf16_t* v_pages;
  const int* block_table; int bt_stride; const int* items; int n_items, n_heads, n_kv, page_size; float scale;
  int window; hipStream_t stream;
};
template <bool PERM, bool PAIR>
static void launch_tile(const TileArgs& a) {
  attn_tile_kernel<PERM, PAIR><<<a.n_items * a.n_kv, PAIR ? 512 : 256, 0, a.stream>>>(
      a.q, a.q_stride, a.out, a.out_stride, a.k_pages, a.v_pages, a.block_table, a.bt_stride, a.items, a.n_heads,
      a.n_kv, a.page_size, page_shift_of(a.page_size), a.scale, a.window);
}
// the form with two tiles at a time exists up to head size 128 only (its LDS)
template <bool EXISTS> struct PairForm {
  static void go(const TileArgs& a) {
    if (a.page_size % 32 == 0) launch_tile<true, true>(a); else launch_tile<false, true>(a);
  }
};
template <> struct PairForm<false> { static void go(const TileArgs&) {} };

// item_rows: the rows an item has at most, fg_attn_tile_rows(0) or fg_attn_tile_rows(1): which form of the kernel runs.
extern "C" int fg_attn_tile(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                            const void* v_pages, const int* block_table, int bt_stride, const int* items,
                            int n_items, int item_rows, int n_heads, int n_kv, int hd, int page_size, float scale,
                            int window, hipStream_t stream) {
  if (n_items <= 0) return FG_OK;
  if (hd != HD || !(scale > 0.f) || n_kv <= 0 || n_heads % n_kv || n_heads / n_kv > item_rows || page_size < 8 || page_size % 8 ||
      (long long)n_items * n_kv > 2147483647LL || window < 0 || q_stride % 8 || out_stride % 4 ||
      (item_rows != TILE_ROWS && item_rows != TILE_ROWS_SMALL))
    return FG_ERR_ARG;
  const TileArgs a{(const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,
                   block_table, bt_stride, items, n_items, n_heads, n_kv, page_size, scale, window, stream};
  if (TILE_PAIR_OK && item_rows == TILE_ROWS) PairForm<TILE_PAIR_OK>::go(a);
  else if (page_size % 32 == 0) launch_tile<true, false>(a);
  else launch_tile<false, false>(a);
  return fg_launch_status();
}

// query rows (tokens x heads of a kv head's group) of one item of fg_attn_tile: of the larger form, or
// (small != 0) of the form with 64-row items
extern "C" int fg_attn_tile_rows(int small) { return small ? TILE_ROWS_SMALL : TILE_ROWS; }

// ReLU linear attention for head_dim 112 (the `linear_head_dim: 112` video configurations) on gfx950,
// bf16 / f16 io.  Same two phases and the same state layout as the head_dim-32 kernels --
// fp32 [B][h][n_chunks][113][112], row 112 = sum_n relu(k_n) -- but one head is now a 112 x 112
// problem of its own (7 x 7 MFMA tiles of 16, padded to 8 x 8 with zero channels):
//
//   phase 1  workgroup = (batch, head, token range): eight waves walk the range in tiles of 32 tokens that come
//            global -> LDS by direct loads into a ring; four waves accumulate the 128 x 128 state in registers
//            (operands read transposed from the token-major tiles), four apply the on-load transforms one tile
//            ahead.  One record per chunk the range touches; a second kernel sums a chunk's records in range
//            order and runs the prefix over chunks.
//   phase 2  without on-load transforms the same walk: four MFMA waves, four waves that issue the loads and carry
//            finished output tiles to global memory.  With transforms: workgroup = (batch, head, token range of
//            192..2048 tokens), 256 threads that all load, transform, multiply and store, steps of 32 tokens
//            through workgroup-shared LDS tiles.  In both, wave w produces output channels [32w, 32w+32) from its
//            own slice of the state (two bf16 terms of the fp32 values as MFMA 16x16x32 A operands for bf16
//            output, three for fp32 output) plus a row block that carries ksum in every row, so each lane gets
//            its token's denominator.
#include <algorithm>
#include <type_traits>

#include "common.h"
#include "linattn_common.h"

namespace sana {
namespace {

constexpr int DH = 112;                 // head dim
constexpr int SE = (DH + 1) * DH;       // 12656 state elements per (batch, head, chunk)
constexpr int NCH = DH / 8;             // 14 16-byte chunks per token and head
constexpr int TILE = 32;

// Workgroup index -> (unit, head).  Heads are taken four at a time: four 224-byte head rows are seven whole
// 128-byte lines, while a single head's row shares its first / last line with a neighbour.  Workgroup i runs on
// XCD i % 8, each XCD has its own L2: the (unit, head group) pairs are cut into 8 contiguous blocks, one per XCD,
// and the four heads of a group take consecutive slots of the XCD.  Shared lines are then fetched into one L2,
// once, and so is what all heads of a unit read alike (the tokens' rotary factors, 1 / rms): a unit's head groups
// sit on one XCD, two where a block boundary cuts through.  Returns false for the padding of the grid.
struct HeadUnit {
  int unit, head;
};
// a wave-uniform value into a scalar register, whatever the compiler thinks of it (integer division runs on the
// vector unit and its result, and all that is derived from it -- buffer resources, loop bounds -- would otherwise
// be handled as per-lane data)
__device__ __forceinline__ int uniform(int x) {
  int r;
  asm volatile("s_mov_b32 %0, %1" : "=s"(r) : "s"(x));
  return r;
}
__device__ __forceinline__ bool head_unit(int idx, int units, int h, HeadUnit& u) {
  const int xcd = idx & 7, slot = idx >> 3;
  const int hgroups = (h + 3) >> 2;
  const int total = units * hgroups;
  const int un = (xcd * total) / 8 + (slot >> 2);
  u.unit = uniform(un / hgroups);
  u.head = (un - u.unit * hgroups) * 4 + (slot & 3);
  return un < ((xcd + 1) * total) / 8 && u.head < h;
}
inline int64_t head_unit_grid(int64_t units, int h) { return (units * ((h + 3) / 4) + 7) / 8 * 8 * 4; }  // 8 x 4 x the largest block

// ----------------------------------------------------------------------------
// phase 1.  grid.x over token ranges x heads, see head_unit, grid.y = batch; block 512 = eight waves.
//
// A workgroup walks ONE contiguous token range of a (batch, head) -- ranges are cut by token count, not by chunk,
// so every workgroup has the same work whatever the chunking -- in tiles of 32 tokens that never straddle a chunk
// boundary, and writes one record (113 x 112 fp32) per chunk its range touches:
//   record[bh * nrec + range + c]
// (walking along the tokens, every new (range, chunk) pair increases the range or the chunk index or both, so
// range + c is different for every pair that occurs and at most ranges + chunks - 2; the records of a chunk are
// consecutive).  reduce112_kernel adds a chunk's records in range order (and runs the prefix over chunks when
// causal).
//
// Everything a tile needs comes global -> LDS by direct loads (`buffer_load_dwordx4 ... lds`, 16 bytes per lane,
// no staging registers) into rings: K and V rows of the head (224 bytes = 14 pieces, stored back to back: a row
// stride of 56 banks makes the transposing operand reads below conflict free as it is, and every lane of every load
// instruction carries data) and the tokens' 1 / rms in a ring of NKV stages, the tokens' rotary factors (448
// bytes) in a ring of NKV - 1.  Tokens past the tile's limit (the chunk or range end) are loaded through an offset
// outside the buffer resource, i.e. as zeros: they add nothing.  The bytes in flight per compute unit are what
// the rings hold, independent of registers.
//
// The state is 8 x 8 tiles of v_mfma_f32_16x16x32 (113 x 112 padded to 128 x 128); wave w < 4 owns rows (dv)
// [64 (w & 1), + 64) x columns (dk) [64 (w >> 1), + 64): 4 x 4 accumulator tiles, 8 operands per tile of tokens
// (the LDS operand traffic, which runs at half the plain read rate, is what the split minimises), no cross-wave
// reduction.  The operands are read from the token-major stage with ds_read_b64_tr_b16 (a 16-lane
// group reads a 4-token x 16-channel block and every lane receives the 4 tokens of ONE channel -- the transpose
// the contraction over tokens needs -- 2 instructions per operand quad).  Row block and column block 112..127 are
// padding and never read from LDS: the column block's operand is zero, the row block's A operand is a constant
// (row 0 all ones), so its accumulator row 0 is sum_n relu(k_n) = row 112 of the state, the "1" column the
// reference pads onto V.
//
// One barrier per tile.  Between two barriers every wave refills the ring entries consumed a tile ago, waves 0..3
// read the operands of tile i and run its MFMAs, and with on-load transforms (q/k RMSNorm, rotary embedding) waves
// 4..7 rewrite the K rows of tile i + 1 in place (16-byte pieces, two per thread): transform arithmetic and MFMA
// operand traffic of consecutive tiles run side by side in different waves.  With a rotary embedding the MFMA
// operands are rotated and ksum must not be, so it is accumulated per thread in the transform and folded through
// the tile's own (consumed) rotary slot when a chunk ends.
// ----------------------------------------------------------------------------
constexpr int S2_ROW = NCH * 16;                // bytes per token row of K / V in a stage
constexpr int S2_KV = 2 * TILE * S2_ROW;        // K rows, then V rows: 14336 bytes
constexpr int S2_ROPE = TILE * DH * 4;          // rotary factors of a tile: 14336 bytes
template <int PRE>
struct Stage2 {
  static constexpr bool has_norm = (PRE & 1) != 0, has_rope = (PRE & 2) != 0;
  static constexpr int kv_bytes = S2_KV + (has_norm ? 1024 : 0);  // (a load instruction always fills 64 slots)
  static constexpr int n_kv = 2 * TILE * NCH / 64, n_rope = has_rope ? TILE * 28 / 64 : 0;   // load instructions: 14, 14
  static constexpr int n_instr = n_kv + n_rope + (has_norm ? 1 : 0);
  static constexpr int NKV = 6;   // ring depth (measured: 4 .. 10 make no difference, the kernel is not bound by latency)
  static constexpr int NR = has_rope ? NKV - 1 : 0;
  static constexpr int bytes = NKV * kv_bytes + NR * S2_ROPE;
  static constexpr int per_wave = (n_instr + 3) / 4;   // load instructions per tile of issuing waves < n_instr % 4; the others one less
  static_assert(bytes <= 160 * 1024, "LDS");
  static_assert((NKV - 2) * per_wave < 64, "vmcnt range");
};

template <typename T>
__device__ __forceinline__ f32x4_t mfma16(u32x4_t a, u32x4_t b, f32x4_t c) {
  if constexpr (is_f16<T>)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  else
    return mfma_16x16x32_bf16(a, b, c);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// The rings are read with asm statements: to the compiler an ordinary LDS read may alias the LDS-writing global
// loads still in flight (the stages further down the ring) and it would wait for ALL of them (vmcnt(0)) in front of
// the first read, which would empty the ring at every tile.  Which loads must have landed is the kernel's own
// business (counted waits + barriers); the waits for the LDS reads themselves are tied to their results.
// Between such a read and its wait there must be no control flow that merges the result with another value: the
// compiler, to which the result exists as soon as the statement has run, may copy it then and there.
// addr: LDS byte address, OFF: immediate byte offset.
//
// read_tr16: 4 tokens x 16 channels of a token-major tile -> this lane's channel, 4 tokens; addr points at the
// lane's 4-channel segment of its token
template <int OFF>
__device__ __forceinline__ u32x2_t read_tr16(uint32_t addr) {
  u32x2_t v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
// the same into a register that already holds a value (read-write operand: a conditional read then needs no
// merge of two registers behind it, where the compiler could copy a result that has not arrived yet)
template <int OFF>
__device__ __forceinline__ void read_tr16_over(u32x2_t& v, uint32_t addr) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "+v"(v) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ u32x4_t lds_read128(uint32_t addr) {
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
__device__ __forceinline__ float lds_read32(uint32_t addr) {
  float v;
  asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr));
  return v;
}
template <int OFF>
__device__ __forceinline__ void lds_write128(uint32_t addr, u32x4_t v) {
  asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(size_t)(__attribute__((address_space(3))) const void*)p;
}

struct TileCur {  // walks the tiles of a token range: 32 tokens at a time, never across a chunk boundary
  int t, c, seg_end;
};
struct Tile112 {
  int start, limit, c;
  bool last;  // of its chunk within the range
};
struct Ops112 {  // MFMA operands of one tile of tokens: [operand][token half]
  u32x2_t v[4][2], k[4][2];
};

template <typename T, int PRE>
__global__ __launch_bounds__(512) void state112_kernel(const uint16_t* __restrict__ K, const uint16_t* __restrict__ V,
                                                       float* __restrict__ partial,
                                                       const int32_t* __restrict__ chunk_starts, int N, int h,
                                                       int nrec, int range_tokens, int units, int64_t stride_b,
                                                       int64_t stride_n, const QkPre pre) {
  typedef Stage2<PRE> ST;
  constexpr bool has_norm = ST::has_norm, has_rope = ST::has_rope;
  constexpr int NKV = ST::NKV, NR = ST::NR;
  constexpr int AHEAD = PRE ? 1 : 0;  // the transform works one tile ahead of the operand reads
  __shared__ __attribute__((aligned(1024))) unsigned char smem[ST::bytes];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  HeadUnit hu;
  if (!head_unit(blockIdx.x, units, h, hu)) return;  // uniform over the workgroup
  const int head = hu.head;
  const int rg = hu.unit, b = blockIdx.y;
  const int r0 = rg * range_tokens, r1 = min(N, r0 + range_tokens);
  if (r0 >= r1) return;
  auto chunk_end = [&](int c) __attribute__((always_inline)) { return chunk_starts ? chunk_starts[c + 1] : N; };
  int c0 = 0;
  while (chunk_end(c0) <= r0) ++c0;  // the chunk of the range's first token (uniform; a few dozen chunks at most)
  const uint32_t smem_addr = lds_addr(smem);
  const uint32_t rope_ring = smem_addr + NKV * ST::kv_bytes;

  // ---- global -> LDS.  Load instruction q of a tile fills slots [64 q', 64 q' + 64) of 16 bytes of its ring entry;
  // wave w < 4 issues q = w, w + 4, ... (a wave that issues loads stalls while the memory pipeline is full, which
  // in a kernel bound by memory is most of the time: the waves that run the transforms must not be among them).
  // Slots: K rows (32 x 14), V rows (32 x 14), 1 / rms (8) | rotary factors (32 x 28)
  const int row_b = (int)stride_n * 2;
  const int64_t tok_bytes = (int64_t)N * stride_n * 2;
  const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(K + (int64_t)b * stride_b + head * DH), 0, (int)(tok_bytes - (int64_t)head * DH * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(V + (int64_t)b * stride_b + head * DH), 0, (int)(tok_bytes - (int64_t)head * DH * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(has_norm ? pre.rinv + (int64_t)b * N : nullptr), 0, has_norm ? N * 4 : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(pre.rope), 0, has_rope ? N * (DH * 4) : 0, 0x00020000);
  const int idle = (int)0x80000000u;
  // per load instruction of this wave: token row (within the tile) of the lane's slot and its byte offset from the
  // tile's first token
  int ld_row[ST::per_wave], ld_off[ST::per_wave];
#pragma unroll
  for (int j = 0; j < ST::per_wave; ++j) {
    const int q = wave + 4 * j;
    ld_row[j] = 0;
    ld_off[j] = idle;
    if (q < ST::n_kv) {
      const int s = (q % (ST::n_kv / 2)) * 64 + lane, row = s / NCH, col = s - row * NCH;
      ld_row[j] = row;
      ld_off[j] = row * row_b + col * 16;
    } else if (q < ST::n_kv + ST::n_rope) {
      const int s = (q - ST::n_kv) * 64 + lane;  // the tile's factors are one contiguous run
      ld_row[j] = s / 28;
      ld_off[j] = s * 16;
    } else if (q < ST::n_instr) {  // 1 / rms: 8 pieces of 4 tokens
      ld_row[j] = 0;   // (tokens past the limit read whatever statistic is there, or zero past the tensor: their K rows are zeros)
      ld_off[j] = lane < 8 ? lane * 16 : idle;
    }
  }
  int issued = 0;  // tiles whose loads have been issued; tile t lives in K/V stage t % NKV and rotary slot t % NR
  auto issue = [&](int start, int limit) __attribute__((always_inline)) {
    if (wave >= 4) {
      ++issued;
      return;
    }
    unsigned char* kvb = smem + (issued % NKV) * ST::kv_bytes;
    unsigned char* rpb = smem + NKV * ST::kv_bytes + (has_rope ? (issued % (NR ? NR : 1)) * S2_ROPE : 0);
#pragma unroll
    for (int j = 0; j < ST::per_wave; ++j) {
      const int q = wave + 4 * j;  // wave-uniform
      if (q >= ST::n_instr) break;
      // the tile's first token goes into the scalar offset, the lane's part is constant; rows past the limit and
      // idle lanes get an offset outside the resource
      const int voff = ld_row[j] < limit - start ? ld_off[j] : idle;
      if (q < ST::n_kv) {
        auto dst = (__attribute__((address_space(3))) void*)(kvb + q * 1024);
        if (q < ST::n_kv / 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_k, dst, 16, voff, start * row_b, 0, 0);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_v, dst, 16, voff, start * row_b, 0, 0);
      } else if (q < ST::n_kv + ST::n_rope) {
        auto dst = (__attribute__((address_space(3))) void*)(rpb + (q - ST::n_kv) * 1024);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_c, dst, 16, voff, start * (DH * 4), 0, 0);
      } else {
        auto dst = (__attribute__((address_space(3))) void*)(kvb + S2_KV);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_r, dst, 16, voff, start * 4, 0, 0);
      }
    }
    ++issued;
  };
  const bool more_loads = ST::n_instr % 4 == 0 || wave < ST::n_instr % 4;  // this wave issues per_wave loads per tile
  // waits until this wave's loads of all but the `keep` youngest tiles have landed; `keep` as a template argument
  // when it is the steady-state figure, everything otherwise (prologue and tail of short ranges)
  auto wait_tiles = [&](auto keep_c, int keep) __attribute__((always_inline)) {
    constexpr int KEEP = decltype(keep_c)::value;
    if (wave >= 4) return;  // nothing of its own in flight
    if (keep == KEEP) {
      if (more_loads) wait_vmcnt<KEEP * ST::per_wave>();
      else wait_vmcnt<KEEP * (ST::per_wave - 1)>();
    } else {
      wait_vmcnt<0>();
    }
  };

  auto has_tile = [&](const TileCur& cur) __attribute__((always_inline)) { return cur.t < r1; };
  auto next_tile = [&](TileCur& cur) __attribute__((always_inline)) {
    Tile112 tl;
    tl.start = cur.t;
    tl.limit = cur.seg_end;
    tl.c = cur.c;
    const int nt = min(cur.t + TILE, cur.seg_end);
    tl.last = nt == cur.seg_end;
    cur.t = nt;
    if (tl.last && nt < r1) {
      ++cur.c;
      cur.seg_end = min(chunk_end(cur.c), r1);
    }
    return tl;
  };
  TileCur icur = {r0, c0, min(chunk_end(c0), r1)}, ccur = icur, tcur = icur;
#pragma unroll 1
  for (int i = 0; i < NKV - 1 && has_tile(icur); ++i) {
    const Tile112 tl = next_tile(icur);
    issue(tl.start, tl.limit);
  }
  auto record_of = [&](int c) __attribute__((always_inline)) {
    const int64_t slot = (int64_t)(b * h + head) * nrec + rg + c;
    return partial + slot * SE;
  };

  // ---- roles.  Waves 0..3 run the MFMAs (and issue the loads), waves 4..7 the transforms.
  const bool mma_role = wave < 4;  // wave-uniform

  // ---- transform side: 16-byte piece i of a tile = piece i % 14 of token i / 14; thread tid - 256 takes pieces
  // tid - 256 and tid (the second one exists for tid < 448)
  const int tq = tid - 256;
  bool tp_ok[2];
  int tp_tok[2];
  u32x4_t kw[2];
  float ks8[2][8];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = tq + 256 * u;
    tp_ok[u] = PRE && !mma_role && i < TILE * NCH;
    tp_tok[u] = i / NCH;
    kw[u] = u32x4_t{0u, 0u, 0u, 0u};
    if (has_norm && tp_ok[u]) kw[u] = *reinterpret_cast<const u32x4_t*>(pre.weight + head * DH + (i - tp_tok[u] * NCH) * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) ks8[u][e] = 0.f;
  }
  int tdone = 0;  // tiles transformed
  // Rewrites the K rows of the next tile of the transform cursor in place; all of its loads have landed and nobody
  // else touches it before the next barrier.  Every wave calls it (the cursor and the barrier of the ksum fold are
  // workgroup business), the transform waves do the work.
  auto transform_next = [&]() __attribute__((always_inline)) {
    const Tile112 tl = next_tile(tcur);
    const uint32_t sa = smem_addr + (tdone % NKV) * ST::kv_bytes;
    const uint32_t ra = rope_ring + (has_rope ? (tdone % (NR ? NR : 1)) * S2_ROPE : 0);
    if (!mma_role) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {  // (one piece after the other: the registers of both at once do not fit)
        if (!tp_ok[u]) continue;
        const int i = tq + 256 * u;
        u32x4_t x = lds_read128<0>(sa + i * 16);
        float rin = 0.f;
        f32x4_t cs0 = {0.f, 0.f, 0.f, 0.f}, cs1 = cs0;
        if (has_norm) rin = lds_read32(sa + S2_KV + tp_tok[u] * 4);
        if (has_rope) {
          cs0 = __builtin_bit_cast(f32x4_t, lds_read128<0>(ra + i * 32));
          cs1 = __builtin_bit_cast(f32x4_t, lds_read128<16>(ra + i * 32));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(x), "+v"(rin), "+v"(cs0), "+v"(cs1));
        if (has_norm) x = rms_scale8(x, rin, kw[u]);
        x = relu_pk16(x);
        if (has_rope) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            ks8[u][2 * e] += bf16_lo(x[e]);
            ks8[u][2 * e + 1] += bf16_hi(x[e]);
          }
          x = rope8(x, cs0, cs1);
        }
        lds_write128<0>(sa + i * 16, x);
      }
    }
    if (has_rope && tl.last) {  // uniform: a chunk (or the range) ends with this tile: its ksum row
      // fold area = the tile's rotary slot: every thread overwrites exactly the bytes it alone has read
      if (!mma_role) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          if (!tp_ok[u]) continue;
          const uint32_t fa = ra + (tq + 256 * u) * 32;
          lds_write128<0>(fa, __builtin_bit_cast(u32x4_t, f32x4_t{ks8[u][0], ks8[u][1], ks8[u][2], ks8[u][3]}));
          lds_write128<16>(fa, __builtin_bit_cast(u32x4_t, f32x4_t{ks8[u][4], ks8[u][5], ks8[u][6], ks8[u][7]}));
#pragma unroll
          for (int e = 0; e < 8; ++e) ks8[u][e] = 0.f;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      if (tq >= 0 && tq < DH) {  // channel tq: piece tq / 8 of the 32 tokens
        const float* fold = reinterpret_cast<const float*>(smem + NKV * ST::kv_bytes + (tdone % (NR ? NR : 1)) * S2_ROPE);
        const int p = tq >> 3, e = tq & 7;
        float sum = 0.f;
#pragma unroll 4
        for (int tk = 0; tk < TILE; ++tk) sum += fold[(tk * NCH + p) * 8 + e];
        record_of(tl.c)[DH * DH + tq] = sum;
        // stores share the counter the rings wait on (and need not retire in order with the loads)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
    }
    ++tdone;
  };

  // ---- MFMA side: lane = 16 g + R; tokens 16 hh + 4 g + R / 4 (hh = 0, 1) are this lane group's 8 contraction
  // slots; both operands use the same map.  Wave w < 4: rows (dv) [64 (w & 1), + 64) x columns (dk) [64 (w >> 1), + 64)
  const int g = lane >> 4, R = lane & 15;
  const int dvh = wave & 1, dkh = (wave >> 1) & 1;   // wave-uniform
  const bool v3_real = dvh == 0, k3_real = dkh == 0;  // row block 112..127 / column block 112..127 are padding
  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int tr_off = (4 * g + (R >> 2)) * S2_ROW + (R & 3) * 8;
  const uint32_t v_off = TILE * S2_ROW + tr_off + dvh * 128, k_off = tr_off + dkh * 128;
  const uint32_t one2 = is_f16<T> ? 0x3c003c00u : 0x3f803f80u;
  const u32x2_t ones2 = R == 0 ? u32x2_t{one2, one2} : u32x2_t{0u, 0u};
  auto read_ops = [&](int tile, Ops112& o) __attribute__((always_inline)) {
    const uint32_t sa = smem_addr + (tile % NKV) * ST::kv_bytes;
    const uint32_t vb = sa + v_off, kb = sa + k_off;
    o.v[0][0] = read_tr16<0>(vb), o.v[0][1] = read_tr16<16 * S2_ROW>(vb);
    o.v[1][0] = read_tr16<32>(vb), o.v[1][1] = read_tr16<32 + 16 * S2_ROW>(vb);
    o.v[2][0] = read_tr16<64>(vb), o.v[2][1] = read_tr16<64 + 16 * S2_ROW>(vb);
    o.v[3][0] = o.v[3][1] = ones2;  // row block 112..127: row 0 of the A operand is all ones
    if (v3_real) read_tr16_over<96>(o.v[3][0], vb), read_tr16_over<96 + 16 * S2_ROW>(o.v[3][1], vb);
    o.k[0][0] = read_tr16<0>(kb), o.k[0][1] = read_tr16<16 * S2_ROW>(kb);
    o.k[1][0] = read_tr16<32>(kb), o.k[1][1] = read_tr16<32 + 16 * S2_ROW>(kb);
    o.k[2][0] = read_tr16<64>(kb), o.k[2][1] = read_tr16<64 + 16 * S2_ROW>(kb);
    o.k[3][0] = o.k[3][1] = u32x2_t{0u, 0u};  // column block 112..127
    if (k3_real) read_tr16_over<96>(o.k[3][0], kb), read_tr16_over<96 + 16 * S2_ROW>(o.k[3][1], kb);
  };
  auto wait_ops = [&](Ops112& o) __attribute__((always_inline)) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(o.v[0][0]), "+v"(o.v[0][1]), "+v"(o.v[1][0]), "+v"(o.v[1][1]), "+v"(o.v[2][0]), "+v"(o.v[2][1]),
                   "+v"(o.v[3][0]), "+v"(o.v[3][1]), "+v"(o.k[0][0]), "+v"(o.k[0][1]), "+v"(o.k[1][0]), "+v"(o.k[1][1]),
                   "+v"(o.k[2][0]), "+v"(o.k[2][1]), "+v"(o.k[3][0]), "+v"(o.k[3][1])
                 :
                 : "memory");
    if (!PRE) {
#pragma unroll
      for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) o.k[ct][hh] = u32x2_t{relu_pk16(o.k[ct][hh].x), relu_pk16(o.k[ct][hh].y)};
    }
  };
  auto mma = [&](const Ops112& o) __attribute__((always_inline)) {
    u32x4_t fk[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) fk[ct] = u32x4_t{o.k[ct][0].x, o.k[ct][0].y, o.k[ct][1].x, o.k[ct][1].y};
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const u32x4_t fv = {o.v[rb][0].x, o.v[rb][0].y, o.v[rb][1].x, o.v[rb][1].y};
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) acc[rb][ct] = mfma16<T>(fv, fk[ct], acc[rb][ct]);  // (zero operand in the padding column block)
    }
  };
  auto record = [&](int c) __attribute__((always_inline)) {  // the accumulators -> the record of chunk c, then zero
    // D layout of the 16x16 MFMA: lane -> column lane % 16 (dk within the tile), register s -> row 4 (lane / 16) + s
    int lane_off = (64 * dvh + 4 * g) * DH + 64 * dkh + R;
    asm volatile("" : "+v"(lane_off));  // (computed here, per record: hoisted out of the tile loop the 64 store
                                        // addresses would sit in registers for the whole kernel)
    float* dst = record_of(c) + lane_off;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        if (ct == 3 && !k3_real) continue;
        if (rb < 3 || v3_real) {
#pragma unroll
          for (int s = 0; s < 4; ++s) dst[(16 * rb + s) * DH + 16 * ct] = acc[rb][ct][s];
        } else if (!has_rope) {  // row 112: ksum
          if (g == 0) dst[(16 * rb) * DH + 16 * ct] = acc[rb][ct][0];
        }
      }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    // the record's stores share the counter the rings wait on (and need not retire in order with the loads):
    // drain it once per record, so that the counts keep meaning "tiles younger than this one"
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };

  int it = 0;  // tile whose operands are read in this iteration
  if (PRE) {   // tile 0 is transformed ahead of the loop
    wait_tiles(std::integral_constant<int, NKV - 2>(), issued - 1);
    __builtin_amdgcn_s_barrier();
    transform_next();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
#pragma unroll 1
  while (has_tile(ccur)) {
    const Tile112 tl = next_tile(ccur);
    // this wave's loads of tile it (+ 1 with transforms) have landed: all but those of the tiles issued after it
    wait_tiles(std::integral_constant<int, NKV - 2 - AHEAD>(), issued - 1 - (it + AHEAD));
    __builtin_amdgcn_s_barrier();  // and everyone else's; every wave is done with tile it - 1 and the transform of
                                   // tile it is in LDS (no fence: younger loads stay in flight)
    if (has_tile(icur)) {          // refill the entries of tile it - 1
      const Tile112 nl = next_tile(icur);
      issue(nl.start, nl.limit);
    }
    if (mma_role) {
      Ops112 o;
      read_ops(it, o);
      wait_ops(o);
      mma(o);
      if (tl.last) record(tl.c);
    }
    if (PRE && has_tile(tcur)) transform_next();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    ++it;
  }
}

// sum of the records of one chunk in range order (+ inclusive prefix over chunks when causal).  A chunk's records
// are those of the ranges [begin / L, (end - 1) / L] that touch it, at record index range + chunk; with
// range_tokens == 0 every chunk has exactly one record, its own (the in-place scan of finished states: partial ==
// state, nrec == n_chunks, every thread rewrites only what it has read itself).  Workgroup = cl chunks (a power of two, at most 16) x nq >= 64 groups of four adjacent
// elements, so that a wave reads whole kilobytes of one record: a thread sums the records of ONE (chunk, element
// group) -- the loads of its first two
// records (a chunk shorter than a range has no more) in flight together -- and the prefix over chunks goes through
// LDS, every thread adding up its predecessors in chunk order, which is the order of a running sum.
__global__ __launch_bounds__(1024) void reduce112_kernel(const float* partial, float* state, const int32_t* chunk_starts,
                                                         int N, int n_chunks, int nrec, int range_tokens, int causal,
                                                         int cl, int nblk) {
  constexpr int SE4 = SE / 4;
  __shared__ f32x4_t sums[1024];
  __shared__ f32x4_t carry_sh[256];
  const int nq = blockDim.x / cl;
  const int q = threadIdx.x % nq, lc = threadIdx.x / nq;
  const int64_t bh = blockIdx.x / nblk;
  const int e4 = (int)(blockIdx.x - bh * nblk) * nq + q;
  const bool e_ok = e4 < SE4;
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  f32x4_t carry = zero;
  for (int c0 = 0; c0 < n_chunks; c0 += cl) {  // uniform
    const int c = c0 + lc;
    const bool ok = e_ok && c < n_chunks;
    f32x4_t s = zero;
    if (ok) {
      int nparts = 1, first = c;
      if (range_tokens > 0) {
        const int cb = chunk_starts ? chunk_starts[c] : 0, ce = chunk_starts ? chunk_starts[c + 1] : N;
        nparts = (ce - 1) / range_tokens - cb / range_tokens + 1;
        first = cb / range_tokens + c;
      }
      const float* p0 = partial + (bh * nrec + first) * SE + e4 * 4;
      const f32x4_t v0 = *reinterpret_cast<const f32x4_t*>(p0);  // (every chunk has a first record)
      const f32x4_t v1 = nparts > 1 ? *reinterpret_cast<const f32x4_t*>(p0 + SE) : zero;
      s = v0 + v1;
      for (int sp0 = 2; sp0 < nparts; sp0 += 8) {  // a chunk spread over more than two ranges: 8 loads at a time
        f32x4_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          w[j] = sp0 + j < nparts ? *reinterpret_cast<const f32x4_t*>(p0 + (int64_t)(sp0 + j) * SE) : zero;
#pragma unroll
        for (int j = 0; j < 8; ++j) s += w[j];
      }
    }
    if (causal) {
      sums[threadIdx.x] = s;
      __syncthreads();
      f32x4_t run = carry;
      for (int j = 0; j <= lc; ++j) run += sums[j * nq + q];
      s = run;
      if (lc == cl - 1) carry_sh[q] = run;
      __syncthreads();
      carry = carry_sh[q];
    }
    if (ok) *reinterpret_cast<f32x4_t*>(state + (bh * n_chunks + c) * SE + e4 * 4) = s;
  }
}

// ----------------------------------------------------------------------------
// phase 2 without on-load transforms.  grid.x over token ranges x heads, see head_unit, grid.y = batch; block 512 =
// eight waves.
//
// Built like phase 1: a workgroup walks ONE contiguous token range of a (batch, head), cut by token count, in
// tiles of 32 tokens that never straddle a chunk boundary.  The q rows of a tile come global -> LDS by direct loads
// into a ring; waves 0..3 run the MFMAs (and the ReLU, on their operands), waves 4..7 issue the loads and carry the
// finished output tile of the step before from LDS to global memory in whole rows.  A wave that talks to global
// memory stalls while the memory pipeline is full, which is most of the time in a kernel bound by it: the MFMA
// waves only ever wait for data that has already landed.  (With on-load transforms the same layout was measured a
// sixth SLOWER than the kernel further down: four waves are too few for the transform arithmetic of a tile.)
//
// q tiles are rows of 16 pieces of 16 bytes (14 of data, 2 of zeros: the padded k range 112..127) with the piece
// index XORed with the token's low four bits: the 16 tokens of an MFMA B operand read (one piece each, same logical
// piece) hit 16 different pieces, i.e. all 64 banks once.  Direct loads fill LDS linearly, lane by lane, so the
// swizzle is applied to the global address a lane fetches.
//
// MFMA wave w produces output channels [32 w, 32 w + 32) from its own slice of the chunk's state (two bf16 terms
// of the fp32 values as MFMA 16x16x32 A operands for bf16 output, three for fp32 output) plus a row block that
// carries ksum in every row, so each lane gets its token's denominator.  The slice is rebuilt when the walk enters
// another chunk.
// ----------------------------------------------------------------------------
// fp32 -> bf16 terms hi + mid (+ lo), pairwise: one packed convert rounds two values
template <int NT>
__device__ __forceinline__ void split_terms(const float x[8], u32x4_t out[NT]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float r0 = x[2 * e], r1 = x[2 * e + 1];
#pragma unroll
    for (int term = 0; term < NT; ++term) {
      const uint32_t pk = pack_bf16(r0, r1);
      out[term][e] = pk;
      if (term + 1 < NT) {
        r0 -= bf16_lo(pk);
        r1 -= bf16_hi(pk);
      }
    }
  }
}

constexpr int A2_QT = TILE * 256;   // a q tile: 32 rows of 16 pieces
constexpr int OROW16 = 272;         // byte row stride of the 16-bit output tile: 68 banks, so the 16 tokens of a b128
                                    // write land on 16 disjoint groups of 4 banks
constexpr int OROW32 = 464;         // of the fp32 output tile (116 banks = 52 mod 64: same argument)
template <bool OUT_F32>
struct Stage3 {
  static constexpr int n_q = A2_QT / 1024;   // load instructions per tile: 8, two per issuing wave
  static constexpr int NQ = 4;               // ring depth
  static constexpr int out_bytes = TILE * (OUT_F32 ? OROW32 : OROW16);
  static constexpr int out_off = NQ * A2_QT;
  static constexpr int bytes = out_off + 2 * out_bytes;
  static constexpr int per_wave = n_q / 4;
};

template <bool OUT_F32>
__global__ __launch_bounds__(512) void apply112_stream_kernel(const uint16_t* __restrict__ Q,
                                                              const float* __restrict__ state, void* __restrict__ out,
                                                              const int32_t* __restrict__ chunk_starts, int N, int h,
                                                              int n_chunks, int range_tokens, int units,
                                                              int64_t q_stride_b, int64_t q_stride_n, int64_t o_stride_b,
                                                              int64_t o_stride_n, float eps) {
  typedef Stage3<OUT_F32> ST;
  constexpr int NQ = ST::NQ;
  constexpr int NT = OUT_F32 ? 3 : 2;    // bf16 terms of an fp32 state value: 24 / 16 mantissa bits
  __shared__ __attribute__((aligned(1024))) unsigned char smem[ST::bytes];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  HeadUnit hu;
  if (!head_unit(blockIdx.x, units, h, hu)) return;  // uniform over the workgroup
  const int head = hu.head;
  const int rg = hu.unit, b = blockIdx.y;
  const int r0 = rg * range_tokens, r1 = min(N, r0 + range_tokens);
  if (r0 >= r1) return;
  auto chunk_end = [&](int c) __attribute__((always_inline)) { return chunk_starts ? chunk_starts[c + 1] : N; };
  int c0 = 0;
  while (chunk_end(c0) <= r0) ++c0;  // the chunk of the range's first token (uniform; a few dozen chunks at most)
  const uint32_t smem_addr = lds_addr(smem);
  const bool mma_role = wave < 4;  // wave-uniform

  // ---- global -> LDS, issued by the helper waves (measured: 73 us against 86 with the MFMA waves issuing, whose
  // instruction stream is the longest here): wave w issues instructions w - 4 and w of a tile, each 4 rows of 16
  // pieces
  const int row_b = (int)q_stride_n * 2;
  const __amdgpu_buffer_rsrc_t rsrc_q = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(Q + (int64_t)b * q_stride_b + head * DH), 0,
      (int)((int64_t)N * q_stride_n * 2 - (int64_t)head * DH * 2), 0x00020000);
  const int idle = (int)0x80000000u;
  // per load instruction of this wave: the lane's token row within the tile and its byte offset from the tile's
  // first token (the padding pieces: an offset outside the resource, i.e. zeros)
  int ld_row[ST::per_wave], ld_off[ST::per_wave];
#pragma unroll
  for (int j = 0; j < ST::per_wave; ++j) {
    const int s = ((wave & 3) + 4 * j) * 64 + lane, row = s >> 4, piece = (s & 15) ^ (row & 15);
    ld_row[j] = row;
    ld_off[j] = piece < NCH ? row * row_b + piece * 16 : idle;
  }
  int issued = 0;  // tiles whose loads have been issued; tile t lives in ring entry t % NQ
  auto issue = [&](int start, int limit) __attribute__((always_inline)) {
    if (!mma_role) {
      unsigned char* qb = smem + (issued % NQ) * A2_QT;
#pragma unroll
      for (int j = 0; j < ST::per_wave; ++j) {
        const int q = (wave & 3) + 4 * j;  // wave-uniform
        // the tile's first token goes into the scalar offset; rows past the limit get an offset outside the resource
        const int voff = ld_row[j] < limit - start ? ld_off[j] : idle;
        auto dst = (__attribute__((address_space(3))) void*)(qb + q * 1024);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_q, dst, 16, voff, start * row_b, 0, 0);
      }
    }
    ++issued;
  };
  // waits until the issuing waves' loads of all but the `keep` youngest tiles have landed; `keep` as a template
  // argument when it is the steady-state figure, everything otherwise (the tail of the range)
  auto wait_tiles = [&](int keep) __attribute__((always_inline)) {
    if (mma_role) return;  // nothing of its own in flight that anyone waits for
    if (keep == NQ - 2) wait_vmcnt<(NQ - 2) * ST::per_wave>();
    else wait_vmcnt<0>();
  };
  auto has_tile = [&](const TileCur& cur) __attribute__((always_inline)) { return cur.t < r1; };
  auto next_tile = [&](TileCur& cur) __attribute__((always_inline)) {
    Tile112 tl;
    tl.start = cur.t;
    tl.limit = cur.seg_end;
    tl.c = cur.c;
    const int nt = min(cur.t + TILE, cur.seg_end);
    tl.last = nt == cur.seg_end;
    cur.t = nt;
    if (tl.last && nt < r1) {
      ++cur.c;
      cur.seg_end = min(chunk_end(cur.c), r1);
    }
    return tl;
  };
  TileCur icur = {r0, c0, min(chunk_end(c0), r1)}, ccur = icur;
#pragma unroll 1
  for (int i = 0; i < NQ - 1 && has_tile(icur); ++i) {
    const Tile112 tl = next_tile(icur);
    issue(tl.start, tl.limit);
  }

  // ---- helper waves: the output tile of a finished step -> global memory, whole rows
  const int tq = tid - 256;
  constexpr int OP = OUT_F32 ? 2 * NCH : NCH;                  // 16-byte pieces per output row
  constexpr int OPT = (TILE * OP + 255) / 256;                 // pieces per helper thread
  auto store_tile = [&](int buf, int start, int limit) __attribute__((always_inline)) {
    if (mma_role) return;
    // (the stores below share the vector memory counter with this wave's loads.  That is harmless for the counted
    // waits: outstanding stores only add to the count, so "at most k operations outstanding" still means "at most k
    // loads outstanding", and loads retire in issue order)
    const uint32_t ta = smem_addr + ST::out_off + buf * ST::out_bytes;
    u32x4_t v[OPT];
    int tok[OPT], p[OPT];
    int tqv = tq;
    asm volatile("" : "+v"(tqv));  // (addresses are computed here, per tile: hoisted out of the tile loop they
                                   // would occupy registers for the whole kernel)
#pragma unroll
    for (int u = 0; u < OPT; ++u) {
      // (every thread reads, the surplus ones the last piece again: no branch between a read and its wait, where
      // the compiler could copy a result that has not arrived yet)
      const int i = min(tqv + 256 * u, TILE * OP - 1);
      tok[u] = i / OP;
      p[u] = i - tok[u] * OP;
      v[u] = lds_read128<0>(ta + tok[u] * (OUT_F32 ? OROW32 : OROW16) + p[u] * 16);
    }
    if (OPT == 2) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[OPT - 1]));
    else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[OPT - 2]), "+v"(v[OPT - 1]));
    unsigned char* ob = reinterpret_cast<unsigned char*>(out) +
                        ((int64_t)b * o_stride_b + head * DH) * (OUT_F32 ? 4 : 2);
#pragma unroll
    for (int u = 0; u < OPT; ++u) {
      const int i = tqv + 256 * u;
      if (i < TILE * OP && start + tok[u] < limit)
        *reinterpret_cast<u32x4_t*>(ob + (int64_t)(start + tok[u]) * o_stride_n * (OUT_F32 ? 4 : 2) + p[u] * 16) = v[u];
    }
  };

  // ---- MFMA waves.  A operands: MFMA 16x16x32 A lane -> row lane % 16, k = 8 (lane / 16) + e.  Row r of row block
  // rb of this wave is output channel 32 wave + 8 (r / 4) + 4 rb + r % 4, so that a lane (token n, group g') ends
  // up with the 8 contiguous channels 32 wave + 8 g' .. + 7 (registers s of blocks 0 and 1).  Block 2 carries ksum
  // in every row.  Channels and k indices past 112 are zero.
  const int n = lane & 15, g = lane >> 4;
  u32x4_t a[3][4][NT];  // [row block][k block][term]
  auto load_state = [&](int c) __attribute__((always_inline)) {
    const float* sp = state + ((int64_t)(b * h + head) * n_chunks + c) * SE;
    // buffer loads: rows / k groups outside the head's state get an out-of-range offset and read as zero
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(sp), 0, SE * 4, 0x00020000);
#pragma unroll
    for (int rb = 0; rb < 3; ++rb) {
      const int ch = 32 * (wave & 3) + 8 * (n >> 2) + 4 * rb + (n & 3);
      const int row = rb < 2 ? ch : DH;
      const bool row_ok = rb == 2 || ch < DH;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const int k0 = kb * 32 + 8 * g;
        const int off = (row_ok && k0 < DH) ? (row * DH + k0) * 4 : idle;
        const f32x4_t x0 = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, off, 0, 0));
        const f32x4_t x1 = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, off + 16, 0, 0));
        const float x[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        split_terms<NT>(x, a[rb][kb]);
      }
    }
  };
  // B operand of k block kb: piece 4 kb + g of the lane's token, at its swizzled place
  uint32_t qoff[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) qoff[kb] = n * 256 + (((4 * kb + g) ^ n) << 4);
  const int och = 32 * (wave & 3) + 8 * g;  // this lane's 8 output channels
  auto mma_tile = [&](int tile) __attribute__((always_inline)) {
    const uint32_t sa = smem_addr + (tile % NQ) * A2_QT;
    const uint32_t to = smem_addr + ST::out_off + (tile & 1) * ST::out_bytes;
    // [token half][k block].  With bf16 output both halves are read up front (the second arrives during the MFMAs
    // of the first); with fp32 output the third state term has taken the registers: one half at a time
    constexpr bool BOTH = !OUT_F32;
    u32x4_t qd[2][4];
    auto read_half = [&](int ss) __attribute__((always_inline)) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) qd[ss][kb] = ss ? lds_read128<16 * 256>(sa + qoff[kb]) : lds_read128<0>(sa + qoff[kb]);
    };
    read_half(0);
    if (BOTH) read_half(1);
#pragma unroll
    for (int ss = 0; ss < 2; ++ss) {
      if (!BOTH && ss == 1) read_half(1);
      if (BOTH && ss == 0)
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(qd[0][0]), "+v"(qd[0][1]), "+v"(qd[0][2]), "+v"(qd[0][3]));
      else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(qd[ss][0]), "+v"(qd[ss][1]), "+v"(qd[ss][2]), "+v"(qd[ss][3]));
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) qd[ss][kb] = relu_pk16(qd[ss][kb]);
      f32x4_t acc[3];
#pragma unroll
      for (int rb = 0; rb < 3; ++rb) acc[rb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int term = NT - 1; term >= 0; --term)  // smallest term first
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
          for (int rb = 0; rb < 3; ++rb)  // three independent chains back to back
            acc[rb] = mfma_16x16x32_bf16(a[rb][kb][term], qd[ss][kb], acc[rb]);
      if (och < DH) {
        const float den = acc[2][0] + eps;
        if (OUT_F32) {
          f32x4_t o0, o1;
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            o0[s] = acc[0][s] / den;
            o1[s] = acc[1][s] / den;
          }
          const uint32_t oa = to + (16 * ss + n) * OROW32 + och * 4;
          lds_write128<0>(oa, __builtin_bit_cast(u32x4_t, o0));
          lds_write128<16>(oa, __builtin_bit_cast(u32x4_t, o1));
        } else {
          const float inv = __builtin_amdgcn_rcpf(den);
          u32x4_t o;
          o.x = pack_bf16(acc[0][0] * inv, acc[0][1] * inv);
          o.y = pack_bf16(acc[0][2] * inv, acc[0][3] * inv);
          o.z = pack_bf16(acc[1][0] * inv, acc[1][1] * inv);
          o.w = pack_bf16(acc[1][2] * inv, acc[1][3] * inv);
          lds_write128<0>(to + (16 * ss + n) * OROW16 + och * 2, o);
        }
      }
    }
  };

  int it = 0, cur_c = -1;
  Tile112 prev = {0, 0, 0, false};
#pragma unroll 1
  while (has_tile(ccur)) {
    const Tile112 tl = next_tile(ccur);
    if (mma_role && tl.c != cur_c) {  // uniform: the walk enters another chunk
      load_state(tl.c);
      cur_c = tl.c;
    }
    wait_tiles(issued - 1 - it);
    __builtin_amdgcn_s_barrier();  // tile it has landed, every wave is done with tile it - 1 and its output tile is
                                   // complete (no fence: younger loads stay in flight)
    if (has_tile(icur)) {          // refill the ring entry of tile it - 1
      const Tile112 nl = next_tile(icur);
      issue(nl.start, nl.limit);
    }
    if (mma_role) mma_tile(it);
    if (it > 0) store_tile((it - 1) & 1, prev.start, prev.limit);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    prev = tl;
    ++it;
  }
  __builtin_amdgcn_s_barrier();
  store_tile((it - 1) & 1, prev.start, prev.limit);
}

// ----------------------------------------------------------------------------
// phase 2 with on-load transforms (q/k RMSNorm, rotary embedding).  grid.x over token ranges x heads, see head_unit,
// grid.y = batch; block 256: every wave loads, transforms, multiplies and stores, and two or three workgroups share
// a compute unit.
//
// As in the kernels above a workgroup walks ONE contiguous token range of a (batch, head), cut by token count
// whatever the chunking, in steps of 32 tokens that never straddle a chunk boundary; the state operands are
// rebuilt when the walk enters another chunk.  Global memory is touched in whole rows
// only: consecutive threads load consecutive 16-byte pieces of the tokens' 224-byte head rows
// (transforms applied once, here) into an LDS tile, every wave takes its MFMA B operands from that
// tile, results go to an LDS output tile and leave as whole rows again.  Tiles are double buffered,
// the next tile's loads are in flight during the MFMAs: one barrier per step.
// ----------------------------------------------------------------------------
constexpr int TT = 32;             // tokens per step
constexpr int QROWE = 136;          // LDS row stride of the 16-bit tiles, elements: 272 B = 68 banks, so the 16 tokens
                                   // of a b128 operand read land on 16 disjoint groups of 4 banks; pieces 14
                                   // and 15 of a row (the padded k range 112..127) stay zero
constexpr int OROWF = 116;        // row stride of the fp32 output tile, floats (same argument: 116 % 64 = 52)

template <bool OUT_F32, int PRE>
__global__ __launch_bounds__(256) void apply112_kernel(const uint16_t* __restrict__ Q, const float* __restrict__ state,
                                                       void* __restrict__ out,
                                                       const int32_t* __restrict__ chunk_starts, int N, int h,
                                                       int n_chunks, int range_tokens, int units,
                                                       int64_t q_stride_b,
                                                       int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n,
                                                       float eps, const QkPre pre) {
  constexpr int NQ = (PRE & 2) ? 2 : 1;  // with a rotary embedding: rotated (numerator) and unrotated (denominator) tiles
  constexpr int OT = OUT_F32 ? TT * OROWF * 2 : TT * QROWE;  // output tile, in 16-bit units
  __shared__ __attribute__((aligned(16))) uint16_t lds_q[2 * NQ * TT * QROWE];
  __shared__ __attribute__((aligned(16))) uint16_t lds_o[2 * OT];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  HeadUnit hu;
  if (!head_unit(blockIdx.x, units, h, hu)) return;  // uniform over the workgroup
  const int head = hu.head;
  const int b = blockIdx.y;
  const int r0 = hu.unit * range_tokens, r1 = min(N, r0 + range_tokens);
  if (r0 >= r1) return;  // uniform over the workgroup
  auto chunk_end = [&](int c) __attribute__((always_inline)) { return chunk_starts ? chunk_starts[c + 1] : N; };
  int c0 = 0;
  while (chunk_end(c0) <= r0) ++c0;  // the chunk of the range's first token (uniform; a few dozen chunks at most)
  const int n = lane & 15, g = lane >> 4;
  constexpr bool has_norm = (PRE & 1) != 0, has_rope = (PRE & 2) != 0;

  // A operands.  MFMA 16x16x32: A lane -> row lane%16, k = 8*(lane/16)+e.  Row r of row block rb of this
  // wave is output channel 32*wave + 8*(r/4) + 4*rb + r%4, so that a lane (token n, group g') ends up
  // with the 8 contiguous channels 32*wave + 8*g' .. +7 (registers s of blocks 0 and 1).  Block 2
  // carries ksum in every row.  Channels and k indices past 112 are zero.
  constexpr int NT = OUT_F32 ? 3 : 2;  // bf16 terms of an fp32 state value: 24 / 16 mantissa bits
  u32x4_t a[3][4][NT];                 // [row block][k block][term]
  auto load_state = [&](int c) __attribute__((always_inline)) {
    const float* sp = state + ((int64_t)(b * h + head) * n_chunks + c) * SE;
    // buffer loads: rows / k groups outside the head's state get an out-of-range offset and read as zero
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(sp), 0, SE * 4, 0x00020000);
#pragma unroll
    for (int rb = 0; rb < 3; ++rb) {
      const int ch = 32 * wave + 8 * (n >> 2) + 4 * rb + (n & 3);
      const int row = rb < 2 ? ch : DH;
      const bool row_ok = rb == 2 || ch < DH;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const int k0 = kb * 32 + 8 * g;
        const int off = (row_ok && k0 < DH) ? (row * DH + k0) * 4 : (int)0x80000000u;
        const f32x4_t x0 = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, off, 0, 0));
        const f32x4_t x1 = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, off + 16, 0, 0));
        const float x[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        split_terms<NT>(x, a[rb][kb]);
      }
    }
  };

  // tile load mapping: piece id = tid + 256 i (i < 2, id < 448): token id / 14, 16-byte piece id % 14
  int ld_tok[2], ld_ch[2];
  bool ld_ok[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int id = tid + 256 * i;
    ld_ok[i] = id < TT * NCH;
    ld_tok[i] = id / NCH;
    ld_ch[i] = id - ld_tok[i] * NCH;
  }
  const uint16_t* qp = Q + (int64_t)b * q_stride_b + head * DH;
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  const f32x4_t zerof = {0.f, 0.f, 0.f, 0.f};
  u32x4_t qreg[2], qw[2] = {zero4, zero4};
  float rin[2] = {0.f, 0.f};
  f32x4_t cs[2][2] = {{zerof, zerof}, {zerof, zerof}};
  if (has_norm) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (ld_ok[i]) qw[i] = *reinterpret_cast<const u32x4_t*>(pre.weight + head * DH + ld_ch[i] * 8);
  }
  auto issue = [&](int t, int t1) {  // the 32 tokens from t, those before t1
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int tok = t + ld_tok[i];
      const bool ok = ld_ok[i] && tok < t1;
      qreg[i] = ok ? *reinterpret_cast<const u32x4_t*>(qp + (int64_t)tok * q_stride_n + ld_ch[i] * 8) : zero4;
      if (has_norm) rin[i] = ok ? pre.rinv[(int64_t)b * N + tok] : 0.f;
      if (has_rope) {
        const float* rp = pre.rope + ((int64_t)min(tok, t1 - 1) * (DH / 2) + ld_ch[i] * 4) * 2;
        cs[i][0] = ok ? *reinterpret_cast<const f32x4_t*>(rp) : zerof;
        cs[i][1] = ok ? *reinterpret_cast<const f32x4_t*>(rp + 4) : zerof;
      }
    }
  };
  auto stage = [&](int buf) {  // registers -> LDS tile(s); tokens past the range are zeros
    uint16_t* td = lds_q + buf * NQ * TT * QROWE;  // unrotated: the denominator operand (and the numerator without rope)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (!ld_ok[i]) continue;
      u32x4_t x = qreg[i];
      if (has_norm) x = rms_scale8(x, rin[i], qw[i]);
      x = relu_pk16(x);
      *reinterpret_cast<u32x4_t*>(td + ld_tok[i] * QROWE + ld_ch[i] * 8) = x;
      if (has_rope)
        *reinterpret_cast<u32x4_t*>(td + TT * QROWE + ld_tok[i] * QROWE + ld_ch[i] * 8) = rope8(x, cs[i][0], cs[i][1]);
    }
  };

  const int och = 32 * wave + 8 * g;  // this lane's 8 output channels
  for (int i = tid; i < 2 * NQ * TT * 3; i += 256)  // pieces 14..16 of every q tile row: written once, as zeros
    *reinterpret_cast<u32x4_t*>(lds_q + (i / 3) * QROWE + (NCH + i % 3) * 8) = zero4;
  auto has_tile = [&](const TileCur& cur) __attribute__((always_inline)) { return cur.t < r1; };
  auto next_tile = [&](TileCur& cur) __attribute__((always_inline)) {
    Tile112 tl;
    tl.start = cur.t;
    tl.limit = cur.seg_end;
    tl.c = cur.c;
    const int nt = min(cur.t + TT, cur.seg_end);
    tl.last = nt == cur.seg_end;
    cur.t = nt;
    if (tl.last && nt < r1) {
      ++cur.c;
      cur.seg_end = min(chunk_end(cur.c), r1);
    }
    return tl;
  };
  TileCur icur = {r0, c0, min(chunk_end(c0), r1)}, ccur = icur;
  {
    const Tile112 ti = next_tile(icur);
    issue(ti.start, ti.limit);
  }
  stage(0);
  if (has_tile(icur)) {
    const Tile112 ti = next_tile(icur);
    issue(ti.start, ti.limit);
  }
  __syncthreads();
  int cur_c = -1;
  for (int buf = 0; has_tile(ccur); buf ^= 1) {
    const Tile112 tl = next_tile(ccur);
    const int t = tl.start, t1 = tl.limit;
    if (tl.c != cur_c) {  // uniform: the walk enters another chunk
      load_state(tl.c);
      cur_c = tl.c;
    }
    const uint16_t* td = lds_q + buf * NQ * TT * QROWE;
    const uint16_t* tb = has_rope ? td + TT * QROWE : td;
    uint16_t* to = lds_o + buf * OT;
#pragma unroll
    for (int ss = 0; ss < TT / 16; ++ss) {
      u32x4_t qd[4], qb[4];
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const int off = (16 * ss + n) * QROWE + (kb * 4 + g) * 8;  // pieces 14, 15 (kb = 3, g >= 2) hold zeros
        qb[kb] = *reinterpret_cast<const u32x4_t*>(tb + off);
        if (has_rope) qd[kb] = *reinterpret_cast<const u32x4_t*>(td + off);
      }
      f32x4_t acc[3];
#pragma unroll
      for (int rb = 0; rb < 3; ++rb) {
        f32x4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int term = NT - 1; term >= 0; --term)  // smallest term first
#pragma unroll
          for (int kb = 0; kb < 4; ++kb) s = mfma_16x16x32_bf16(a[rb][kb][term], (has_rope && rb == 2) ? qd[kb] : qb[kb], s);
        acc[rb] = s;
      }
      if (och < DH) {
        const float den = acc[2][0] + eps;
        if (OUT_F32) {
          f32x4_t o0, o1;
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            o0[s] = acc[0][s] / den;
            o1[s] = acc[1][s] / den;
          }
          float* op = reinterpret_cast<float*>(to) + (16 * ss + n) * OROWF + och;
          *reinterpret_cast<f32x4_t*>(op) = o0;
          *reinterpret_cast<f32x4_t*>(op + 4) = o1;
        } else {
          const float inv = __builtin_amdgcn_rcpf(den);
          u32x4_t o;
          o.x = pack_bf16(acc[0][0] * inv, acc[0][1] * inv);
          o.y = pack_bf16(acc[0][2] * inv, acc[0][3] * inv);
          o.z = pack_bf16(acc[1][0] * inv, acc[1][1] * inv);
          o.w = pack_bf16(acc[1][2] * inv, acc[1][3] * inv);
          *reinterpret_cast<u32x4_t*>(to + (16 * ss + n) * QROWE + och) = o;
        }
      }
    }
    // next tile: registers -> the other q tile (its last readers passed the previous barrier); loads of the one after
    if (has_tile(ccur)) {
      stage(buf ^ 1);
      if (has_tile(icur)) {
        const Tile112 ti = next_tile(icur);
        issue(ti.start, ti.limit);
      }
    }
    __syncthreads();
    // this step's output tile leaves as whole rows (it is next written two steps from now, behind the next barrier)
    if (OUT_F32) {
      float* ob = reinterpret_cast<float*>(out) + (int64_t)b * o_stride_b + head * DH;
      const float* tf = reinterpret_cast<const float*>(to);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int id = tid + 256 * i, tok = id / (2 * NCH), piece = id - tok * (2 * NCH);
        if (id < TT * 2 * NCH && t + tok < t1)
          *reinterpret_cast<f32x4_t*>(ob + (int64_t)(t + tok) * o_stride_n + piece * 4) =
              *reinterpret_cast<const f32x4_t*>(tf + tok * OROWF + piece * 4);
      }
    } else {
      uint16_t* ob = reinterpret_cast<uint16_t*>(out) + (int64_t)b * o_stride_b + head * DH;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (ld_ok[i] && t + ld_tok[i] < t1)
          *reinterpret_cast<u32x4_t*>(ob + (int64_t)(t + ld_tok[i]) * o_stride_n + ld_ch[i] * 8) =
              *reinterpret_cast<const u32x4_t*>(to + ld_tok[i] * QROWE + ld_ch[i] * 8);
      }
    }
  }
}

// MI355X: 256 compute units (a constant, so plans do not depend on the host the call is made on)
constexpr int compute_units112() { return 256; }

struct Plan112 {
  int range_tokens, nrec;  // tokens per range; records per (batch, head)
};
// One workgroup (eight waves) per compute unit: each (batch, head) is cut into 256 / (B h) token ranges of equal
// length, whatever the chunking.  The plan must not depend on N (the workspace query does not know it), so the
// length comes from the upper bound n_chunks * max_chunk_tokens, and so does the number of ranges the records
// are sized for.
Plan112 plan112(int B, int h, int n_chunks, int max_chunk_tokens) {
  const int64_t n_ub = (int64_t)n_chunks * max_chunk_tokens;
  int nr = compute_units112() / (B * h);  // rounding down: 260 workgroups on 256 CUs would take two rounds
  if (nr < 1) nr = 1;
  int64_t L = ((n_ub + nr - 1) / nr + 63) / 64 * 64;
  if (L < 256) L = 256;
  Plan112 pl;
  pl.range_tokens = (int)std::min<int64_t>(L, 1 << 30);
  pl.nrec = (int)((n_ub + pl.range_tokens - 1) / pl.range_tokens) + n_chunks - 1;  // index range + chunk
  return pl;
}

struct Reduce112Plan {
  int cl, threads, nblk;  // chunks per workgroup (power of two <= 16), its size, workgroups per (batch, head)
};
Reduce112Plan reduce112_plan(int n_chunks) {
  Reduce112Plan p;
  p.cl = 1;
  while (p.cl < n_chunks && p.cl < 16) p.cl *= 2;
  const int nq = std::max(64, 256 / p.cl);
  p.threads = nq * p.cl;
  p.nblk = (SE / 4 + nq - 1) / nq;
  return p;
}

}  // namespace

size_t workspace_bytes112(int B, int h, int n_chunks, int max_chunk_tokens) {
  const Plan112 pl = plan112(B, h, n_chunks, max_chunk_tokens);
  return (size_t)B * h * pl.nrec * SE * sizeof(float);  // the records are always written
}

int launch_state112(const void* k, const void* v, float* state, void* workspace, size_t workspace_bytes, int B, int N,
                    int h, int64_t stride_b, int64_t stride_n, const int32_t* chunk_starts, int n_chunks,
                    int max_chunk_tokens, int causal, int io_dtype, const QkPre& pre, hipStream_t s) {
  if (io_dtype != SANA_DT_BF16 && io_dtype != SANA_DT_F16) return SANA_ERR_DTYPE;
  const bool use_pre = pre.rinv || pre.rope;
  if (use_pre && io_dtype != SANA_DT_BF16) return SANA_ERR_DTYPE;
  // the kernel addresses one batch entry's tokens with 32-bit byte offsets (buffer loads)
  if ((int64_t)N * stride_n * 2 >= (int64_t)1 << 31 || (int64_t)N * DH * 4 >= (int64_t)1 << 31) return SANA_ERR_SHAPE;
  const Plan112 pl = plan112(B, h, n_chunks, max_chunk_tokens);
  const size_t need = workspace_bytes112(B, h, n_chunks, max_chunk_tokens);
  if (!workspace || workspace_bytes < need) return SANA_ERR_WORKSPACE;
  if (!aligned16(workspace)) return SANA_ERR_ALIGN;
  float* part = static_cast<float*>(workspace);
  const int nranges = (N + pl.range_tokens - 1) / pl.range_tokens;
  if (nranges + n_chunks - 1 > pl.nrec) return SANA_ERR_SHAPE;  // N beyond n_chunks * max_chunk_tokens
  const int64_t units = nranges, nwg = head_unit_grid(units, h);
  if (nwg > 0x7fffffff || units * ((h + 3) / 4) * 8 > 0x7fffffff || B > 65535 || (int64_t)B * h > (1 << 22))
    return SANA_ERR_SHAPE;
  dim3 grid((unsigned)nwg, (unsigned)B);
  const uint16_t* kp = static_cast<const uint16_t*>(k);
  const uint16_t* vp = static_cast<const uint16_t*>(v);
#define SANA_ST112(T, PRE)                                                                                        \
  hipLaunchKernelGGL((state112_kernel<T, PRE>), grid, dim3(512), 0, s, kp, vp, part, chunk_starts, N, h, pl.nrec, \
                     pl.range_tokens, (int)units, stride_b, stride_n, pre)
  const int mode = (pre.rinv ? 1 : 0) | (pre.rope ? 2 : 0);
  if (io_dtype == SANA_DT_F16) SANA_ST112(F16, 0);
  else if (mode == 3) SANA_ST112(BF16, 3);
  else if (mode == 2) SANA_ST112(BF16, 2);
  else if (mode == 1) SANA_ST112(BF16, 1);
  else SANA_ST112(BF16, 0);
#undef SANA_ST112
  if (hipGetLastError() != hipSuccess) return SANA_ERR_LAUNCH;
  const Reduce112Plan rp = reduce112_plan(n_chunks);
  hipLaunchKernelGGL(reduce112_kernel, dim3((unsigned)((int64_t)B * h * rp.nblk)), dim3(rp.threads), 0, s, part, state, chunk_starts,
                     N, n_chunks, pl.nrec, pl.range_tokens, (causal && n_chunks > 1) ? 1 : 0, rp.cl, rp.nblk);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

int launch_scan112(float* state, int B, int h, int n_chunks, hipStream_t s) {
  if ((int64_t)B * h > (1 << 22)) return SANA_ERR_SHAPE;
  const Reduce112Plan rp = reduce112_plan(n_chunks);
  hipLaunchKernelGGL(reduce112_kernel, dim3((unsigned)((int64_t)B * h * rp.nblk)), dim3(rp.threads), 0, s, state, state,
                     static_cast<const int32_t*>(nullptr), 0, n_chunks, n_chunks, 0, 1, rp.cl, rp.nblk);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

static int launch_apply112_pre(const void* q, const float* state, void* out, int B, int N, int h, int64_t q_stride_b,
                    int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n, const int32_t* chunk_starts,
                    int n_chunks, int max_chunk_tokens, float eps, int io_dtype, int out_dtype, const QkPre& pre,
                    hipStream_t s) {
  if (io_dtype != SANA_DT_BF16) return SANA_ERR_DTYPE;
  // Tokens per workgroup (a multiple of the 32-token step), whatever the chunking: long enough to pay for building
  // the state operands (worth ~48 tokens of work, once per chunk the range touches), and such that the grid fills
  // whole rounds of the chip -- 3 workgroups per CU fit (2 with transforms or fp32 output: registers), so 4 rounds
  // of 256 tokens with the last one a third full lose to 3 rounds of 288, and at the video shape one round of
  // 1312-token ranges beats three or four rounds of ~400 by 6 - 8 %.
  const int mode = (pre.rinv ? 1 : 0) | (pre.rope ? 2 : 0);
  int range_tokens = 256;
  {
    const int64_t slots = (int64_t)compute_units112() * ((mode || out_dtype == SANA_DT_F32) ? 2 : 3);
    double best = 1e30;
    for (int t = 192; t <= 2048; t += 32) {
      const int64_t wgs = (int64_t)((N + t - 1) / t) * B * h;
      const double builds = 1.0 + (double)t / std::max(max_chunk_tokens, 1);  // chunks a range touches, roughly
      const double cost = (double)((wgs + slots - 1) / slots) * (t + 48.0 * builds);
      if (cost < best) {
        best = cost;
        range_tokens = t;
      }
    }
  }
  const int64_t units = (N + range_tokens - 1) / range_tokens, total = head_unit_grid(units, h);
  if (total > 0x7fffffff || units * ((h + 3) / 4) * 8 > 0x7fffffff || B > 65535) return SANA_ERR_SHAPE;
  dim3 grid((unsigned)total, (unsigned)B);
  const uint16_t* qp = static_cast<const uint16_t*>(q);
#define SANA_AP112(F32, PRE)                                                                                         \
  hipLaunchKernelGGL((apply112_kernel<F32, PRE>), grid, dim3(256), 0, s, qp, state, out, chunk_starts, N, h, n_chunks, \
                     range_tokens, (int)units, q_stride_b, q_stride_n, o_stride_b, o_stride_n, eps, pre)
  if (out_dtype == SANA_DT_F32) {
    if (mode == 3) SANA_AP112(true, 3);
    else if (mode == 2) SANA_AP112(true, 2);
    else if (mode == 1) SANA_AP112(true, 1);
    else SANA_AP112(true, 0);
  } else {
    if (mode == 3) SANA_AP112(false, 3);
    else if (mode == 2) SANA_AP112(false, 2);
    else if (mode == 1) SANA_AP112(false, 1);
    else SANA_AP112(false, 0);
  }
#undef SANA_AP112
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}


int launch_apply112(const void* q, const float* state, void* out, int B, int N, int h, int64_t q_stride_b,
                    int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n, const int32_t* chunk_starts,
                    int n_chunks, int max_chunk_tokens, float eps, int io_dtype, int out_dtype, const QkPre& pre,
                    hipStream_t s) {
  if (io_dtype != SANA_DT_BF16) return SANA_ERR_DTYPE;
  const int mode = (pre.rinv ? 1 : 0) | (pre.rope ? 2 : 0);
  // the streaming kernel addresses one batch entry's tokens with 32-bit byte offsets (buffer loads)
  if (mode != 0 || (int64_t)N * q_stride_n * 2 >= (int64_t)1 << 31)
    return launch_apply112_pre(q, state, out, B, N, h, q_stride_b, q_stride_n, o_stride_b, o_stride_n, chunk_starts, n_chunks,
                               max_chunk_tokens, eps, io_dtype, out_dtype, pre, s);
  // one workgroup (eight waves) per compute unit: 256 / (B h) token ranges of equal length per (batch, head)
  int nr = compute_units112() / (B * h);
  if (nr < 1) nr = 1;
  int64_t L = (((int64_t)N + nr - 1) / nr + TILE - 1) / TILE * TILE;
  if (L < 256) L = 256;
  const int range_tokens = (int)L;
  const int nranges = (N + range_tokens - 1) / range_tokens;
  const int64_t units = nranges, total = head_unit_grid(units, h);
  if (total > 0x7fffffff || units * ((h + 3) / 4) * 8 > 0x7fffffff || B > 65535) return SANA_ERR_SHAPE;
  (void)max_chunk_tokens;
  dim3 grid((unsigned)total, (unsigned)B);
  const uint16_t* qp = static_cast<const uint16_t*>(q);
#define SANA_AP112S(F32)                                                                                            \
  hipLaunchKernelGGL((apply112_stream_kernel<F32>), grid, dim3(512), 0, s, qp, state, out, chunk_starts, N, h, n_chunks, \
                     range_tokens, (int)units, q_stride_b, q_stride_n, o_stride_b, o_stride_n, eps)
  if (out_dtype == SANA_DT_F32) SANA_AP112S(true);
  else SANA_AP112S(false);
#undef SANA_AP112S
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

}  // namespace sana

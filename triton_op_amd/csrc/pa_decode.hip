// Split-KV paged-attention decode for MI355X (gfx950 / CDNA4): the two partition kernels, the reduce
// kernel and the C ABI declared in include/pa_decode.h.
//
// pa_partition_kernel (up to 16 query rows per kv head, and every bf16 cache) is described first;
// pa_partition_shared_kernel (17..64 rows over an FP8 cache) does the same arithmetic with the row tiles
// of a kv head sharing one pass over the pages through LDS, and is described where it is defined.
//
// Work decomposition.  A workgroup of 1, 2 or 4 waves owns one item: (sequence, partition, 16-row
// query tile, kv head).  Each wave streams a contiguous slice of the partition in steps of 64 tokens
// (four 16-token tiles) with private online-softmax state (m, l, O); the waves merge through LDS at the
// end.  A sequence that fits in one partition gets its final output from this kernel directly.
//
//   K tile  (16 tokens x 128 dims): every lane loads 16 bytes = one [token][16-byte chunk] cell of
//           the cache; lanes 0-15 are the 16 tokens of a page, lane>>4 picks the chunk row, so a
//           wave load covers 4 x 256 contiguous bytes in storage order.  The dot product does not care
//           in which order the head dimension is summed, so the query operand is built in the order
//           the loads deliver it.
//   S^T = K Q^T: tokens are the M rows, query rows (GQA group x MTP position, padded to 16) are
//           the N columns, so a lane ends up with 4 tokens of ONE query row per tile and the softmax
//           max/sum need only two cross-lane steps (lane^16, lane^32).
//   V tile  (128 dims x 16 tokens): every lane loads 16 bytes = 16 tokens of one head dim, lanes
//           0-15 are 16 consecutive dims (256 contiguous bytes with block 16), lane>>4 picks one of
//           the four tiles of the step.  O^T = V^T P^T accumulates in 8 MFMA tiles of [16 dims x 16 rows].
//
// FP8 cache: the cache bytes are MFMA operands as they are (v_mfma_f32_16x16x128_f8f6f4 for Q K^T,
// v_mfma_f32_16x16x32_fp8_fp8 for P V); the bf16 query and P are each carried as an FP8 head plus an
// FP8 residual (x*c = hi + lo, every product exact in the f32 accumulator), about 2^-8 relative per
// element, so there is no FP8->bf16 conversion work at all; P reaches the B-operand layout through a 4x4
// (lane group x register) transpose with v_permlane{16,32}_swap, not through LDS.  Per-tensor scales
// fold into the softmax scale (K) and the epilogue (V); per-token scales multiply S and P in f32.
// bf16 cache: bf16 MFMA (v_mfma_f32_16x16x32_bf16), P through a wave-private LDS tile.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "../../include/pa_decode.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(8))) int i32x8;

constexpr int kHeadSize = 128;
constexpr int kStepTokens = 64;     // tokens per pipeline step (4 tiles of 16)
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kPRowBytes = 144;     // 64 tokens * 2 B + 16 B pad per query row of the P tile

union Bf16x8Bits {
  bf16x8 v;
  bf16x2 p[4];
  u32x4 u;
};

// two FP8 e4m3fn bytes -> two bf16, exactly (an e4m3 value has 3 mantissa bits, bf16 keeps 7)
__device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t word, bool high_half) {
  // v_cvt_pk_f32_fp8, then keep the upper 16 bits of each f32
  f32x2 f = high_half ? __builtin_amdgcn_cvt_pk_f32_fp8((int)word, true)
                      : __builtin_amdgcn_cvt_pk_f32_fp8((int)word, false);
  return __builtin_amdgcn_perm(__float_as_uint(f[1]), __float_as_uint(f[0]), 0x07060302u);
}

__device__ __forceinline__ bf16x8 fp8x8_to_bf16x8(uint32_t lo, uint32_t hi) {
  Bf16x8Bits r;
  r.u[0] = fp8x2_to_bf16x2(lo, false);
  r.u[1] = fp8x2_to_bf16x2(lo, true);
  r.u[2] = fp8x2_to_bf16x2(hi, false);
  r.u[3] = fp8x2_to_bf16x2(hi, true);
  return r.v;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  union {
    bf16x2 v;
    uint32_t u;
  } r;
  r.v[0] = (__bf16)a;
  r.v[1] = (__bf16)b;
  return r.u;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }

// wave-uniform 32-bit load through the scalar (constant) path: no VGPR, no vmcnt slot
__device__ __forceinline__ int sload_i32(const int* p) {
  return *reinterpret_cast<const __attribute__((address_space(4))) int*>(reinterpret_cast<uintptr_t>(p));
}
__device__ __forceinline__ float sload_f32(const float* p) {
  return *reinterpret_cast<const __attribute__((address_space(4))) float*>(reinterpret_cast<uintptr_t>(p));
}

// max / sum over the four lanes {l, l^16, l^32, l^48}: v_permlane{16,32}_swap exchange 16- and
// 32-lane halves inside the VALU (no LDS round trip)
__device__ __forceinline__ float quad_row_max(float x) {
  uint32_t u = __float_as_uint(x);
  auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  u = __float_as_uint(x);
  auto b = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_row_sum(float x) {
  uint32_t u = __float_as_uint(x);
  auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  u = __float_as_uint(x);
  auto b = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// 4x4 transpose over (lane group l>>4, register): afterwards register k of lane group g holds what
// register g of lane group k held
__device__ __forceinline__ void quad_transpose(uint32_t (&d)[4]) {
  auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
  auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
  auto s01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
  auto s23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
  d[0] = s01[0];
  d[1] = s01[1];
  d[2] = s23[0];
  d[3] = s23[1];
}

// keep the first `n` (0..16) bytes of a 16-byte vector, zero the rest
__device__ __forceinline__ u32x4 keep_first_bytes(u32x4 v, int n) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    int k = n - 4 * w;
    uint32_t m = k >= 4 ? 0xffffffffu : (k <= 0 ? 0u : ((1u << (8 * k)) - 1u));
    v[w] &= m;
  }
  return v;
}

// Writes one 16-row x 128-dim f32 tile of O^T (acc[db][r] = head dim 16*db + 4*kg + r of row li) as bf16
// rows of the partial output.  The tile is transposed through a wave-private LDS buffer so that every
// store instruction writes four whole 256-byte rows (16 bytes per lane) instead of 32-byte fragments.
constexpr int kORowBytes = 272;  // 256 B of bf16 + 16 B pad
__device__ __forceinline__ void store_partial_tile(char* lds, const f32x4 (&acc)[8], float inv, char* dst,
                                                   int64_t row_stride_bytes, char* dst2, int64_t row_stride2_bytes,
                                                   int rows_to_write, int lane) {
  const int li = lane & 15, kg = lane >> 4;
#pragma unroll
  for (int db = 0; db < 8; ++db) {
    const f32x4 o = acc[db] * inv;
    u32x2 pk;
    pk[0] = pack_bf16x2(o[0], o[1]);
    pk[1] = pack_bf16x2(o[2], o[3]);
    *reinterpret_cast<u32x2*>(lds + li * kORowBytes + (16 * db + 4 * kg) * 2) = pk;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * i + kg;
    const u32x4 v = *reinterpret_cast<const u32x4*>(lds + r * kORowBytes + li * 16);
    if (r < rows_to_write) {
      *reinterpret_cast<u32x4*>(dst + (int64_t)r * row_stride_bytes + li * 16) = v;
      if (dst2) *reinterpret_cast<u32x4*>(dst2 + (int64_t)r * row_stride2_bytes + li * 16) = v;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// One step's worth of cache data, as loaded (still FP8 / bf16 bit patterns).
template <int KVT, bool PER_TOKEN>
struct StepData {
  static constexpr int NKL = KVT == PA_DTYPE_FP8_E4M3FN ? 2 : 4;  // 16-byte K loads per lane per tile
  static constexpr int NVL = KVT == PA_DTYPE_FP8_E4M3FN ? 1 : 2;  // 16-byte V loads per lane per 16 dims
  u32x4 k[4][NKL];
  u32x4 v[8][NVL];
  f32x4 ks[PER_TOKEN ? 4 : 1];
  f32x4 vs[PER_TOKEN ? 4 : 1];
};

// The partition kernel.  OCC is the number of waves per SIMD the register budget is cut for.
//
// Software pipeline of one wave (each line is issued in order; loads return in order):
//   QK(s)      needs K(s)            -> then K(s+1) is loaded into the registers K(s) just left
//   softmax(s)                          (K(s+1) and V(s) in flight)
//   PV(s)      needs V(s)            -> then V(s+1) is loaded into the registers V(s) just left
// so about one step (16 KiB) of cache data per wave is in flight at any time without a second
// register copy.  Steps that need no masking and have a successor run in a branch-free loop, so
// the compiler's vmcnt waits stay partial; the last step(s) go through the masked variants.
//
// BS16 (block size 16) turns every stride inside a page into a compile-time constant, so the loads
// of a tile share one address register pair and differ by immediate offsets.
constexpr int kQueueMaxSeqs = 2048;  // sequences the item table of the queued launch can hold

template <int NT, int KVT, bool PER_TOKEN, bool BS16, int WAVES, int OCC, bool QUEUE>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void pa_partition_kernel(const PaDecodeArgs a) {
  constexpr bool kFp8 = KVT == PA_DTYPE_FP8_E4M3FN;
  constexpr bool FP8MATH = kFp8;  // an FP8 cache is multiplied on the FP8 MFMAs, a bf16 cache on the bf16 ones
  constexpr int esz = kFp8 ? 1 : 2;
  typedef StepData<KVT, PER_TOKEN> SD;

  __shared__ __attribute__((aligned(16))) char p_lds[FP8MATH ? 1 : WAVES][FP8MATH ? 1 : NT][FP8MATH ? 16 : 16 * kPRowBytes];
  __shared__ __attribute__((aligned(16))) char o_lds[1][16 * kORowBytes];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15;
  const int kg = lane >> 4;

  // ---- which (sequence, head, partition): all wave-uniform -----------------------------------------
  const int P = a.max_num_partitions;
  const int Hkv = a.num_kv_heads;
  // The WAVES waves of a workgroup share one item: (sequence, partition, group of NT 16-row query tiles,
  // kv head).  The head varies fastest, so the workgroups that stream the same pages (the other heads, and
  // the other row tiles of the same head, 8 ids apart with 8 kv heads: the same XCD and L2) run together.
  const int Ge = a.q_len * a.group_size;  // rows per kv head in the buffers
  const int RT = (Ge + 16 * NT - 1) / (16 * NT);

  // QUEUE: a resident grid of workgroups pulls live items from a counter in the caller's workspace.  Only
  // partitions a sequence reaches and row tiles that hold real query rows are items, so a ragged batch
  // launches no workgroup that would exit at once (each of those still costs a wave slot for a
  // microsecond).  Every workgroup builds, once, the exclusive prefix sum of the per-sequence item counts
  // in LDS and decodes an item index by binary search in it.
  __shared__ int q_cum[QUEUE ? kQueueMaxSeqs + 1 : 1];
  __shared__ int q_ctx[QUEUE ? kQueueMaxSeqs : 1];
  __shared__ int q_tiles[QUEUE ? kQueueMaxSeqs : 1];
  __shared__ int q_item;
  int total_items = 0;
  if constexpr (QUEUE) {
    if (wave == 0) {
      int running = 0;
      for (int b0 = 0; b0 < a.num_seqs; b0 += 64) {
        const int bb = b0 + lane;
        const int c = bb < a.num_seqs ? a.context_lens[bb] : 0;
        int np = (c + a.partition_size - 1) / a.partition_size;
        np = np < 0 ? 0 : (np > P ? P : np);
        const int ql = bb < a.num_seqs ? (a.q_lens ? a.q_lens[bb] : a.q_len) : 0;
        int tiles = (ql * a.group_size + 16 * NT - 1) / (16 * NT);
        tiles = tiles > RT ? RT : tiles;
        const int n = np * tiles;
        int x = n;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int y = __shfl_up(x, d);
          if (lane >= d) x += y;
        }
        if (bb < a.num_seqs) {
          q_cum[bb] = running + x - n;
          q_ctx[bb] = c;
          q_tiles[bb] = tiles;
        }
        running += __builtin_amdgcn_readlane(x, 63);
      }
      if (lane == 0) q_cum[a.num_seqs] = running;
    }
    __syncthreads();
    total_items = q_cum[a.num_seqs] * Hkv;
  }

  for (;;) {  // one pass without the queue
  int h, rt, b, part, tiles_b = RT;
  if constexpr (QUEUE) {
    if (threadIdx.x == 0) q_item = atomicAdd(a.workspace, 1);
    __syncthreads();
    const int item = __builtin_amdgcn_readfirstlane(q_item);
    __syncthreads();  // everybody has read q_item (and is done with the LDS buffers of the previous item)
    if (item >= total_items) break;
    h = item % Hkv;
    const int j = item / Hkv;
    int lo = 0, hi = a.num_seqs;  // q_cum[lo] <= j < q_cum[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (__builtin_amdgcn_readfirstlane(q_cum[mid]) <= j)
        lo = mid;
      else
        hi = mid;
    }
    b = lo;
    tiles_b = __builtin_amdgcn_readfirstlane(q_tiles[b]);
    const int local = j - __builtin_amdgcn_readfirstlane(q_cum[b]);
    part = local / tiles_b;
    rt = local - part * tiles_b;
  } else {
    // The partition index varies slowest: in a ragged batch the partitions that only the longest
    // sequences reach (workgroups that exit at once for everybody else) come last.
    const long long wid = blockIdx.x;
    h = (int)(wid % Hkv);
    rt = (int)((wid / Hkv) % RT);
    b = (int)((wid / ((long long)Hkv * RT)) % a.num_seqs);
    part = (int)(wid / ((long long)Hkv * RT * a.num_seqs));
  }
  const int row0 = 16 * NT * rt;  // first query row of this workgroup inside its kv-head group
  do {  // the body of one item; `break` leaves it

  const int ctx = sload_i32(a.context_lens + b);
  const int wg_start = part * a.partition_size;
  if (wg_start >= ctx) break;
  const int wg_end = min(wg_start + a.partition_size, ctx);
  // The waves take the partition's 64-token steps round robin (wave w: steps w, w + WAVES, ...), so at any
  // time the workgroup reads WAVES * 64 consecutive tokens: with large blocks that is whole 128-byte lines of
  // every V row and long runs of every K chunk row, requested by the waves together.  A wave with no step
  // idles until the merge.
  const int wg_steps = (wg_end - wg_start + kStepTokens - 1) / kStepTokens;
  constexpr int kWaveStride = WAVES * kStepTokens;
  const int part_start = wg_start + wave * kStepTokens;
  const bool active = part_start < wg_end;
  const int G = a.group_size;
  const int qb = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
  const int rows_valid = qb * G;
  if (row0 >= rows_valid) {
    // only padding rows (a ragged batch): nothing to stream; the rows read as "no visible key"
    if (wave == 0) {
      const int64_t eo = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (int64_t)part * a.stride_es_p;
      char* tp = (char*)a.tmp_output + ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h +
                                        (int64_t)part * a.stride_tmp_p) * 2;
      char* op = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2;
      const bool dir = ctx <= a.partition_size && a.output != nullptr && a.sinks == nullptr;
      for (int r = row0 + kg; r < row0 + 16 * NT && r < Ge; r += 4) {
        if (li == 0) {
          a.max_logits[eo + r] = -INFINITY;
          a.exp_sums[eo + r] = 0.f;
        }
        *reinterpret_cast<u32x4*>(tp + (int64_t)r * a.stride_tmp_g * 2 + li * 16) = u32x4{0, 0, 0, 0};
        if (dir) *reinterpret_cast<u32x4*>(op + (int64_t)r * a.stride_out_h * 2 + li * 16) = u32x4{0, 0, 0, 0};
      }
    }
    break;
  }

  // ---- cache addressing -------------------------------------------------------------------------------
  const int log2_bs = 31 - __builtin_clz(a.block_size);
  const int bs_mask = a.block_size - 1;
  const char* kbase = (const char*)a.key_cache + (int64_t)h * a.stride_k_h * esz;
  const char* vbase = (const char*)a.value_cache + (int64_t)h * a.stride_v_h * esz;
  const int64_t k_block_bytes = a.stride_k_b * esz;
  const int64_t v_block_bytes = a.stride_v_b * esz;
  const float* ksbase = PER_TOKEN ? a.key_scale + (int64_t)h * a.stride_kvscale_h : nullptr;
  const float* vsbase = PER_TOKEN ? a.value_scale + (int64_t)h * a.stride_kvscale_h : nullptr;
  const uint32_t k_chunk_bytes = BS16 ? 256u : (uint32_t)(a.stride_k_c * esz);
  uint32_t k_lane_off[SD::NKL];  // per-lane byte offset of K load ld inside a tile
#pragma unroll
  for (int ld = 0; ld < SD::NKL; ++ld) k_lane_off[ld] = (uint32_t)(kg * k_chunk_bytes + li * 16) + 4 * ld * k_chunk_bytes;
  // V: byte offset of this lane's head dim inside a tile, distance of the second 8-token half
  // (bf16 only) and, for the transposed layout, of consecutive 16-token tiles of a page
  // (with block size 16 the plain and the transposed FP8 layouts are the same bytes; for bf16 they
  // differ, so the constant-stride form is used for the plain layout only)
  const bool vt = a.v_transposed;
  const uint32_t v_row_bytes = BS16 ? 16u * esz : (vt ? 16u : (uint32_t)(a.stride_v_2 * esz));
  const uint32_t v_half_bytes = BS16 ? 16u : (vt ? (uint32_t)(a.stride_v_2 * esz) : 16u);
  const int64_t v_tile_bytes = BS16 ? 16 * esz : (vt ? a.stride_v_2 * esz * esz : 16 * esz);
  uint32_t v_lane_off[8];
#pragma unroll
  for (int db = 0; db < 8; ++db) v_lane_off[db] = li * v_row_bytes + 16 * db * v_row_bytes;

  const int* bt = a.block_tables + (int64_t)b * a.stride_bt_s;
  const int last_tile_tok = (wg_end - 1) & ~15;  // first token of the last tile that holds a live token

  // page ids of the four tiles of the step that starts at token tok0 (scalar loads; tiles past the
  // last live one repeat it, so no block-table slot or page beyond the sequence is ever touched)
  struct Pages {
    int p[4];
    int off[4];  // token offset of the tile inside its page
  };
  auto load_pages = [&](int tok0) {
    Pages pg;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int t = tok0 + 16 * j;
      t = t > last_tile_tok ? last_tile_tok : t;
      pg.p[j] = sload_i32(bt + (t >> log2_bs));
      pg.off[j] = t & bs_mask;
    }
    return pg;
  };
  auto issue_k = [&](SD& sd, const Pages& pg) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const char* tb = kbase + (int64_t)pg.p[j] * k_block_bytes + (int64_t)pg.off[j] * 16;
#pragma unroll
      for (int ld = 0; ld < SD::NKL; ++ld) sd.k[j][ld] = load16(tb + k_lane_off[ld]);
      if constexpr (PER_TOKEN) {
        const int64_t so = (int64_t)pg.p[j] * a.stride_kvscale_b + pg.off[j] + 4 * kg;
        sd.ks[j] = *reinterpret_cast<const f32x4*>(ksbase + so);
      }
    }
  };
  auto issue_v = [&](SD& sd, const Pages& pg) {
    // lane group kg owns tile kg of the step
    const int page = kg == 0 ? pg.p[0] : (kg == 1 ? pg.p[1] : (kg == 2 ? pg.p[2] : pg.p[3]));
    const int off = kg == 0 ? pg.off[0] : (kg == 1 ? pg.off[1] : (kg == 2 ? pg.off[2] : pg.off[3]));
    const char* tb = vbase + (int64_t)page * v_block_bytes + (int64_t)(off >> 4) * v_tile_bytes;
#pragma unroll
    for (int db = 0; db < 8; ++db) {
#pragma unroll
      for (int hf = 0; hf < SD::NVL; ++hf) sd.v[db][hf] = load16(tb + v_lane_off[db] + hf * v_half_bytes);
    }
    if constexpr (PER_TOKEN) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t so = (int64_t)pg.p[j] * a.stride_kvscale_b + pg.off[j] + 4 * kg;
        sd.vs[j] = *reinterpret_cast<const f32x4*>(vsbase + so);
      }
    }
  };

  // ---- first loads go out before anything else is set up ---------------------------------------------
  const int n_steps = active ? (wg_steps - wave + WAVES - 1) / WAVES : 0;
  SD buf_a;  // one step of cache data, refilled in place for the next step
  if (active) {
    Pages pg0 = load_pages(part_start);
    issue_k(buf_a, pg0);
    issue_v(buf_a, pg0);
  }

  // ---- per-lane row bookkeeping -------------------------------------------------------------------------
  int limit[NT];      // number of visible keys of this lane's query row
  float slope2[NT];   // ALiBi slope * log2e
  const bool has_alibi = a.alibi_slopes != nullptr;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int row = row0 + 16 * nt + li;
    int t = row / G;
    limit[nt] = row < rows_valid ? ctx - (qb - 1 - t) : 0;
    slope2[nt] = 0.f;
    if (has_alibi && row < rows_valid) slope2[nt] = a.alibi_slopes[h * G + (row - t * G)] * kLog2e;
  }
  const int min_limit = ctx - (qb - 1);  // keys below this index are visible to every real row

  // ---- query: B operand of S^T = K Q^T --------------------------------------------------------------------
  // k-step s of a tile covers, for lane group kg, the 8 head dims the K load puts in that slot.
  // Rows past the last real one are loaded from row 0 and zeroed, which keeps this branch-free.
  bf16x8 qreg[NT][4];
  {
    const char* q_ptr = (const char*)a.query;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int row = row0 + 16 * nt + li;
      const bool ok = row < rows_valid;
      const int64_t e0 = (int64_t)b * a.stride_q_s + (int64_t)(h * Ge + (ok ? row : 0)) * a.stride_q_h;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int dim = kFp8 ? (64 * (s >> 1) + 16 * kg + 8 * (s & 1)) : (32 * s + 8 * kg);
        Bf16x8Bits q;
        if (a.query_dtype == PA_DTYPE_BF16) {
          q.u = load16(q_ptr + (e0 + dim) * 2);
        } else {
          u32x2 raw = *reinterpret_cast<const u32x2*>(q_ptr + e0 + dim);
          q.v = fp8x8_to_bf16x8(raw[0], raw[1]);
        }
        if (!ok) q.u = u32x4{0, 0, 0, 0};
        qreg[nt][s] = q.v;
      }
    }
  }
  // per-row query scale (FP8 query) multiplies the logits of that row
  float k_tensor_scale = 1.f, v_tensor_scale = 1.f;
  if (a.kv_quant_mode == PA_QUANT_PER_TENSOR) {
    k_tensor_scale = sload_f32(a.key_scale);
    v_tensor_scale = sload_f32(a.value_scale);
  }
  const float scale2 = a.softmax_scale * k_tensor_scale * kLog2e;
  float rscale[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int row = row0 + 16 * nt + li;
    float qs = 1.f;
    if (a.query_quant_mode == PA_QUANT_PER_TENSOR) qs = sload_f32(a.query_scale);
    if (a.query_quant_mode == PA_QUANT_PER_TOKEN && row < rows_valid)
      qs = a.query_scale[(int64_t)b * a.stride_qscale_s + h * Ge + row];
    rscale[nt] = scale2 * qs;
  }
  // FP8 math: q * cq = hi + lo with hi, lo in e4m3 (|q * cq| <= 224); the logits are divided by cq again
  i32x8 qhi[FP8MATH ? NT : 1], qlo[FP8MATH ? NT : 1];
  if constexpr (FP8MATH) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      float f[32];
      float amax = 0.f;
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        Bf16x8Bits q;
        q.v = qreg[nt][s4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          f[8 * s4 + 2 * e] = bf16_bits_to_f32(q.u[e] & 0xffffu);
          f[8 * s4 + 2 * e + 1] = __uint_as_float(q.u[e] & 0xffff0000u);
        }
      }
#pragma unroll
      for (int e = 0; e < 32; ++e) amax = fmaxf(amax, fabsf(f[e]));
      amax = quad_row_max(amax);
      const float cq = amax > 0.f ? 224.f / amax : 1.f;
      rscale[nt] *= amax > 0.f ? amax * (1.f / 224.f) : 1.f;
#pragma unroll
      for (int w = 0; w < 8; ++w) {
        const float x0 = f[4 * w] * cq, x1 = f[4 * w + 1] * cq, x2 = f[4 * w + 2] * cq, x3 = f[4 * w + 3] * cq;
        int hi = 0, lo = 0;
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(x0, x1, hi, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(x2, x3, hi, true);
        const f32x2 b01 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
        const f32x2 b23 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(x0 - b01[0], x1 - b01[1], lo, false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(x2 - b23[0], x3 - b23[1], lo, true);
        qhi[nt][w] = hi;
        qlo[nt][w] = lo;
      }
    }
  }
  float v_run = 1e-30f;  // FP8 math with per-token V scales: running max of the scales seen so far

  float m_run[NT];      // running max of the scaled logits, log2 domain (-inf before the first visible key)
  float l_run[NT];      // this lane's share of the running sum of exp2(s - m)
  f32x4 acc[NT][8];     // O^T: acc[nt][db][r] is head dim 16*db + 4*kg + r of query row 16*nt + li
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    m_run[nt] = -INFINITY;
    l_run[nt] = 0.f;
#pragma unroll
    for (int db = 0; db < 8; ++db) acc[nt][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  char* plds = &p_lds[wave][0][0];

  // ---- one step of 64 tokens ------------------------------------------------------------------------------
  // FULL: every token of the step is visible to every row and there is no ALiBi term.
  // PREFETCH: a next step exists; its K and V are requested as soon as this step's are consumed.
  auto step = [&]<bool FULL, bool PREFETCH>(SD& sd, int tok0, const Pages& pg_next) {
    // S^T tiles
    f32x4 s[NT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) s[nt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      if constexpr (FP8MATH) {
        const i32x8 ka = {(int)sd.k[j][0][0], (int)sd.k[j][0][1], (int)sd.k[j][0][2], (int)sd.k[j][0][3],
                          (int)sd.k[j][1][0], (int)sd.k[j][1][1], (int)sd.k[j][1][2], (int)sd.k[j][1][3]};
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          s[nt][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka, qhi[nt], s[nt][j], 0, 0, 0, 0, 0, 0);
          s[nt][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka, qlo[nt], s[nt][j], 0, 0, 0, 0, 0, 0);
        }
      } else
#pragma unroll
      for (int ld = 0; ld < SD::NKL; ++ld) {
        Bf16x8Bits ka;
        ka.u = sd.k[j][ld];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          s[nt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka.v, qreg[nt][ld], s[nt][j], 0, 0, 0);
      }
    }
    f32x4 ks_cur[PER_TOKEN ? 4 : 1];
    if constexpr (PER_TOKEN) {
#pragma unroll
      for (int j = 0; j < 4; ++j) ks_cur[j] = sd.ks[j];
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PREFETCH) issue_k(sd, pg_next);
    __builtin_amdgcn_sched_barrier(0);

    // FP8 math, per-token V scales: P carries v_scale / v_run (<= 1); the accumulator is kept in units
    // of the running maximum v_run
    // FP8 math: P is produced already multiplied by pmul = 256 / v_run; log2(pmul) rides in the exponent's
    // additive term, so the factor costs nothing per element
    float vfac = 1.f, log2_pmul = FP8MATH ? 8.f : 0.f, inv_pmul = FP8MATH ? 1.f / 256.f : 1.f;
    f32x4 vs_cur[(PER_TOKEN && FP8MATH) ? 4 : 1];
    if constexpr (PER_TOKEN && FP8MATH) {
      float vmx = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        vs_cur[j] = sd.vs[j];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (!FULL) {
            const int col = tok0 + 16 * j + 4 * kg + r;
            vs_cur[j][r] = col < ctx ? vs_cur[j][r] : 0.f;
          }
          vmx = fmaxf(vmx, vs_cur[j][r]);
        }
      }
      vmx = quad_row_max(vmx);
      const float v_new = fmaxf(v_run, vmx);
      vfac = v_new == v_run ? 1.f : v_run * __builtin_amdgcn_rcpf(v_new);
      log2_pmul = 8.f - __builtin_amdgcn_logf(v_new);
      inv_pmul = v_new * (1.f / 256.f);
      v_run = v_new;
    }
    uint32_t ph[FP8MATH ? NT : 1][4], pl[FP8MATH ? NT : 1][4];  // FP8 math: P head / residual, 4 tokens per dword

#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float rs = rscale[nt];
      float mx = -INFINITY;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // FULL: the row's scale (>= 0 on this path) is applied inside the exponent's fma, and to the maximum once
          float v = s[nt][j][r];
          if constexpr (PER_TOKEN) v *= ks_cur[j][r];
          if constexpr (!FULL) {
            const int col = tok0 + 16 * j + 4 * kg + r;
            v = v * rs + slope2[nt] * (float)(col - ctx + 1);
            v = col < limit[nt] ? v : -INFINITY;
          }
          s[nt][j][r] = v;
          mx = fmaxf(mx, v);
        }
      }
      mx = quad_row_max(mx);
      if constexpr (FULL) mx *= rs;
      const float m_new = fmaxf(m_run[nt], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = fast_exp2(m_run[nt] - m_safe);  // exp2(-inf) = 0 on the first visible step
      m_run[nt] = m_new;
      const float e_add = log2_pmul - m_safe;
      const float e_mul = FULL ? rs : 1.f;
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float p0 = fast_exp2(__builtin_fmaf(s[nt][j][0], e_mul, e_add));
        float p1 = fast_exp2(__builtin_fmaf(s[nt][j][1], e_mul, e_add));
        float p2 = fast_exp2(__builtin_fmaf(s[nt][j][2], e_mul, e_add));
        float p3 = fast_exp2(__builtin_fmaf(s[nt][j][3], e_mul, e_add));
        psum += (p0 + p1) + (p2 + p3);
        if constexpr (FP8MATH) {
          if constexpr (PER_TOKEN) {
            p0 *= vs_cur[j][0];
            p1 *= vs_cur[j][1];
            p2 *= vs_cur[j][2];
            p3 *= vs_cur[j][3];
          }
          int hi = 0, lo = 0;
          hi = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, hi, false);
          hi = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, hi, true);
          const f32x2 b01 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
          const f32x2 b23 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
          lo = __builtin_amdgcn_cvt_pk_fp8_f32(p0 - b01[0], p1 - b01[1], lo, false);
          lo = __builtin_amdgcn_cvt_pk_fp8_f32(p2 - b23[0], p3 - b23[1], lo, true);
          ph[nt][j] = (uint32_t)hi;
          pl[nt][j] = (uint32_t)lo;
          continue;
        }
        if constexpr (PER_TOKEN) {
          // a masked token's scale may be stale memory (NaN): its weight must stay exactly 0
          f32x4 vsc = sd.vs[j];
          if constexpr (!FULL) {
#pragma unroll
            for (int r = 0; r < 4; ++r) vsc[r] = s[nt][j][r] == -INFINITY ? 0.f : vsc[r];
          }
          p0 *= vsc[0];
          p1 *= vsc[1];
          p2 *= vsc[2];
          p3 *= vsc[3];
        }
        u32x2 pk;
        pk[0] = pack_bf16x2(p0, p1);
        pk[1] = pack_bf16x2(p2, p3);
        *reinterpret_cast<u32x2*>(plds + nt * (16 * kPRowBytes) + li * kPRowBytes + (16 * j + 4 * kg) * 2) = pk;
      }
      l_run[nt] = l_run[nt] * alpha + psum * inv_pmul;
      const float alpha_acc = alpha * vfac;
#pragma unroll
      for (int db = 0; db < 8; ++db) acc[nt][db] *= alpha_acc;
    }

    if constexpr (!FULL) {
      // zero the V bytes of tokens at or beyond ctx (stale cache contents may decode to NaN)
      int nvalid = ctx - (tok0 + 16 * kg);
      nvalid = nvalid < 0 ? 0 : (nvalid > 16 ? 16 : nvalid);
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        if constexpr (kFp8) {
          sd.v[db][0] = keep_first_bytes(sd.v[db][0], nvalid);
        } else {
          sd.v[db][0] = keep_first_bytes(sd.v[db][0], 2 * (nvalid > 8 ? 8 : nvalid));
          sd.v[db][1] = keep_first_bytes(sd.v[db][1], 2 * (nvalid > 8 ? nvalid - 8 : 0));
        }
      }
    }

    if constexpr (FP8MATH) {
      // lane group kg holds, per tile j, tokens 4kg..4kg+3; the B operand of O^T += V^T P^T wants lane
      // group kg to hold all 16 tokens of tile kg: a 4x4 transpose over (lane group, register)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        quad_transpose(ph[nt]);
        quad_transpose(pl[nt]);
      }
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
        for (int db = 0; db < 8; ++db) {
          const long va = (long)(((uint64_t)sd.v[db][0][2 * hf + 1] << 32) | sd.v[db][0][2 * hf]);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const long bh = (long)(((uint64_t)ph[nt][2 * hf + 1] << 32) | ph[nt][2 * hf]);
            const long bl = (long)(((uint64_t)pl[nt][2 * hf + 1] << 32) | pl[nt][2 * hf]);
            acc[nt][db] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(va, bh, acc[nt][db], 0, 0, 0);
            acc[nt][db] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(va, bl, acc[nt][db], 0, 0, 0);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (PREFETCH) issue_v(sd, pg_next);
      __builtin_amdgcn_sched_barrier(0);
      return;
    }

    // the P tile is written and read by this wave only; LDS operations of one wave complete in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // O^T += V^T P^T
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      bf16x8 pb[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        Bf16x8Bits t;
        t.u = *reinterpret_cast<const u32x4*>(plds + nt * (16 * kPRowBytes) + li * kPRowBytes +
                                              (16 * kg + 8 * hf) * 2);
        pb[nt] = t.v;
      }
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        Bf16x8Bits va;
        va.u = sd.v[db][hf];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[nt][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va.v, pb[nt], acc[nt][db], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PREFETCH) issue_v(sd, pg_next);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  // ---- main loop -------------------------------------------------------------------------------------------
  // the unmasked variant of the step scales the row maximum after taking it: only right for scales >= 0
  bool rs_neg = false;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) rs_neg = rs_neg || rscale[nt] < 0.f;
  // leading steps of this wave that need no masking: part_start + i * stride + 64 <= min_limit
  int n_full = 0;
  if (!has_alibi && __builtin_amdgcn_ballot_w64(rs_neg) == 0 && min_limit - part_start >= kStepTokens)
    n_full = (min_limit - part_start - kStepTokens) / kWaveStride + 1;
  int sidx = 0;
  int tok0 = part_start;
  if (active) {
    const int n_fast = n_full < n_steps - 1 ? n_full : n_steps - 1;
    Pages pg_next = load_pages(part_start + kWaveStride);
    for (; sidx < n_fast; ++sidx) {
      // Waves that share a SIMD do not progress evenly by themselves (the older one wins every
      // arbitration and finishes a third earlier, leaving the SIMD half empty at the end): the further a
      // wave is from its end, the higher its issue priority.
      {
        const int rem4 = (n_steps - sidx) * 4 / n_steps;
        if (rem4 >= 3)
          __builtin_amdgcn_s_setprio(3);
        else if (rem4 == 2)
          __builtin_amdgcn_s_setprio(2);
        else if (rem4 == 1)
          __builtin_amdgcn_s_setprio(1);
        else
          __builtin_amdgcn_s_setprio(0);
      }
      const Pages pg_after = load_pages(tok0 + 2 * kWaveStride);
      step.template operator()<true, true>(buf_a, tok0, pg_next);
      pg_next = pg_after;
      tok0 += kWaveStride;
    }
    for (; sidx < n_steps - 1; ++sidx) {
      const Pages pg_after = load_pages(tok0 + 2 * kWaveStride);
      step.template operator()<false, true>(buf_a, tok0, pg_next);
      pg_next = pg_after;
      tok0 += kWaveStride;
    }
    if (n_full >= n_steps)
      step.template operator()<true, false>(buf_a, tok0, pg_next);
    else
      step.template operator()<false, false>(buf_a, tok0, pg_next);
  }

  // ---- epilogue ------------------------------------------------------------------------------------------------
  // max_logits holds the maximum of the scaled logits in the natural-log domain, exp_sums the
  // un-normalised sum, tmp_output the normalised bf16 partial.  For a sequence that fits in one partition the
  // partial is the result, and it is written to output as well.
  const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (int64_t)part * a.stride_es_p;
  char* tmp = (char*)a.tmp_output + ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h +
                                     (int64_t)part * a.stride_tmp_p) * 2;
  // a sequence that fits in one partition needs no merge: its partial is the result
  const bool direct = ctx <= a.partition_size && a.output != nullptr && a.sinks == nullptr;
  char* outp = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2;
  const float acc_unit = FP8MATH ? (PER_TOKEN ? v_run : 1.f) * (1.f / 256.f) : 1.f;
  float l_tot[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    l_tot[nt] = quad_row_sum(l_run[nt]);
    if (row0 + 16 * nt + li >= rows_valid) {  // padding rows of a ragged batch: no visible key
      l_tot[nt] = 0.f;
      m_run[nt] = -INFINITY;
    }
  }
  if constexpr (WAVES == 1) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int row = row0 + 16 * nt + li;
      const float inv = l_tot[nt] > 0.f ? v_tensor_scale * acc_unit / l_tot[nt] : 0.f;
      if (row < Ge && kg == 0) {
        a.max_logits[es_off + row] = m_run[nt] * (1.0f / kLog2e);
        a.exp_sums[es_off + row] = l_tot[nt];
      }
      store_partial_tile(&o_lds[0][0], acc[nt], inv, tmp + (int64_t)(row0 + 16 * nt) * a.stride_tmp_g * 2,
                         a.stride_tmp_g * 2, direct ? outp + (int64_t)(row0 + 16 * nt) * a.stride_out_h * 2 : nullptr,
                         a.stride_out_h * 2, Ge - row0 - 16 * nt, lane);
    }
  } else {
    // merge the waves' (m, l, O): every wave holds the same (row, head dim) in the same lane and register,
    // so the merge is lane-wise; wave w merges head-dim blocks [w*8/WAVES, (w+1)*8/WAVES)
    __shared__ float mg_m[WAVES][NT * 16];
    __shared__ float mg_l[WAVES][NT * 16];
    __shared__ f32x4 mg_acc[WAVES][NT][8][64];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (kg == 0) {
        mg_m[wave][16 * nt + li] = m_run[nt];
        mg_l[wave][16 * nt + li] = l_tot[nt];
      }
#pragma unroll
      for (int db = 0; db < 8; ++db) mg_acc[wave][nt][db][lane] = acc[nt][db] * acc_unit;
    }
    __syncthreads();
    constexpr int DBW = 8 / WAVES;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int lrow = 16 * nt + li;
      const int row = row0 + lrow;
      float M = -INFINITY;
#pragma unroll
      for (int w2 = 0; w2 < WAVES; ++w2) M = fmaxf(M, mg_m[w2][lrow]);
      const float M_safe = M == -INFINITY ? 0.f : M;
      float e[WAVES];
      float L = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < WAVES; ++w2) {
        e[w2] = fast_exp2(mg_m[w2][lrow] - M_safe);
        L += mg_l[w2][lrow] * e[w2];
      }
      const float inv = L > 0.f ? v_tensor_scale / L : 0.f;
#pragma unroll
      for (int d = 0; d < DBW; ++d) {
        const int db = wave * DBW + d;
        f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2) o += mg_acc[w2][nt][db][lane] * e[w2];
        o *= inv;
        u32x2 pk;
        pk[0] = pack_bf16x2(o[0], o[1]);
        pk[1] = pack_bf16x2(o[2], o[3]);
        *reinterpret_cast<u32x2*>(&o_lds[0][0] + li * kORowBytes + (16 * db + 4 * kg) * 2) = pk;
      }
      if (wave == 0 && kg == 0 && row < Ge) {
        a.max_logits[es_off + row] = M * (1.0f / kLog2e);
        a.exp_sums[es_off + row] = L;
      }
      __syncthreads();
      for (int i = wave; i < 4; i += WAVES) {
        const int r = 4 * i + kg;
        const u32x4 v = *reinterpret_cast<const u32x4*>(&o_lds[0][0] + r * kORowBytes + li * 16);
        if (r < Ge - row0 - 16 * nt) {
          *reinterpret_cast<u32x4*>(tmp + (int64_t)(row0 + 16 * nt + r) * a.stride_tmp_g * 2 + li * 16) = v;
          if (direct)
            *reinterpret_cast<u32x4*>(outp + (int64_t)(row0 + 16 * nt + r) * a.stride_out_h * 2 + li * 16) = v;
        }
      }
      if (nt + 1 < NT) __syncthreads();
    }
  }
  if constexpr (QUEUE) {
    // rows of padding query positions beyond the last real tile: this workgroup fills them
    if (rt == tiles_b - 1 && wave == 0) {
      for (int r = 16 * NT * tiles_b + kg; r < Ge; r += 4) {
        if (li == 0) {
          a.max_logits[es_off + r] = -INFINITY;
          a.exp_sums[es_off + r] = 0.f;
        }
        *reinterpret_cast<u32x4*>(tmp + (int64_t)r * a.stride_tmp_g * 2 + li * 16) = u32x4{0, 0, 0, 0};
        if (direct) *reinterpret_cast<u32x4*>(outp + (int64_t)r * a.stride_out_h * 2 + li * 16) = u32x4{0, 0, 0, 0};
      }
    }
  }
  } while (0);
  if constexpr (!QUEUE) break;
  }  // for (;;)
  if constexpr (QUEUE) {
    // the last workgroup out leaves the workspace as it found it: zero
    if (threadIdx.x == 0) {
      __threadfence();
      if (atomicAdd(a.workspace + 1, 1) == (int)gridDim.x - 1) {
        a.workspace[0] = 0;
        a.workspace[1] = 0;
      }
    }
  }
}

// Global memory -> LDS without passing through registers: lane i's 16 (4) bytes land at lds_offset + 16 (4) * i.
// The loads count in vmcnt like any other vector load, but the compiler does not see them: whoever reads
// the LDS bytes waits with dma_wait<N>() (at most N vector memory operations still outstanding) first.
__device__ __forceinline__ void dma_load16(const void* gptr, uint32_t lds_offset) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_offset) : "memory");
}
__device__ __forceinline__ void dma_load4(const void* gptr, uint32_t lds_offset) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gptr), "s"(lds_offset) : "memory");
}
// the same with the address split into a wave-uniform base and a 32-bit per-lane byte offset
__device__ __forceinline__ void dma_load16(const void* base, uint32_t lane_offset, uint32_t lds_offset) {
  // the base is wave-uniform by construction; readfirstlane makes the compiler keep it in scalar registers
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  // (the builtin returns a signed int: widen through uint32_t, or a low word with bit 31 set would smear
  // ones over the high word)
  const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
  const uint64_t sb = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(sb),
               "s"(lds_offset)
               : "memory");
}
template <int N>
__device__ __forceinline__ void dma_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ uint32_t lds_offset_of(const void* p) {
  return (uint32_t)reinterpret_cast<uintptr_t>(
      (const __attribute__((address_space(3))) char*)(const char*)p);
}

// ---------------------------------------------------------------------------------------------
// Partition kernel for more than 16 query rows per kv head (large GQA groups, MTP) over an FP8 cache.
// The up to four 16-row query tiles of one (sequence, kv head, partition) are the four waves of ONE
// workgroup and share a single pass over the pages.  Of every 64-token step each wave fetches a quarter
// (K tile `wave`, V head-dim blocks 2*wave and 2*wave+1) into registers and parks it in LDS in exactly the
// per-lane operand order of the MFMAs; after a workgroup barrier every wave reads the whole step back
// with lane-contiguous 16-byte LDS reads.  Two LDS buffers: step s+1 travels from HBM while step s is multiplied,
// one barrier per step.  Against one workgroup per row tile this reads every page once instead of once per
// tile (the repeats hit the L2, but each costs a full trip through the vector memory path).
// ---------------------------------------------------------------------------------------------
struct StepLds {
  u32x4 k[4][2][64];  // [tile][load][lane]: the K operand of a tile as its two loads deliver it
  u32x4 v[4][128];    // [tile][head dim]: 16 tokens of one head dim
  float sc[4][2][16]; // [tile][K scales, V scales][token]
};

template <bool PER_TOKEN, bool BS16, int NB, int OCC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void pa_partition_shared_kernel(const PaDecodeArgs a) {
  __shared__ __attribute__((aligned(16))) StepLds stage[NB];  // ring of steps: NB-1 in flight, one being read
  static_assert(sizeof(StepLds) * NB >= 4 * 16 * kORowBytes, "the output tiles reuse the stage buffers");
  constexpr int kLoadsPerStep = PER_TOKEN ? 5 : 4;  // vector memory operations one wave issues per step

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15;
  const int kg = lane >> 4;

  // ---- which (sequence, head, partition): workgroup-uniform; head fastest, partition slowest ----------
  const int Hkv = a.num_kv_heads;
  const int G = a.group_size;
  const int Ge = a.q_len * G;
  const long long wid = blockIdx.x;
  const int h = (int)(wid % Hkv);
  const int b = (int)((wid / Hkv) % a.num_seqs);
  const int part = (int)(wid / ((long long)Hkv * a.num_seqs));

  const int ctx = sload_i32(a.context_lens + b);
  const int wg_start = part * a.partition_size;
  if (wg_start >= ctx) return;
  const int wg_end = min(wg_start + a.partition_size, ctx);
  const int n_steps = (wg_end - wg_start + kStepTokens - 1) / kStepTokens;
  const int qb = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
  const int rows_valid = qb * G;
  const int row0 = 16 * wave;               // this wave's query tile
  const bool has_rows = row0 < rows_valid;  // else the wave only helps to fetch

  // ---- cache addressing ----------------------------------------------------------------------------------
  const int log2_bs = 31 - __builtin_clz(a.block_size);
  const int bs_mask = a.block_size - 1;
  const char* kbase = (const char*)a.key_cache + (int64_t)h * a.stride_k_h;
  const char* vbase = (const char*)a.value_cache + (int64_t)h * a.stride_v_h;
  const int64_t k_block_bytes = a.stride_k_b;
  const int64_t v_block_bytes = a.stride_v_b;
  const float* ksbase = PER_TOKEN ? a.key_scale + (int64_t)h * a.stride_kvscale_h : nullptr;
  const float* vsbase = PER_TOKEN ? a.value_scale + (int64_t)h * a.stride_kvscale_h : nullptr;
  const uint32_t k_chunk_bytes = BS16 ? 256u : (uint32_t)a.stride_k_c;
  uint32_t k_lane_off[2];
#pragma unroll
  for (int ld = 0; ld < 2; ++ld) k_lane_off[ld] = (uint32_t)(kg * k_chunk_bytes + li * 16) + 4 * ld * k_chunk_bytes;
  const bool vt = a.v_transposed;
  const uint32_t v_row_bytes = BS16 ? 16u : (vt ? 16u : (uint32_t)a.stride_v_2);
  const int64_t v_tile_bytes = BS16 ? 16 : (vt ? a.stride_v_2 : 16);
  uint32_t v_lane_off[2];  // V loads: lane = head dim (0..63, 64..127) of one tile
#pragma unroll
  for (int i = 0; i < 2; ++i) v_lane_off[i] = (uint32_t)(lane + 64 * i) * v_row_bytes;
  const float* sc_lane = PER_TOKEN ? ((lane & 16) ? vsbase : ksbase) + li : nullptr;

  const int* bt = a.block_tables + (int64_t)b * a.stride_bt_s;
  const int last_tile_tok = (wg_end - 1) & ~15;
  // wave w fetches tile w of every step: its page id (a scalar load) and the tile's token offset inside the
  // page.  Tiles past the last live one repeat it, so no block-table slot or page beyond the sequence is touched.
  struct TilePage {
    int page;
    int off;
  };
  auto load_page = [&](int tok0) {
    int t = tok0 + 16 * wave;
    t = t > last_tile_tok ? last_tile_tok : t;
    TilePage tp;
    tp.page = sload_i32(bt + (t >> log2_bs));
    tp.off = t & bs_mask;
    return tp;
  };
  // this wave's quarter of the step whose page ids are pg, sent to ring slot `slot`
  const uint32_t stage_base = lds_offset_of(&stage[0]);
  auto fetch = [&](int slot, const TilePage& tp) {
    const uint32_t st = stage_base + (uint32_t)slot * (uint32_t)sizeof(StepLds);
    // every address is a wave-uniform base plus a per-lane constant
    const int page = tp.page;
    const int off = tp.off;
    const char* kt = kbase + (int64_t)page * k_block_bytes + (int64_t)off * 16;
    const uint32_t kdst = st + (uint32_t)offsetof(StepLds, k) + (uint32_t)wave * 2048u;
    dma_load16(kt, k_lane_off[0], kdst);
    dma_load16(kt, k_lane_off[1], kdst + 1024u);
    const char* vt_ = vbase + (int64_t)page * v_block_bytes + (int64_t)(off >> 4) * v_tile_bytes;
    const uint32_t vdst = st + (uint32_t)offsetof(StepLds, v) + (uint32_t)wave * 2048u;
    dma_load16(vt_, v_lane_off[0], vdst);   // head dims 0..63 (lane = dim)
    dma_load16(vt_, v_lane_off[1], vdst + 1024u);  // head dims 64..127
    if constexpr (PER_TOKEN) {
      // lanes 0-15: the K scales of the tile's 16 tokens, lanes 16-31: the V scales
      if (lane < 32)
        dma_load4(sc_lane + ((int64_t)page * a.stride_kvscale_b + off),
                  st + (uint32_t)offsetof(StepLds, sc) + (uint32_t)wave * 128u);
    }
  };

  // ---- the first NB-1 steps go out before anything else is set up ----------------------------------------------
  TilePage pg_next = load_page(wg_start);  // of the next step to fetch
  int fetch_tok = wg_start;
#pragma unroll
  for (int i = 0; i < NB - 1; ++i) {
    if (i < n_steps) {
      fetch(i, pg_next);
      fetch_tok += kStepTokens;
      pg_next = load_page(fetch_tok);
    }
  }

  // ---- buffers of this item ---------------------------------------------------------------------------------
  const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (int64_t)part * a.stride_es_p;
  char* tmp = (char*)a.tmp_output + ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h +
                                     (int64_t)part * a.stride_tmp_p) * 2;
  const bool direct = ctx <= a.partition_size && a.output != nullptr && a.sinks == nullptr;
  char* outp = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2;
  // ---- per-lane row bookkeeping ---------------------------------------------------------------------------------
  const bool has_alibi = a.alibi_slopes != nullptr;
  const int row = row0 + li;
  const bool row_ok = row < rows_valid;
  const int t_row = row / G;
  const int limit = row_ok ? ctx - (qb - 1 - t_row) : 0;  // number of visible keys of this lane's query row
  float slope2 = 0.f;
  if (has_alibi && row_ok) slope2 = a.alibi_slopes[h * G + (row - t_row * G)] * kLog2e;
  const int min_limit = ctx - (qb - 1);

  // ---- query: q * cq = hi + lo in e4m3 (|q * cq| <= 224), the B operand of S^T = K Q^T -------------------
  float k_tensor_scale = 1.f, v_tensor_scale = 1.f;
  if (a.kv_quant_mode == PA_QUANT_PER_TENSOR) {
    k_tensor_scale = sload_f32(a.key_scale);
    v_tensor_scale = sload_f32(a.value_scale);
  }
  float rscale = a.softmax_scale * k_tensor_scale * kLog2e;
  if (a.query_quant_mode == PA_QUANT_PER_TENSOR) rscale *= sload_f32(a.query_scale);
  if (a.query_quant_mode == PA_QUANT_PER_TOKEN && row_ok)
    rscale *= a.query_scale[(int64_t)b * a.stride_qscale_s + h * Ge + row];
  i32x8 qhi, qlo;
  {
    const char* q_ptr = (const char*)a.query;
    const int64_t e0 = (int64_t)b * a.stride_q_s + (int64_t)(h * Ge + (row_ok ? row : 0)) * a.stride_q_h;
    float f[32];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int dim = 64 * (s >> 1) + 16 * kg + 8 * (s & 1);
      Bf16x8Bits q;
      if (a.query_dtype == PA_DTYPE_BF16) {
        q.u = load16(q_ptr + (e0 + dim) * 2);
      } else {
        u32x2 raw = *reinterpret_cast<const u32x2*>(q_ptr + e0 + dim);
        q.v = fp8x8_to_bf16x8(raw[0], raw[1]);
      }
      if (!row_ok) q.u = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        f[8 * s + 2 * e] = bf16_bits_to_f32(q.u[e] & 0xffffu);
        f[8 * s + 2 * e + 1] = __uint_as_float(q.u[e] & 0xffff0000u);
      }
    }
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 32; ++e) amax = fmaxf(amax, fabsf(f[e]));
    amax = quad_row_max(amax);
    const float cq = amax > 0.f ? 224.f / amax : 1.f;
    rscale *= amax > 0.f ? amax * (1.f / 224.f) : 1.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const float x0 = f[4 * w] * cq, x1 = f[4 * w + 1] * cq, x2 = f[4 * w + 2] * cq, x3 = f[4 * w + 3] * cq;
      int hi = 0, lo = 0;
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(x0, x1, hi, false);
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(x2, x3, hi, true);
      const f32x2 b01 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
      const f32x2 b23 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(x0 - b01[0], x1 - b01[1], lo, false);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(x2 - b23[0], x3 - b23[1], lo, true);
      qhi[w] = hi;
      qlo[w] = lo;
    }
  }

  const bool rs_nonneg = __builtin_amdgcn_ballot_w64(rscale < 0.f) == 0;
  float v_run = 1e-30f;  // per-token V scales: running max of the scales seen so far
  float m_run = -INFINITY;
  float l_run = 0.f;
  f32x4 acc[8];
#pragma unroll
  for (int db = 0; db < 8; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- one step of 64 tokens out of LDS: the arithmetic of pa_partition_kernel's FP8 step, one row tile ----
  auto compute = [&]<bool FULL>(const StepLds& st, int tok0) {
    f32x4 s[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const u32x4 k0 = st.k[j][0][lane], k1 = st.k[j][1][lane];
      const i32x8 ka = {(int)k0[0], (int)k0[1], (int)k0[2], (int)k0[3], (int)k1[0], (int)k1[1], (int)k1[2], (int)k1[3]};
      s[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      s[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka, qhi, s[j], 0, 0, 0, 0, 0, 0);
      s[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka, qlo, s[j], 0, 0, 0, 0, 0, 0);
    }
    // P is produced already multiplied by pmul = 256 / v_run (per-token V scales: v_run is the running
    // maximum of the scales, P then also carries v_scale / v_run <= 1 and the accumulator is kept in units
    // of v_run): log2(pmul) rides in the exponent's additive term, so it costs nothing per element
    float vfac = 1.f, log2_pmul = 8.f, inv_pmul = 1.f / 256.f;
    f32x4 ks_cur[PER_TOKEN ? 4 : 1], vs_cur[PER_TOKEN ? 4 : 1];
    if constexpr (PER_TOKEN) {
      float vmx = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        ks_cur[j] = *reinterpret_cast<const f32x4*>(&st.sc[j][0][4 * kg]);
        vs_cur[j] = *reinterpret_cast<const f32x4*>(&st.sc[j][1][4 * kg]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (!FULL) {
            const int col = tok0 + 16 * j + 4 * kg + r;
            vs_cur[j][r] = col < ctx ? vs_cur[j][r] : 0.f;
          }
          vmx = fmaxf(vmx, vs_cur[j][r]);
        }
      }
      vmx = quad_row_max(vmx);
      const float v_new = fmaxf(v_run, vmx);
      vfac = v_new == v_run ? 1.f : v_run * __builtin_amdgcn_rcpf(v_new);
      log2_pmul = 8.f - __builtin_amdgcn_logf(v_new);
      inv_pmul = v_new * (1.f / 256.f);
      v_run = v_new;
    }
    // FULL: the row's scale (>= 0 on this path) is applied inside the exponent's fma, and to the maximum once
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = s[j][r];
        if constexpr (PER_TOKEN) v *= ks_cur[j][r];
        if constexpr (!FULL) {
          const int col = tok0 + 16 * j + 4 * kg + r;
          v = v * rscale + slope2 * (float)(col - ctx + 1);
          v = col < limit ? v : -INFINITY;
        }
        s[j][r] = v;
        mx = fmaxf(mx, v);
      }
    }
    mx = quad_row_max(mx);
    if constexpr (FULL) mx *= rscale;
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    m_run = m_new;
    const float e_add = log2_pmul - m_safe;
    const float e_mul = FULL ? rscale : 1.f;
    float psum = 0.f;
    uint32_t ph[4], pl[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float p0 = fast_exp2(__builtin_fmaf(s[j][0], e_mul, e_add));
      float p1 = fast_exp2(__builtin_fmaf(s[j][1], e_mul, e_add));
      float p2 = fast_exp2(__builtin_fmaf(s[j][2], e_mul, e_add));
      float p3 = fast_exp2(__builtin_fmaf(s[j][3], e_mul, e_add));
      psum += (p0 + p1) + (p2 + p3);
      if constexpr (PER_TOKEN) {
        p0 *= vs_cur[j][0];
        p1 *= vs_cur[j][1];
        p2 *= vs_cur[j][2];
        p3 *= vs_cur[j][3];
      }
      int hi = 0, lo = 0;
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, hi, false);
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, hi, true);
      const f32x2 b01 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
      const f32x2 b23 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(p0 - b01[0], p1 - b01[1], lo, false);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(p2 - b23[0], p3 - b23[1], lo, true);
      ph[j] = (uint32_t)hi;
      pl[j] = (uint32_t)lo;
    }
    l_run = l_run * alpha + psum * inv_pmul;
    // the accumulator is rescaled only when some row's maximum (or the V scale unit) moved
    const float alpha_acc = alpha * vfac;
    if (__builtin_amdgcn_ballot_w64(alpha_acc != 1.f)) {
#pragma unroll
      for (int db = 0; db < 8; ++db) acc[db] *= alpha_acc;
    }

    // lane group kg holds, per tile j, tokens 4kg..4kg+3; the B operand of O^T += V^T P^T wants lane group
    // kg to hold all 16 tokens of tile kg: a 4x4 transpose over (lane group, register)
    quad_transpose(ph);
    quad_transpose(pl);
    // one 128-deep MFMA per 16 head dims covers head and residual of P at once: its reduction index runs
    // over (tile kg's 16 tokens with P head, the same 16 tokens with P residual), so the A operand is the V
    // bytes twice -- read from LDS twice, which costs no VALU slot
    const i32x8 pb = {(int)ph[0], (int)ph[1], (int)ph[2], (int)ph[3], (int)pl[0], (int)pl[1], (int)pl[2], (int)pl[3]};
    int nvalid = 16;
    if constexpr (!FULL) {
      // V bytes of tokens at or beyond ctx are zeroed (stale cache contents may decode to NaN)
      nvalid = ctx - (tok0 + 16 * kg);
      nvalid = nvalid < 0 ? 0 : (nvalid > 16 ? 16 : nvalid);
    }
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      const u32x4* vp = &st.v[kg][16 * db + li];
      typedef const volatile __attribute__((address_space(3))) u32x4* LdsVec;
      u32x4 v0 = *vp;
      u32x4 v1 = *(LdsVec)vp;  // a second LDS read, not a register copy
      if constexpr (!FULL) {
        v0 = keep_first_bytes(v0, nvalid);
        v1 = keep_first_bytes(v1, nvalid);
      }
      const i32x8 va = {(int)v0[0], (int)v0[1], (int)v0[2], (int)v0[3], (int)v1[0], (int)v1[1], (int)v1[2], (int)v1[3]};
      acc[db] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(va, pb, acc[db], 0, 0, 0, 0, 0, 0);
    }
  };

  // ---- main loop ---------------------------------------------------------------------------------------------
  int n_full = has_alibi ? 0 : (min_limit - wg_start) / kStepTokens;  // leading steps that need no masking
  n_full = n_full < 0 ? 0 : n_full;
  int tok0 = wg_start;
  int slot = 0;             // ring slot of step s
  int fetch_slot = NB - 1;  // ring slot the next fetch goes to
  int s = 0;
  // what every wave does at the head of step s, whether it has rows to compute or not
  auto enter_step = [&]() {
    // step s has landed once at most the loads of the steps after it are outstanding
    const int after = n_steps - 1 - s;
    if (after >= NB - 2)
      dma_wait<(NB - 2) * kLoadsPerStep>();
    else if (NB > 3 && after == 1)
      dma_wait<kLoadsPerStep>();
    else
      dma_wait<0>();
    // everybody's quarter of step s is in LDS, and everybody is done reading step s-1, whose slot is refilled now
    __syncthreads();
    if (s + NB - 1 < n_steps) {
      fetch(fetch_slot, pg_next);
      fetch_tok += kStepTokens;
      pg_next = load_page(fetch_tok);
    }
  };
  auto leave_step = [&]() {
    ++s;
    tok0 += kStepTokens;
    slot = slot + 1 == NB ? 0 : slot + 1;
    fetch_slot = fetch_slot + 1 == NB ? 0 : fetch_slot + 1;
  };
  // Three loops, each with one variant of the step (one loop with a choice inside would make the compiler
  // copy the whole accumulator state where the variants join, every step).  The waves of a workgroup may be
  // in different loops: all of them pass the same number of barriers.
  if (has_rows) {
    const int n_fast = rs_nonneg ? (n_full < n_steps ? n_full : n_steps) : 0;
    while (s < n_fast) {
      enter_step();
      compute.template operator()<true>(stage[slot], tok0);
      leave_step();
    }
    while (s < n_steps) {
      enter_step();
      compute.template operator()<false>(stage[slot], tok0);
      leave_step();
    }
  } else {
    while (s < n_steps) {
      enter_step();
      leave_step();
    }
  }
  __syncthreads();  // the stage buffers are free

  // ---- epilogue: every wave writes its own row tile -----------------------------------------------------------
  if (!has_rows) {
    // a tile of padding rows only (a ragged batch): the rows read as "no visible key"
    for (int r = row0 + kg; r < row0 + 16 && r < Ge; r += 4) {
      if (li == 0) {
        a.max_logits[es_off + r] = -INFINITY;
        a.exp_sums[es_off + r] = 0.f;
      }
      *reinterpret_cast<u32x4*>(tmp + (int64_t)r * a.stride_tmp_g * 2 + li * 16) = u32x4{0, 0, 0, 0};
      if (direct) *reinterpret_cast<u32x4*>(outp + (int64_t)r * a.stride_out_h * 2 + li * 16) = u32x4{0, 0, 0, 0};
    }
    return;
  }
  float l_tot = quad_row_sum(l_run);
  if (!row_ok) {
    l_tot = 0.f;
    m_run = -INFINITY;
  }
  const float acc_unit = (PER_TOKEN ? v_run : 1.f) * (1.f / 256.f);
  const float inv = l_tot > 0.f ? v_tensor_scale * acc_unit / l_tot : 0.f;
  if (row < Ge && kg == 0) {
    a.max_logits[es_off + row] = m_run * (1.0f / kLog2e);
    a.exp_sums[es_off + row] = l_tot;
  }
  char* olds = reinterpret_cast<char*>(&stage[0]) + wave * (16 * kORowBytes);
  store_partial_tile(olds, acc, inv, tmp + (int64_t)row0 * a.stride_tmp_g * 2, a.stride_tmp_g * 2,
                     direct ? outp + (int64_t)row0 * a.stride_out_h * 2 : nullptr, a.stride_out_h * 2, Ge - row0, lane);
}

// ---------------------------------------------------------------------------------------------
// reduce: a workgroup owns 16 consecutive output rows of one (sequence, kv head); a wave works on one row at
// a time, two head dims per lane.  Lane p of a 64-partition chunk owns (m_p, l_p); the weights
// w_p = l_p e^{m_p - M} are broadcast with v_readlane while the partial outputs stream in.  A sequence with one
// partition was finished by the partition kernel: its workgroups leave after one scalar load.
//   ROWS = 1: 16 waves, one row each -- the least code and the shortest critical path, for batches with few rows
//             (a launch this short is dominated by fetching its own code and by one or two memory latencies).
//   ROWS = 4: 4 waves, four rows each -- for big batches, where the number of resident waves is the limit: with up
//             to 8 partitions (the tuning layer picks few, large ones) all loads of the four rows go out before
//             anything is waited for.
// ---------------------------------------------------------------------------------------------
// one row, any number of partitions; returns two packed bf16 head dims
__device__ __forceinline__ uint32_t reduce_row(const PaDecodeArgs& a, int b, int h, int row, int n, int lane) {
  const int Ge = a.q_len * a.group_size;
  const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + row;
  const float* ml = a.max_logits + es_off;
  const float* es = a.exp_sums + es_off;
  const char* tmp = (const char*)a.tmp_output +
                    ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h + (int64_t)row * a.stride_tmp_g) * 2 +
                    lane * 4;
  const int64_t tp = a.stride_tmp_p * 2;
  const int64_t sp = a.stride_es_p;

  // this lane's (m, l) of the first chunk and the first eight partials (indices past the end repeat the last
  // partition and get weight 0), requested together
  float m0 = lane < n ? ml[(int64_t)lane * sp] : -INFINITY;
  float l0 = lane < n ? es[(int64_t)lane * sp] : 0.f;
  uint32_t t0[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t0[i] = *reinterpret_cast<const uint32_t*>(tmp + (int64_t)(i < n ? i : n - 1) * tp);
  float M = m0;
  for (int p = lane + 64; p < n; p += 64) M = fmaxf(M, ml[p * sp]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
  const float M_safe = M == -INFINITY ? 0.f : M;

  float acc0 = 0.f, acc1 = 0.f, wsum = 0.f;
  for (int c0 = 0; c0 < n; c0 += 64) {
    const int cnt = n - c0 < 64 ? n - c0 : 64;
    float m = m0, l = l0;
    if (c0) {
      m = lane < cnt ? ml[(int64_t)(c0 + lane) * sp] : -INFINITY;
      l = lane < cnt ? es[(int64_t)(c0 + lane) * sp] : 0.f;
    }
    const float w = l > 0.f ? l * __expf(m - M_safe) : 0.f;  // 0 in lanes at or past cnt
    wsum += w;
    const char* tc = tmp + (int64_t)c0 * tp;
    int u = 0;
    if (c0 == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float wi = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), i));
        acc0 += bf16_bits_to_f32(t0[i] & 0xffffu) * wi;
        acc1 += __uint_as_float(t0[i] & 0xffff0000u) * wi;
      }
      u = 8;
    }
    for (; u + 8 <= cnt; u += 8) {
      uint32_t t[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) t[i] = *reinterpret_cast<const uint32_t*>(tc + (int64_t)(u + i) * tp);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float wi = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), u + i));
        acc0 += bf16_bits_to_f32(t[i] & 0xffffu) * wi;
        acc1 += __uint_as_float(t[i] & 0xffff0000u) * wi;
      }
    }
    for (; u < cnt; ++u) {
      const uint32_t t = *reinterpret_cast<const uint32_t*>(tc + (int64_t)u * tp);
      const float wi = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), u));
      acc0 += bf16_bits_to_f32(t & 0xffffu) * wi;
      acc1 += __uint_as_float(t & 0xffff0000u) * wi;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) wsum += __shfl_xor(wsum, o);
  // attention sink: one more term in the softmax denominator, exp(sink - M), with no value attached
  if (a.sinks) wsum += __expf(a.sinks[h * Ge + row] - M_safe);
  const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
  return pack_bf16x2(acc0 * inv, acc1 * inv);
}

// rows row0, row0+4, row0+8, row0+12 with 1 <= n <= 8 partitions: every load goes out first; maximum and sum
// are taken over v_readlane broadcasts, which every lane computes alike
__device__ __forceinline__ void reduce_four_rows(const PaDecodeArgs& a, int b, int h, int row0, int n, int rows_valid,
                                                 char* outp, int lane) {
  const int Ge = a.q_len * a.group_size;
  const int64_t sp = a.stride_es_p;
  const int64_t tp = a.stride_tmp_p * 2;
  float m[4], l[4];
  uint32_t t[4][8];
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int row = row0 + 4 * rr;
    const bool live = row < rows_valid;
    const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (live ? row : 0);
    const bool mine = live && lane < n;
    m[rr] = mine ? a.max_logits[es_off + (int64_t)lane * sp] : -INFINITY;
    l[rr] = mine ? a.exp_sums[es_off + (int64_t)lane * sp] : 0.f;
    const char* tmp = (const char*)a.tmp_output +
                      ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h + (int64_t)(live ? row : 0) * a.stride_tmp_g) * 2 +
                      lane * 4;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      t[rr][i] = live ? *reinterpret_cast<const uint32_t*>(tmp + (int64_t)(i < n ? i : n - 1) * tp) : 0u;
  }
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int row = row0 + 4 * rr;
    float M = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) M = fmaxf(M, __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(m[rr]), i)));
    const float M_safe = M == -INFINITY ? 0.f : M;
    const float w = l[rr] > 0.f ? l[rr] * __expf(m[rr] - M_safe) : 0.f;
    float wsum = 0.f, acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float wi = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), i));
      wsum += wi;
      acc0 += bf16_bits_to_f32(t[rr][i] & 0xffffu) * wi;
      acc1 += __uint_as_float(t[rr][i] & 0xffff0000u) * wi;
    }
    if (a.sinks && row < rows_valid) wsum += __expf(a.sinks[h * Ge + row] - M_safe);
    const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
    if (row < Ge) *reinterpret_cast<uint32_t*>(outp + (int64_t)row * a.stride_out_h * 2) = pack_bf16x2(acc0 * inv, acc1 * inv);
  }
}

template <bool SKIP_SINGLE, int ROWS>
__global__ __launch_bounds__(1024 / ROWS) void pa_reduce_kernel(const PaDecodeArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int Ge = a.q_len * a.group_size;
  const int RT = (Ge + 15) / 16;
  const long long wid = blockIdx.x;
  const int rt = (int)(wid % RT);
  const int h = (int)((wid / RT) % a.num_kv_heads);
  const int b = (int)(wid / ((long long)RT * a.num_kv_heads));
  const int row0 = 16 * rt + wave;  // ROWS = 4: this wave's rows are row0 + 4 * rr
  if (row0 >= Ge) return;

  const int ctx = sload_i32(a.context_lens + b);
  int n = (ctx + a.partition_size - 1) / a.partition_size;
  n = n > a.max_num_partitions ? a.max_num_partitions : n;
  // SKIP_SINGLE: the partition kernel of the same call has written the rows of sequences with one partition
  if (SKIP_SINGLE && n == 1 && !a.sinks) return;
  const int qb = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
  const int rows_valid = n <= 0 ? 0 : qb * a.group_size;  // rows at or beyond read as zero

  char* outp = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2 + lane * 4;
  if (ROWS == 4 && n >= 1 && n <= 8) {
    reduce_four_rows(a, b, h, row0, n, rows_valid, outp, lane);
    return;
  }
  for (int rr = 0; rr < ROWS; ++rr) {
    const int row = row0 + 4 * rr;
    if (row >= Ge) break;
    const uint32_t v = row < rows_valid ? reduce_row(a, b, h, row, n, lane) : 0u;
    *reinterpret_cast<uint32_t*>(outp + (int64_t)row * a.stride_out_h * 2) = v;
  }
}

__global__ void pa_fp8_decode_kernel(const uint8_t* codes, float* out, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  // same path as the partition kernel: byte -> bf16 bit pattern -> f32
  uint32_t w = (uint32_t)codes[i] | ((uint32_t)codes[i] << 16);
  uint32_t lo = fp8x2_to_bf16x2(w, false);
  uint32_t hi = fp8x2_to_bf16x2(w, true);
  float a = bf16_bits_to_f32(lo & 0xffffu);
  float b = bf16_bits_to_f32(hi & 0xffffu);
  out[i] = (i & 1) ? b : a;
}

thread_local int g_last_hip_error = 0;

int check_common(const PaDecodeArgs* a) {
  if (!a) return PA_ERR_NULL_POINTER;
  if (a->struct_size != sizeof(PaDecodeArgs)) return PA_ERR_BAD_STRUCT;
  if (!a->context_lens || !a->exp_sums || !a->max_logits || !a->tmp_output) return PA_ERR_NULL_POINTER;
  if (a->num_seqs <= 0 || a->num_kv_heads <= 0 || a->group_size <= 0 || a->q_len <= 0 ||
      a->max_num_partitions <= 0)
    return PA_ERR_BAD_SHAPE;
  if (a->partition_size <= 0 || a->partition_size % 256) return PA_ERR_BAD_SHAPE;
  if (a->head_size != kHeadSize) return PA_ERR_UNSUPPORTED;
  if (a->q_len * a->group_size > 64) return PA_ERR_UNSUPPORTED;  // the reference's limit
  return PA_OK;
}

int device_num_cus() {
  static const int n = [] {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 256;
    return prop.multiProcessorCount;
  }();
  return n;
}

// The queued launch is used when the caller gave a workspace and per-sequence query lengths (row tiles of
// padding rows are then common): a resident grid pulls live items from a counter.  Without query lengths
// the only workgroups with nothing to do are partitions past a sequence's end, which the plain launch
// orders last; there the queue's bookkeeping costs more than it saves (measured: +10 % on a uniform batch).
bool use_queue(const PaDecodeArgs& a) {
  static const bool off = [] {
    const char* e = getenv("PA_DECODE_QUEUE");
    return e && e[0] == '0';
  }();
  return !off && a.workspace != nullptr && a.num_seqs <= kQueueMaxSeqs && a.q_lens != nullptr;
}

template <int NT, int KVT, bool PT, bool BS16, int W>
int launch_partition_w(const PaDecodeArgs& a, hipStream_t stream) {
  constexpr int OCC = NT == 1 ? 2 : 1;
  const int ge = a.q_len * a.group_size;
  const int row_tiles = (ge + 16 * NT - 1) / (16 * NT);
  const long long blocks = (long long)a.num_seqs * a.num_kv_heads * a.max_num_partitions * row_tiles;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  if (use_queue(a)) {
    long long resident = (long long)device_num_cus() * 4 * OCC / W;
    resident = resident < blocks ? resident : blocks;
    hipLaunchKernelGGL((pa_partition_kernel<NT, KVT, PT, BS16, W, OCC, true>), dim3((unsigned)resident),
                       dim3(64 * W), 0, stream, a);
  } else
  hipLaunchKernelGGL((pa_partition_kernel<NT, KVT, PT, BS16, W, OCC, false>), dim3((unsigned)blocks), dim3(64 * W), 0, stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    g_last_hip_error = (int)e;
    return PA_ERR_LAUNCH;
  }
  return PA_OK;
}


// 16-row query tiles per workgroup.  More than 16 query rows per kv head (large GQA groups, MTP) are split
// over workgroups of one tile each by default: they re-read the same pages at the same time from the
// same L2, run the 2-waves-per-SIMD variant, and tiles that hold only padding rows cost nothing.
// PA_DECODE_TILES=2 keeps two tiles in one workgroup (one pass over the pages, 1 wave per SIMD).
int tiles_per_workgroup(int total_tiles) {
  static const int forced = [] {
    const char* e = getenv("PA_DECODE_TILES");
    return e ? atoi(e) : 0;
  }();
  const int t = forced == 2 ? 2 : 1;
  return t < total_tiles ? t : total_tiles;
}

// Waves per workgroup: about 256 tokens (4 steps) per wave at least, and at most 4 / NT waves (the
// merge buffer of a workgroup is NT * WAVES * 8 KiB of LDS).
int waves_per_workgroup(const PaDecodeArgs& a, int nt) {
  static const int forced = [] {
    const char* e = getenv("PA_DECODE_WAVES");
    return e ? atoi(e) : 0;
  }();
  int w = a.partition_size >= 1024 ? 4 : (a.partition_size >= 512 ? 2 : 1);
  if (forced > 0) w = forced;
  const int cap = nt == 1 ? 4 : (nt == 2 ? 2 : 1);
  w = w > cap ? cap : w;
  return w >= 4 ? 4 : (w >= 2 ? 2 : 1);
}

// More than one 16-row query tile per kv head over an FP8 cache: the tiles share one pass over the pages
// (pa_partition_shared_kernel).  PA_DECODE_SHARED=0 falls back to one workgroup per tile.
bool use_shared_stream(int kv_dtype, int rows_per_group) {
  static const bool off = [] {
    const char* e = getenv("PA_DECODE_SHARED");
    return e && e[0] == '0';
  }();
  return !off && kv_dtype == PA_DTYPE_FP8_E4M3FN && rows_per_group > 16;
}

template <bool PT, bool BS16>
int launch_partition_shared(const PaDecodeArgs& a, hipStream_t stream) {
  const long long blocks = (long long)a.num_seqs * a.num_kv_heads * a.max_num_partitions;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  // ring depth / waves per SIMD: without per-token scales the kernel fits 128 registers, and a fourth workgroup
  // per CU is worth more than a deeper ring (measured); with them it needs about 140
  if constexpr (PT)
    hipLaunchKernelGGL((pa_partition_shared_kernel<true, BS16, 3, 3>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL((pa_partition_shared_kernel<false, BS16, 2, 4>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    g_last_hip_error = (int)e;
    return PA_ERR_LAUNCH;
  }
  return PA_OK;
}

template <int KVT, bool PT, bool BS16>
int launch_partition_nt(const PaDecodeArgs& a, int nt, hipStream_t stream) {
  const int w = waves_per_workgroup(a, nt);
  switch (nt) {
    case 1:
      if (w == 4) return launch_partition_w<1, KVT, PT, BS16, 4>(a, stream);
      if (w == 2) return launch_partition_w<1, KVT, PT, BS16, 2>(a, stream);
      return launch_partition_w<1, KVT, PT, BS16, 1>(a, stream);
    case 2:
      if (w == 2) return launch_partition_w<2, KVT, PT, BS16, 2>(a, stream);
      return launch_partition_w<2, KVT, PT, BS16, 1>(a, stream);
  }
  return PA_ERR_UNSUPPORTED;
}

int launch_reduce(const PaDecodeArgs* a, void* hip_stream, bool skip_single) {
  int rc = check_common(a);
  if (rc) return rc;
  if (!a->output) return PA_ERR_NULL_POINTER;
  if (a->stride_out_h % 2 || a->stride_out_s % 2 || a->stride_tmp_g % 2 || a->stride_tmp_p % 2 ||
      a->stride_tmp_h % 2 || a->stride_tmp_s % 2)
    return PA_ERR_BAD_SHAPE;
  const long long blocks = (long long)a->num_seqs * a->num_kv_heads * ((a->q_len * a->group_size + 15) / 16);
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  // enough rows to fill the GPU's wave slots several times over: four rows per wave
  const bool big = blocks * 16 >= 16384;
  if (skip_single) {
    if (big)
      hipLaunchKernelGGL((pa_reduce_kernel<true, 4>), dim3((unsigned)blocks), dim3(256), 0, stream, *a);
    else
      hipLaunchKernelGGL((pa_reduce_kernel<true, 1>), dim3((unsigned)blocks), dim3(1024), 0, stream, *a);
  } else {
    if (big)
      hipLaunchKernelGGL((pa_reduce_kernel<false, 4>), dim3((unsigned)blocks), dim3(256), 0, stream, *a);
    else
      hipLaunchKernelGGL((pa_reduce_kernel<false, 1>), dim3((unsigned)blocks), dim3(1024), 0, stream, *a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    g_last_hip_error = (int)e;
    return PA_ERR_LAUNCH;
  }
  return PA_OK;
}

}  // namespace

extern "C" {

int pa_decode_abi_version(void) { return PA_DECODE_ABI_VERSION; }
uint32_t pa_decode_args_size(void) { return (uint32_t)sizeof(PaDecodeArgs); }
int pa_decode_last_hip_error(void) { return g_last_hip_error; }

const char* pa_decode_error_string(int code) {
  switch (code) {
    case PA_OK: return "ok";
    case PA_ERR_NULL_POINTER: return "a required pointer is NULL";
    case PA_ERR_BAD_STRUCT: return "PaDecodeArgs.struct_size does not match this library";
    case PA_ERR_UNSUPPORTED: return "unsupported dtype, head size, block size or group size";
    case PA_ERR_BAD_SHAPE: return "bad size, partition size or stride";
    case PA_ERR_LAUNCH: return "HIP launch failed";
    case PA_ERR_NO_DEVICE: return "no HIP device";
  }
  return "unknown error code";
}

int pa_decode_select_partition_size(int32_t num_seqs, int32_t num_kv_heads, int32_t rows_per_group,
                                    int32_t max_context_len, int32_t block_size, int32_t num_cus) {
  (void)block_size;
  if (num_seqs <= 0 || num_kv_heads <= 0 || max_context_len <= 0 || rows_per_group <= 0) return PA_ERR_BAD_SHAPE;
  if (num_cus <= 0) num_cus = device_num_cus();
  // The fewest partitions per sequence that still give every wave slot of the GPU a wave: each extra
  // partition costs a (rows x 128) bf16 partial written and read back plus the merge, and a single
  // partition needs no second kernel at all.  A workgroup (one 16-row query tile) splits its partition over
  // up to 4 waves (at least 256 tokens each); no wave is given more than 2048 tokens, which keeps ragged
  // batches balanced.
  const int total_tiles = (rows_per_group + 15) / 16;
  if (use_shared_stream(PA_DTYPE_FP8_E4M3FN, rows_per_group)) {
    // All row tiles of a kv head in one workgroup that walks its partition alone: three workgroups fit a CU, and
    // no workgroup gets more than 4096 tokens (measured on a ragged batch: 3072-4096 is the flat optimum, 8192
    // costs 7 % in balance, 1024 costs 8 % in partials and merge).
    const long long slots = (long long)num_cus * 3;
    const long long items = (long long)num_seqs * num_kv_heads;
    for (int parts = 1;; ++parts) {
      int ps = (max_context_len + parts - 1) / parts;
      ps = (ps + 255) / 256 * 256;
      if (ps <= 256) return 256;
      if (ps <= 4096 && items * parts >= slots) return ps;
    }
  }
  const int nt = tiles_per_workgroup(total_tiles);
  const int cap_w = nt <= 1 ? 4 : 2;
  const long long slots = (long long)num_cus * 4 * (nt <= 1 ? 2 : 1);
  const long long rows = (long long)num_seqs * num_kv_heads * ((total_tiles + nt - 1) / nt);
  for (int parts = 1;; ++parts) {
    int ps = (max_context_len + parts - 1) / parts;
    ps = (ps + 255) / 256 * 256;
    int w = ps >= 1024 ? 4 : (ps >= 512 ? 2 : 1);
    w = w > cap_w ? cap_w : w;
    if (ps <= 256) return 256;
    if (ps <= 2048 * w && rows * parts * w >= slots) return ps;
  }
}

int pa_decode_partition(const PaDecodeArgs* a, void* hip_stream) {
  int rc = check_common(a);
  if (rc) return rc;
  if (!a->query || !a->key_cache || !a->value_cache || !a->block_tables) return PA_ERR_NULL_POINTER;
  if (a->block_size != 16 && a->block_size != 64 && a->block_size != 1024) return PA_ERR_UNSUPPORTED;
  if (a->kv_dtype != PA_DTYPE_BF16 && a->kv_dtype != PA_DTYPE_FP8_E4M3FN) return PA_ERR_UNSUPPORTED;
  if (a->query_dtype != PA_DTYPE_BF16 && a->query_dtype != PA_DTYPE_FP8_E4M3FN) return PA_ERR_UNSUPPORTED;
  if (a->kv_quant_mode != PA_QUANT_NONE && (!a->key_scale || !a->value_scale)) return PA_ERR_NULL_POINTER;
  if (a->query_quant_mode != PA_QUANT_NONE && !a->query_scale) return PA_ERR_NULL_POINTER;
  if (a->kv_quant_mode < -1 || a->kv_quant_mode > 1 || a->query_quant_mode < -1 || a->query_quant_mode > 1)
    return PA_ERR_UNSUPPORTED;
  const int esz = a->kv_dtype == PA_DTYPE_FP8_E4M3FN ? 1 : 2;
  // 16-byte vector loads: every stride that moves a vector must keep it 16-byte aligned
  if ((a->stride_k_b * esz) % 16 || (a->stride_k_h * esz) % 16 || (a->stride_k_c * esz) % 16 ||
      (a->stride_v_b * esz) % 16 || (a->stride_v_h * esz) % 16 || (a->stride_v_2 * esz) % 16)
    return PA_ERR_BAD_SHAPE;
  const int qsz = a->query_dtype == PA_DTYPE_FP8_E4M3FN ? 1 : 2;
  if ((a->stride_q_s * qsz) % 16 || (a->stride_q_h * qsz) % 16) return PA_ERR_BAD_SHAPE;
  if ((a->stride_tmp_g * 2) % 16 || (a->stride_tmp_p * 2) % 16 || (a->stride_tmp_h * 2) % 16 || (a->stride_tmp_s * 2) % 16 ||
      (reinterpret_cast<uintptr_t>(a->tmp_output) & 15))
    return PA_ERR_BAD_SHAPE;
  if (a->kv_quant_mode == PA_QUANT_PER_TOKEN && (a->stride_kvscale_b % 4 || a->stride_kvscale_h % 4))
    return PA_ERR_BAD_SHAPE;
  if ((long long)(4 * 3 + 3) * a->stride_k_c * esz + 15 * 16 >= (1LL << 32)) return PA_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(a->key_cache) | reinterpret_cast<uintptr_t>(a->value_cache) |
       reinterpret_cast<uintptr_t>(a->query)) & 15)
    return PA_ERR_BAD_SHAPE;

  const int Ge = a->q_len * a->group_size;
  const int nt = tiles_per_workgroup((Ge + 15) / 16);
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  const bool pt = a->kv_quant_mode == PA_QUANT_PER_TOKEN;
  if (a->kv_dtype == PA_DTYPE_FP8_E4M3FN) {
    // constant in-page strides: block size 16 with the default dense layout
    const bool bs16 = a->block_size == 16 && a->stride_k_c == 256 &&
                      (a->v_transposed ? a->stride_v_2 == 2048 : a->stride_v_2 == 16);
    if (use_shared_stream(a->kv_dtype, Ge)) {
      if (bs16) return pt ? launch_partition_shared<true, true>(*a, stream) : launch_partition_shared<false, true>(*a, stream);
      return pt ? launch_partition_shared<true, false>(*a, stream) : launch_partition_shared<false, false>(*a, stream);
    }
    if (bs16)
      return pt ? launch_partition_nt<PA_DTYPE_FP8_E4M3FN, true, true>(*a, nt, stream)
                : launch_partition_nt<PA_DTYPE_FP8_E4M3FN, false, true>(*a, nt, stream);
    return pt ? launch_partition_nt<PA_DTYPE_FP8_E4M3FN, true, false>(*a, nt, stream)
              : launch_partition_nt<PA_DTYPE_FP8_E4M3FN, false, false>(*a, nt, stream);
  }
  if (pt) return PA_ERR_UNSUPPORTED;  // per-token scales belong to the FP8 cache
  return launch_partition_nt<PA_DTYPE_BF16, false, false>(*a, nt, stream);
}

int pa_decode_reduce(const PaDecodeArgs* a, void* hip_stream) { return launch_reduce(a, hip_stream, false); }

int pa_decode(const PaDecodeArgs* a, void* hip_stream) {
  if (a && a->struct_size == sizeof(PaDecodeArgs) && !a->output) return PA_ERR_NULL_POINTER;
  int rc = pa_decode_partition(a, hip_stream);
  if (rc) return rc;
  // the partition kernel has written the rows of every sequence that fits in one partition itself
  if (a->max_num_partitions == 1 && !a->sinks) return PA_OK;
  return launch_reduce(a, hip_stream, true);
}

int pa_debug_fp8_decode(const uint8_t* codes, float* out, int32_t n, void* hip_stream) {
  if (!codes || !out) return PA_ERR_NULL_POINTER;
  if (n <= 0) return PA_ERR_BAD_SHAPE;
  hipLaunchKernelGGL(pa_fp8_decode_kernel, dim3((n + 255) / 256), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(hip_stream), codes, out, n);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    g_last_hip_error = (int)e;
    return PA_ERR_LAUNCH;
  }
  return PA_OK;
}

}  // extern "C"

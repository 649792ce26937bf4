// Scaled dot-product attention forward on MFMA (flash-attention style: scores
// never leave the CU).
//
// One workgroup of 8 wavefronts owns 256 query rows of one (batch, head); each
// wavefront owns 32 of them and walks the keys in tiles of 64:
//   * K and V tiles go global -> LDS by LDS-DMA into a ring of stages, two
//     tiles ahead of the math; K rows are read back with 16-byte loads, V with
//     the transposing 8-byte loads, both conflict-free by chunk permutation;
//   * scores are computed TRANSPOSED, S^T = K Q^T, so that an MFMA lane holds
//     32 scores of ONE query: the row maximum and row sum of the online
//     softmax are in-register reductions plus one exchange between the two
//     half-wavefronts, and the probabilities, rounded to the input type, are
//     already laid out as the MFMA operand of O^T += V^T P^T;
//   * Q fragments stay in registers for the whole kernel; the output
//     accumulator O^T is rescaled only when some row maximum moved;
//   * causal workgroups stop at the diagonal, and a wavefront skips tiles that
//     lie wholly above its own rows;
//   * a mask tensor (boolean, or additive in f32 / bf16 / f16, broadcast over
//     batch and heads as its dims say): every wavefront brings the 32 x 64
//     mask elements of its next tile into an LDS region of its own by LDS-DMA
//     (whole rows, coalesced) and reads them back in the score layout, four
//     consecutive keys per lane and read, one MFMA phase after the load was
//     issued; masks whose rows are not 16-byte aligned are read straight into
//     registers instead (MASK == 1), four keys per load;
//   * the two wavefronts of a SIMD (w and w + 4) alternate: a tile is an MFMA
//     phase (S^T of tile t and the O^T update of tile t - 1, 32 MFMAs) and a
//     vector-ALU phase (online softmax of tile t) of about equal length,
//     separated by workgroup barriers, and wavefronts 4..7 run one phase behind
//     wavefronts 0..3 -- the matrix pipe works on one wavefront's tile while
//     the other computes its exponentials.
//
// Head dim 64 or 128 (template parameter); bf16 or f16.
//
// Reference semantics: aten.scaled_dot_product_attention (reference
// support/asm_emitter.h:2409-2468, node/sdpa_node.h:36-236), GQA by head
// repetition, causal mask aligned top-left; mask tensors as in
// node/sdpa_node.h:138-176 (rank 4, every dim 1 or the full extent).
#include "common.h"
#include "fast_paths.h"

#include <type_traits>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

#define SD_AS1 __attribute__((address_space(1)))
#define SD_AS3 __attribute__((address_space(3)))

constexpr int kBQ = 256;        // query rows per workgroup
constexpr int kBKV = 64;        // keys per tile
constexpr int kWaves = 8;
constexpr int kStages = 3;
constexpr float kNegBig = -1.0e30f;
constexpr float kMaxSlack = 8.0f; // see the softmax phase
constexpr float kRedoSum = 8192.0f; // 32 probabilities of 2^kMaxSlack

// Sizes that follow from the head dimension HD (Q/K and V), 64 or 128.
template <int HD> struct SdShape {
  static constexpr int kRowB = HD * 2;             // bytes per K / V row
  static constexpr int kChunks = kRowB / 16;       // 16-byte chunks per row
  static constexpr int kRowsPerLoad = 64 / kChunks; // rows of one wave DMA
  static constexpr int kTileB = kBKV * kRowB;      // one K (or V) tile
  static constexpr int kLoadsPerTile = kTileB / 1024 / kWaves; // per wave
  static constexpr int kOutPitch = kRowB + 16;     // epilogue rows, padded
  static constexpr int kRingB = 2 * kStages * kTileB; // K ring and V ring
  static constexpr int kLdsB = kRingB > kWaves * 32 * kOutPitch
                                   ? kRingB
                                   : kWaves * 32 * kOutPitch;
  // kernels that stage the mask: 8 KB per wavefront behind the rings
  static constexpr int kMaskB = 8192;
  static constexpr int kLdsMaskB = kLdsB + kWaves * kMaskB;
};

struct SdpaArgs {
  const char *q, *k, *v;
  char *o;
  int64_t q_sb, q_sh, q_ss; // strides in elements (last dim contiguous)
  int64_t k_sb, k_sh, k_ss;
  int64_t v_sb, v_sh, v_ss;
  int64_t o_sb, o_sh, o_ss;
  int32_t Sq, Skv, group; // group = Hq / Hkv
  int32_t causal;
  // XCD-aware order of a one-dimensional grid (0: the grid is heads x batch x
  // query-tile groups): heads and query-tile groups per head
  int32_t xcd_heads, xcd_groups;
  float scale_log2e; // softmax scale * log2(e)
  float scale;       // softmax scale
  // mask tensor (kernels with MASK): strides in elements, 0 where broadcast;
  // the key stride is 1
  const char *mask;
  int64_t m_sb, m_sh, m_sq;
  uint32_t m_bytes; // bytes of one (batch, head) slab
  int32_t m_dt;     // FHIP_BOOLEAN / FHIP_FLOAT / FHIP_BFLOAT16 / FHIP_HALF
};

template <int N, typename F> __device__ __forceinline__ void sd_static_for(F &&f) {
  if constexpr (N > 0) {
    sd_static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

template <bool BF16>
__device__ __forceinline__ f32x16 sd_mfma(const uint32_t (&a)[4],
                                          const uint32_t (&b)[4], f32x16 c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
        __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// two floats -> one register of two 16-bit values (lo = a)
template <bool BF16> __device__ __forceinline__ uint32_t sd_pack(float a, float b) {
  if constexpr (BF16) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v;
    v[0] = (__bf16)a;
    v[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, v);
  } else {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    f16x2 v;
    v[0] = (_Float16)a;
    v[1] = (_Float16)b;
    return __builtin_bit_cast(uint32_t, v);
  }
}

// maximum / sum over the two half-wavefronts (lanes l and l ^ 32)
__device__ __forceinline__ float sd_half_max(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const uint32_t r0 = r[0], r1 = r[1];
  return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}
__device__ __forceinline__ float sd_half_sum(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const uint32_t r0 = r[0], r1 = r[1];
  return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

// Chunk permutation of the K tile (16-byte reads, 16 consecutive rows at one
// chunk index per pass): position of chunk c in row `row` is c ^ sd_kswz(row).
template <int HD> __device__ __forceinline__ int sd_kswz(int row) {
  if constexpr (HD == 128)
    return row & 15;
  else // 128-byte rows: two rows share the 64 banks
    return (row & 7) ^ ((row >> 3) & 1);
}

// Chunk permutation of the V tile (read by transposing 8-byte loads): spreads
// the 4 rows x 64 bytes a half-wavefront touches over all 64 banks.  sd_vpos
// maps a chunk to its position in the row, sd_vchunk is its inverse; both
// depend on the row only through row % 4, which the fragment walk (steps of 8
// rows) preserves.
template <int HD> __device__ __forceinline__ int sd_vpos(int row, int c) {
  if constexpr (HD == 128)
    return c ^ ((row & 3) << 1) ^ ((c & 2) << 2);
  else // rows r and r + 2 start in the same bank: swap the row's halves
    return c ^ (((row >> 1) & 1) << 2);
}
template <int HD> __device__ __forceinline__ int sd_vchunk(int row, int p) {
  if constexpr (HD == 128) {
    const int t = p ^ ((row & 3) << 1);
    return t ^ ((t & 2) << 2);
  } else {
    return p ^ (((row >> 1) & 1) << 2);
  }
}

__device__ __forceinline__ constexpr int sd_wait_imm(int vm) {
  return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | (0x0 << 8);
}

// Transposing 8-byte LDS read (4 consecutive rows of one 16-bit column per
// lane) that the compiler does not see as a memory access, and the wait that
// goes with it: at most N LDS operations still outstanding, after which the
// two registers may be used.
template <int OFFSET>
__device__ __forceinline__ void sd_read_tr16(u32x2 &dst, uint32_t addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "16-bit offset field");
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
               : "=v"(dst)
               : "v"(addr), "n"(OFFSET));
}
template <int OFFSET>
__device__ __forceinline__ void sd_read_b32(uint32_t &dst, uint32_t addr) {
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET));
}
template <int OFFSET>
__device__ __forceinline__ void sd_read_b64(u32x2 &dst, uint32_t addr) {
  asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET));
}
template <int OFFSET>
__device__ __forceinline__ void sd_read_b128(u32x4 &dst, uint32_t addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "16-bit offset field");
  asm volatile("ds_read_b128 %0, %1 offset:%2"
               : "=v"(dst)
               : "v"(addr), "n"(OFFSET));
}
template <int N, typename... R>
__device__ __forceinline__ void sd_wait_pin(R &...regs) {
  static_assert(N >= 0 && N <= 15, "lgkmcnt is a 4-bit field");
  if constexpr (sizeof...(R) == 4) {
    auto f = [](auto &a, auto &b, auto &c, auto &d) {
      asm volatile("s_waitcnt lgkmcnt(%4)"
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d)
                   : "n"(N));
    };
    f(regs...);
  } else {
    static_assert(sizeof...(R) == 8, "four or eight register tuples");
    auto f = [](auto &a, auto &b, auto &c, auto &d, auto &e, auto &g, auto &h,
                auto &i) {
      asm volatile("s_waitcnt lgkmcnt(%8)"
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(g),
                     "+v"(h), "+v"(i)
                   : "n"(N));
    };
    f(regs...);
  }
}

// Workgroup barrier without the release fence's "wait for everything": the
// callers wait for exactly the loads whose data the other wavefronts need
// (LDS-DMA completion is on the vector-memory counter, LDS reads have been
// consumed by the MFMAs before every barrier); the empty asm statements keep
// the compiler from moving memory operations across.
__device__ __forceinline__ void sd_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// MASK: 0 no mask tensor, 1 mask read into registers, 2 mask staged in LDS
template <bool BF16, bool CAUSAL, int HD, int MASK>
__global__ __launch_bounds__(kWaves * 64) void sdpa_fwd_kernel(SdpaArgs g) {
  static_assert(!(CAUSAL && MASK), "a mask tensor excludes the causal flag");
  using C = SdShape<HD>;
  constexpr int kD = HD;
  constexpr int kRowB = C::kRowB, kTileB = C::kTileB;
  constexpr int kLoadsPerTile = C::kLoadsPerTile, kOutPitch = C::kOutPitch;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  // wave index as a scalar: everything derived from it stays in SGPRs
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l = threadIdx.x & 63;
  const int half = l >> 5, lq = l & 31;
  // Causal masks: a workgroup runs query tile (last - z) and then tile z, a
  // long and a short one, so all workgroups do the same work (tiles of one
  // head need 1 .. n key-tile rows).  Otherwise one tile per workgroup.
  // Hardware deals consecutive workgroup ids to the 8 XCDs in turn.  All query
  // tiles of a (batch, head) read the same K and V: the remapped order runs
  // them side by side on one XCD, so that its L2 fetches every K / V tile once
  // for all of them.
  int h = blockIdx.x, b = blockIdx.y, z = blockIdx.z;
  if (g.xcd_heads) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    z = slot % g.xcd_groups;
    const int head = (slot / g.xcd_groups) * 8 + xcd;
    h = head % g.xcd_heads;
    b = head / g.xcd_heads;
  }
  const int n_qtiles = (g.Sq + kBQ - 1) / kBQ;
  const int passes = CAUSAL && n_qtiles - 1 - z != z ? 2 : 1;
  for (int pass = 0; pass < passes; ++pass) {
  const int qtile = CAUSAL && pass == 0 ? n_qtiles - 1 - z : z;
  if (pass) // the first tile's output staging has been read
    __builtin_amdgcn_s_barrier();
  const int hk = h / g.group;
  const int q0 = qtile * kBQ;
  const int qw0 = q0 + wave * 32; // first query row of this wavefront
  const int qrow = qw0 + lq;      // query this lane's scores belong to

  const char *qp = g.q + (b * g.q_sb + h * g.q_sh) * 2;
  const char *kp = g.k + (b * g.k_sb + hk * g.k_sh) * 2;
  const char *vp = g.v + (b * g.v_sb + hk * g.v_sh) * 2;
  const int64_t k_rowb = g.k_ss * 2, v_rowb = g.v_ss * 2;
  const int64_t k_bytes = (int64_t)(g.Skv - 1) * k_rowb + kRowB;
  const int64_t v_bytes = (int64_t)(g.Skv - 1) * v_rowb + kRowB;

  // number of key tiles this workgroup visits
  int kv_end = g.Skv;
  if (CAUSAL) {
    const int last_q = q0 + kBQ - 1 < g.Sq - 1 ? q0 + kBQ - 1 : g.Sq - 1;
    kv_end = last_q + 1 < g.Skv ? last_q + 1 : g.Skv;
  }
  const int tiles = (kv_end + kBKV - 1) / kBKV;

  // ---- Q fragments (B operand of S^T = K Q^T): row lq, 8 d per register quad
  uint32_t qf[kD / 16][4];
  {
    const int qr = qrow < g.Sq ? qrow : g.Sq - 1;
    const char *src = qp + (int64_t)qr * g.q_ss * 2 + half * 16;
#pragma unroll
    for (int ds = 0; ds < kD / 16; ++ds) {
      const u32x4 v = *(const SD_AS1 u32x4 *)(src + ds * 32);
      qf[ds][0] = v.x;
      qf[ds][1] = v.y;
      qf[ds][2] = v.z;
      qf[ds][3] = v.w;
    }
  }

  // ---- DMA addressing: a wave instruction moves 1 KB, 4 or 8 whole rows ------
  uint32_t koff[kLoadsPerTile], voff[kLoadsPerTile];
#pragma unroll
  for (int j = 0; j < kLoadsPerTile; ++j) {
    const int row = (j * kWaves + wave) * C::kRowsPerLoad + l / C::kChunks;
    const int p = l % C::kChunks;
    koff[j] = (uint32_t)(row * k_rowb + ((p ^ sd_kswz<HD>(row)) << 4));
    voff[j] = (uint32_t)(row * v_rowb + (sd_vchunk<HD>(row, p) << 4));
  }
  // K tiles live in stages [0, kStages), V tiles in [kStages, 2 kStages).
  // One buffer descriptor per operand covers the whole (batch, head) slab; the
  // tile's byte offset is added to the lanes' offsets.  Rows at or past Skv
  // read as zeros (out of the descriptor's range), and so do whole tiles past
  // the end, whose offset is pushed out of range.
  auto slab_rsrc = [&](const char *base, int64_t bytes) {
    const uint64_t b64 = (uint64_t)base;
    const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64);
    const uint32_t bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
    return __builtin_amdgcn_make_buffer_rsrc(
        (void *)(((uint64_t)bhi << 32) | blo), 0,
        (int)__builtin_amdgcn_readfirstlane((uint32_t)bytes), 0x00020000);
  };
  const __amdgpu_buffer_rsrc_t k_rsrc = slab_rsrc(kp, k_bytes);
  const __amdgpu_buffer_rsrc_t v_rsrc = slab_rsrc(vp, v_bytes);
  // Mask: a lane's 32 scores of a tile are 8 runs of 4 consecutive keys (run i
  // starts at key 32 * (i / 4) + 8 * (i % 4) + 4 * half); the element size
  // picks the access width.  Runs past the slab's end read as zeros; their
  // keys are dead anyway.
  const int m_esh = !MASK ? 0 : g.m_dt == FHIP_BOOLEAN ? 0 : g.m_dt == FHIP_FLOAT ? 2 : 1;
  __amdgpu_buffer_rsrc_t m_rsrc = k_rsrc;
  if constexpr (MASK != 0)
    m_rsrc = slab_rsrc(g.mask + ((b * g.m_sb + h * g.m_sh) << m_esh), g.m_bytes);
  // MASK == 1: one register load per run, issued at the top of a round
  uint32_t m_off = 0;
  if constexpr (MASK == 1) {
    const int qr = qrow < g.Sq ? qrow : g.Sq - 1;
    m_off = (uint32_t)(((int64_t)qr * g.m_sq + half * 4) << m_esh);
  }
  u32x4 mreg[MASK == 1 ? 8 : 1];
  auto load_mask = [&](int t) {
    const int so = (t * kBKV) << m_esh;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int run = 32 * (i / 4) + 8 * (i % 4);
      if (m_esh == 0) {
        mreg[i].x = __builtin_amdgcn_raw_buffer_load_b32(m_rsrc, (int)m_off + run, so, 0);
      } else if (m_esh == 1) {
        const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(m_rsrc, (int)m_off + run * 2, so, 0);
        mreg[i].x = v.x;
        mreg[i].y = v.y;
      } else {
        mreg[i] = __builtin_amdgcn_raw_buffer_load_b128(m_rsrc, (int)m_off + run * 4, so, 0);
      }
    }
  };
  // MASK == 2: the tile's 32 rows of 64 elements go to this wavefront's LDS
  // region by LDS-DMA, 1 KB (16 / 8 / 4 whole rows) per instruction; chunk c of
  // row r sits at position c ^ ((r / 2) % chunks-per-row), which spreads the
  // runs that the lanes of a read touch over the banks.
  const uint32_t m_lds = lds0 + (uint32_t)C::kLdsB + (uint32_t)wave * C::kMaskB;
  uint32_t m_dma[MASK == 2 ? 8 : 1]; // lane offsets of the DMA instructions
  uint32_t m_rd[MASK == 2 ? 8 : 1];  // LDS address of this lane's run i
  if constexpr (MASK == 2) {
    const int cpr = 4 << m_esh;        // 16-byte chunks per row
    const int rows_per = 64 / cpr;     // rows per instruction
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = j * rows_per + l / cpr;
      const int c = (l % cpr) ^ ((row >> 1) & (cpr - 1));
      const int qr = qw0 + row < g.Sq ? qw0 + row : g.Sq - 1;
      m_dma[j] = (uint32_t)((((int64_t)qr * g.m_sq) << m_esh) + c * 16);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int bo = (32 * (i / 4) + 8 * (i % 4) + 4 * half) << m_esh;
      const int c = (bo >> 4) ^ ((lq >> 1) & (cpr - 1));
      m_rd[i] = m_lds + (uint32_t)(lq * (64 << m_esh) + (c << 4) + (bo & 15));
    }
  }
  auto issue_mask = [&](int t) {
    const int so = t < tiles ? (t * kBKV) << m_esh : 0;
    const int n = 2 << m_esh; // instructions per tile
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < n)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            m_rsrc,
            (SD_AS3 char *)(uintptr_t)__builtin_amdgcn_readfirstlane(m_lds + j * 1024u),
            16, (int)m_dma[j], so, 0, 0);
  };
  // the staged loads still in flight next to the K / V loads of a round
  auto wait_all_but_round = [&]() {
    if (MASK != 2)
      __builtin_amdgcn_s_waitcnt(sd_wait_imm(2 * kLoadsPerTile));
    else if (m_esh == 0)
      __builtin_amdgcn_s_waitcnt(sd_wait_imm(2 * kLoadsPerTile + 2));
    else if (m_esh == 1)
      __builtin_amdgcn_s_waitcnt(sd_wait_imm(2 * kLoadsPerTile + 4));
    else
      __builtin_amdgcn_s_waitcnt(sd_wait_imm(2 * kLoadsPerTile + 8));
  };
  auto issue_kv = [&](const __amdgpu_buffer_rsrc_t &r, uint32_t tile_bytes,
                      const uint32_t (&off)[kLoadsPerTile], int t,
                      uint32_t stage) {
    const uint32_t toff = t < tiles ? (uint32_t)t * tile_bytes : 0x80000000u;
#pragma unroll
    for (int j = 0; j < kLoadsPerTile; ++j) {
      const uint32_t dst = stage + (uint32_t)(j * kWaves + wave) * 1024u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          r, (SD_AS3 char *)(uintptr_t)__builtin_amdgcn_readfirstlane(dst), 16,
          (int)(off[j] + toff), 0, 0, 0);
    }
  };
  // ring slot (0 .. kStages - 1) -> LDS address
  auto k_stage = [&](int slot) { return lds0 + (uint32_t)slot * kTileB; };
  auto v_stage = [&](int slot) {
    return lds0 + (uint32_t)(kStages + slot) * kTileB;
  };
  auto issue_k = [&](int t, int slot) {
    issue_kv(k_rsrc, (uint32_t)(kBKV * k_rowb), koff, t, k_stage(slot));
  };
  auto issue_v = [&](int t, int slot) {
    issue_kv(v_rsrc, (uint32_t)(kBKV * v_rowb), voff, t, v_stage(slot));
  };
  auto next_slot = [](int s) { return s + 1 == kStages ? 0 : s + 1; };

  // ---- fragment addressing ----------------------------------------------------
  // K (A operand of S^T): row lq of a 32-key block, 16-byte chunk 2*ds + half
  // (the chunk index is ds * 2 + half XOR a value below 16: K-step ds moves
  // the address by XOR with ds << 5, which costs one instruction per read and
  // saves a register per K-step; the stages start on multiples of 16 KB)
  const uint32_t kaddr0 = (uint32_t)(lq * kRowB + ((half ^ sd_kswz<HD>(lq)) << 4));
  // V^T (A operand of O^T += V^T P^T): the keys a lane needs are those whose
  // probabilities it holds: key = 32*kb + 8*(i/4) + 4*half + i%4 for score
  // register i; one transposing read returns 4 consecutive keys of one column
  // (chunk dt * 4 + x with x < 4: both permutations leave the dt bits alone,
  // so feature block dt moves the address by XOR with dt << 6)
  uint32_t vaddr0;
  {
    const int L = l & 15, h16 = (l >> 4) & 1;
    const int row = half * 4 + (L >> 2);
    const int c = h16 * 2 + ((L & 3) >> 1);
    vaddr0 = (uint32_t)(row * kRowB + (sd_vpos<HD>(row, c) << 4) + (L & 1) * 8);
  }

  f32x16 o[kD / 32];
#pragma unroll
  for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      o[dt][r] = 0.f;
  float m_run = kNegBig; // running row maximum (raw scores), same in both halves
  float l_run = 0.f;     // running row sum, this half's share

  // ---- rounds ---------------------------------------------------------------
  // Per key tile t a wavefront runs
  //   MFMA(t): S^T of tile t (K tile t) and O^T += V^T P^T of tile t - 1
  //   VALU(t): online softmax of tile t
  // and one workgroup barrier.  Wavefronts 0..3 place the barrier after
  // VALU(t), wavefronts 4..7 after MFMA(t): between two barriers one team
  // runs MFMA(t + 1), VALU(t + 1) and the other VALU(t), MFMA(t + 1), so the
  // two wavefronts of a SIMD use the matrix pipe and the vector ALU in turn
  // without waiting for each other in the middle.  Between barrier t and
  // barrier t + 1 only K tile t + 1 and V tile t are read; the loads issued at
  // the top of round t (K tile t + 2, V tile t + 1) reuse the stages of K tile
  // t - 1 and V tile t - 2 and have to land by barrier t + 1.
  const int team = __builtin_amdgcn_readfirstlane(wave >> 2);
  constexpr bool kLoadsInValuPhase = MASK == 0 && HD == 128;
#ifndef SD_FUSE_PLAIN
#define SD_FUSE_PLAIN 0
#endif
  constexpr bool kFusedPipeline = MASK != 0 || SD_FUSE_PLAIN;
  if constexpr (MASK == 2)
    issue_mask(0); // older than every K / V load: landed by the first wait
  issue_k(0, 0);
  issue_v(0, 0);
  issue_k(1, 1);
  // K tile 0 has landed
  __builtin_amdgcn_s_waitcnt(sd_wait_imm(2 * kLoadsPerTile));
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

  uint32_t pf[4][4]; // probabilities as B-operand fragments, 16 keys each
  // a wavefront whose rows all lie above a tile has nothing to add
  auto active = [&](int t) { return !(CAUSAL && t * kBKV > qw0 + 31); };
  // ring slots of tile t - 1, t, t + 1, t + 2 (slot of t + 2 == slot of t - 1)
  int sl_prev = kStages - 1, sl_cur = 0, sl_next = 1;
  // One round.  The first (tile 0: no O^T update, and the softmax always takes
  // its full route) and the last (t == tiles: only the O^T update of the last
  // tile) are peeled off the loop as straight-line code, so that the loop holds
  // a single variant of the MFMA pipeline.
  auto round = [&](const int t, auto which_c) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(which_c)::value == 0;
    constexpr bool LAST = decltype(which_c)::value == 2;
    f32x16 s[2]; // scores of tile t: written by the MFMA phase, read by the softmax
    // (the mask first: the waits below count the K / V loads issued after it)
    if constexpr (MASK == 1)
      if (t < tiles)
        load_mask(t);
    // This round's loads, K tile t + 2 and V tile t + 1.  Under memory
    // back-pressure every LDS-DMA instruction holds its wavefront at issue for
    // tens of clocks.  They go in front of the shorter of a round's two phases:
    // the MFMA phase with a mask tensor or head dim 64, the vector-ALU phase
    // otherwise (the SIMD's other wavefront feeds the matrix pipe meanwhile).
    if constexpr (!kLoadsInValuPhase) {
      issue_k(t + 2, sl_prev);
      issue_v(t + 1, sl_next);
    }
    // ---- MFMA phase -----------------------------------------------------------
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(2);
    // The phase is one software pipeline over up to 32 MFMAs: NS for S^T of
    // tile t (ds-major, kb-minor: K fragment m, Q fragment m / 2), then NP for
    // O^T += V^T P^T of tile t - 1 (j-major, dt-minor).  Every MFMA takes a
    // fresh A fragment from LDS (one 16-byte read of K, or two transposing
    // 8-byte reads of V).  The reads are written as asm: the compiler neither
    // sees them as LDS accesses (it would make the transposing reads wait for
    // every outstanding global -> LDS load, the tiles fetched ahead included)
    // nor waits for them; they run kAhead MFMAs ahead, straight across the
    // boundary between the two products, and one sd_wait_pin per kGroup MFMAs
    // waits for that group's fragments.
    constexpr int kAhead = 8, kGroup = 4;
    constexpr int NS = 2 * (kD / 16), NP = 4 * (kD / 32);
    static_assert(NS % kGroup == 0 && NP % kGroup == 0 && NS >= kAhead && NP >= kAhead,
                  "groups do not straddle the two products");
    auto mfma_range = [&](auto first_c, auto last_c) __attribute__((always_inline)) {
      constexpr int M0 = decltype(first_c)::value, M1 = decltype(last_c)::value;
      const uint32_t sk = k_stage(sl_cur) + kaddr0, sv = v_stage(sl_prev) + vaddr0;
      u32x4 kr[NS];
      u32x2 vr[NP][2];
      auto read = [&](auto mc) __attribute__((always_inline)) {
        constexpr int m = decltype(mc)::value;
        if constexpr (m < NS) {
          sd_read_b128<(m % 2) * 32 * kRowB>(kr[m], sk ^ (uint32_t)((m / 2) << 5));
        } else {
          constexpr int j = (m - NS) / (kD / 32), dt = (m - NS) % (kD / 32);
          const uint32_t ad = sv ^ (uint32_t)(dt << 6);
          sd_read_tr16<(j * 16 + 0) * kRowB>(vr[m - NS][0], ad);
          sd_read_tr16<(j * 16 + 8) * kRowB>(vr[m - NS][1], ad);
        }
      };
      sd_static_for<kAhead>([&](auto ic) {
        read(std::integral_constant<int, M0 + decltype(ic)::value>{});
      });
      sd_static_for<(M1 - M0) / kGroup>([&](auto gc) {
        constexpr int m0 = M0 + decltype(gc)::value * kGroup;
        // LDS operations younger than this group's: the next group's reads
        constexpr int n1 = m0 + 2 * kGroup < M1 ? m0 + 2 * kGroup : M1;
        constexpr int young_k = n1 < NS ? n1 - (m0 + kGroup) : (m0 + kGroup < NS ? NS - (m0 + kGroup) : 0);
        constexpr int young = n1 <= m0 + kGroup ? 0 : young_k + 2 * ((n1 - (m0 + kGroup)) - young_k);
        if constexpr (m0 < NS) {
          sd_wait_pin<young>(kr[m0], kr[m0 + 1], kr[m0 + 2], kr[m0 + 3]);
#pragma unroll
          for (int i = 0; i < kGroup; ++i) {
            const int m = m0 + i;
            const uint32_t kf[4] = {kr[m].x, kr[m].y, kr[m].z, kr[m].w};
            f32x16 zero;
#pragma unroll
            for (int r = 0; r < 16; ++r)
              zero[r] = 0.f;
            s[m % 2] = sd_mfma<BF16>(kf, qf[m / 2], m < 2 ? zero : s[m % 2]);
          }
        } else {
          constexpr int v0 = m0 - NS;
          sd_wait_pin<young>(vr[v0][0], vr[v0][1], vr[v0 + 1][0], vr[v0 + 1][1],
                             vr[v0 + 2][0], vr[v0 + 2][1], vr[v0 + 3][0], vr[v0 + 3][1]);
#pragma unroll
          for (int i = 0; i < kGroup; ++i) {
            const int m = v0 + i;
            const int j = m / (kD / 32), dt = m % (kD / 32);
            const uint32_t vf[4] = {vr[m][0].x, vr[m][0].y, vr[m][1].x, vr[m][1].y};
            o[dt] = sd_mfma<BF16>(vf, pf[j], o[dt]);
          }
        }
        __builtin_amdgcn_sched_barrier(0); // keep the MFMAs at their wait
        sd_static_for<kGroup>([&](auto ic) {
          constexpr int m = m0 + kAhead + decltype(ic)::value;
          if constexpr (m < M1)
            read(std::integral_constant<int, m>{});
        });
      });
    };
    {
      using I0 = std::integral_constant<int, 0>;
      using IS = std::integral_constant<int, NS>;
      using IE = std::integral_constant<int, NS + NP>;
      // A tile that is live for a wavefront has a live predecessor.  In the
      // round after a wavefront's last live tile S^T of a dead tile is computed
      // along with the O^T update and never looked at: a second variant of the
      // pipeline inside the loop costs registers the kernel does not have.
      if constexpr (FIRST) {
        mfma_range(I0{}, IS{});
      } else if constexpr (LAST) {
        if (active(t - 1))
          mfma_range(IS{}, IE{});
      } else if constexpr (kFusedPipeline) {
        if (active(t - 1))
          mfma_range(I0{}, IE{});
      } else {
        if (active(t))
          mfma_range(I0{}, IS{});
        if (active(t - 1))
          mfma_range(IS{}, IE{});
      }
    }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
    // wavefronts 4..7 end their round here: everything but the loads of this
    // round has landed (which, in the vector-ALU phase, have not been issued
    // yet)
    if (team) {
      __builtin_amdgcn_s_waitcnt(sd_wait_imm(kLoadsInValuPhase ? 0 : 2 * kLoadsPerTile));
      sd_barrier();
    }
    if constexpr (LAST)
      return;
    if constexpr (kLoadsInValuPhase) {
      issue_k(t + 2, sl_prev);
      issue_v(t + 1, sl_next);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- vector-ALU phase -------------------------------------------------------
    if (active(t)) {
      const int kv0 = t * kBKV;
      // with a mask the scores are scaled here, with the mask folded in, and
      // the softmax below converts them to log2 units
      const float sl2 = MASK ? 1.4426950408889634f : g.scale_log2e;
      if constexpr (MASK != 0) {
        // s <- s * scale + mask, or -inf where a boolean mask is false (one
        // multiply-add per score; the softmax below then runs in natural-log
        // units, its scale being log2(e))
        // (one loop per element kind: the kind is a run-time value, and a
        // choice per score would cut the loop into 32 scalar branches)
        auto fold_with = [&](auto value) __attribute__((always_inline)) {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              s[kb][r] = value(kb * 4 + (r >> 2), r & 3, s[kb][r]);
        };
        auto fold = [&](const u32x4 (&mraw)[8]) __attribute__((always_inline)) {
          const float scale = g.scale;
          if (m_esh == 0) {
            fold_with([&](int i, int e, float sv) {
              return ((mraw[i].x >> (8 * e)) & 0xffu) != 0 ? sv * scale : -INFINITY;
            });
          } else if (m_esh == 2) {
            // (through a scalar: bit-casting a vector's element in place
            // reads element 0)
            fold_with([&](int i, int e, float sv) {
              const u32x4 w = mraw[i];
              const uint32_t word = e == 0 ? w.x : e == 1 ? w.y : e == 2 ? w.z : w.w;
              return __builtin_fmaf(sv, scale, __builtin_bit_cast(float, word));
            });
          } else if (g.m_dt == FHIP_BFLOAT16) {
            fold_with([&](int i, int e, float sv) {
              const uint32_t word = e < 2 ? mraw[i].x : mraw[i].y;
              const float mv =
                  __builtin_bit_cast(float, (e & 1) ? (word & 0xffff0000u) : (word << 16));
              return __builtin_fmaf(sv, scale, mv);
            });
          } else {
            fold_with([&](int i, int e, float sv) {
              const uint32_t word = e < 2 ? mraw[i].x : mraw[i].y;
              const float mv =
                  (float)__builtin_bit_cast(_Float16, (uint16_t)((e & 1) ? word >> 16 : word));
              return __builtin_fmaf(sv, scale, mv);
            });
          }
        };
        if constexpr (MASK == 1) {
          fold(mreg);
        } else {
          u32x4 mraw[8];
          // the tile's mask was issued a round ago, before this round's K / V
          __builtin_amdgcn_s_waitcnt(sd_wait_imm(2 * kLoadsPerTile));
          asm volatile("" ::: "memory");
          if (m_esh == 2) {
            sd_static_for<8>([&](auto ic) {
              sd_read_b128<0>(mraw[decltype(ic)::value], m_rd[decltype(ic)::value]);
            });
            sd_wait_pin<0>(mraw[0], mraw[1], mraw[2], mraw[3], mraw[4], mraw[5],
                           mraw[6], mraw[7]);
          } else if (m_esh == 1) {
            u32x2 t2[8];
            sd_static_for<8>([&](auto ic) {
              sd_read_b64<0>(t2[decltype(ic)::value], m_rd[decltype(ic)::value]);
            });
            sd_wait_pin<0>(t2[0], t2[1], t2[2], t2[3], t2[4], t2[5], t2[6], t2[7]);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              mraw[i].x = t2[i].x;
              mraw[i].y = t2[i].y;
            }
          } else {
            uint32_t t1[8];
            sd_static_for<8>([&](auto ic) {
              sd_read_b32<0>(t1[decltype(ic)::value], m_rd[decltype(ic)::value]);
            });
            sd_wait_pin<0>(t1[0], t1[1], t1[2], t1[3], t1[4], t1[5], t1[6], t1[7]);
#pragma unroll
            for (int i = 0; i < 8; ++i)
              mraw[i].x = t1[i];
          }
          // the region is free again: next tile's mask (younger than this
          // round's K / V loads, so the waits at the barriers leave it alone)
          issue_mask(t + 1);
          fold(mraw);
        }
      }
      const bool edge = (CAUSAL && kv0 + kBKV - 1 > qw0) || kv0 + kBKV > g.Skv;
      if (edge) {
        // (masked kernels use -inf: a row may see dead keys before its first
        // live one, and exp2(-inf - reference) is 0 whatever the reference)
        const float gone = MASK ? -INFINITY : kNegBig;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = kv0 + kb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            const bool dead = key >= g.Skv || (CAUSAL && key > qrow);
            s[kb][r] = dead ? gone : s[kb][r];
          }
      }
      // Exponentials of the tile's scores against reference point `ref` (raw
      // score units): the probabilities, rounded to the input type, go into
      // the fragments of the next MFMA phase; returns this lane's sum.  (Summing
      // the rounded pairs with v_dot2c_f32_bf16 measured slower than two adds.)
      auto exps = [&](float ref) __attribute__((always_inline)) {
        // (one fused multiply-add per score, spelled out: left to itself the
        // compiler scales every score first and fuses the reference instead)
        const float mc = -(ref * sl2);
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][r], sl2, mc));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][r + 1], sl2, mc));
            const uint32_t pk = sd_pack<BF16>(p0, p1);
            pf[kb * 2 + (r >> 3)][(r & 7) >> 1] = pk;
            psum += p0 + p1;
          }
        return psum;
      };
      // The reference point of the exponentials follows the row maximum
      // lazily.  Without a mask tensor a tile first runs against the reference
      // point it inherits, with no maximum taken at all: as long as no lane's
      // sum exceeds kRedoSum every probability is at most that, sums and
      // outputs stay far inside float range, and O = sum(p v) / sum(p) does not
      // depend on the reference point.  Only the first tile, and a tile in which
      // some row's scores rose that far above the reference, take the full
      // route: row maximum, a reference point that moves when the maximum has
      // risen by more than kMaxSlack (log2 units of the scaled scores), O^T
      // rescaled, the exponentials (again).  One copy of the code serves both:
      // the second trip of the loop is the full route.
      if constexpr (HD == 128) {
        bool full = FIRST || MASK != 0;
        float psum;
  #pragma clang loop unroll(disable)
        for (;;) {
          if (full) {
            // (the asm keeps the row maximum inside this branch: the compiler
            // would compute it on the common route as well)
            float mx = s[0][0];
            asm volatile("" : "+v"(mx));
  #pragma unroll
            for (int kb = 0; kb < 2; ++kb)
  #pragma unroll
              for (int r = 0; r < 16; ++r)
                mx = fmaxf(mx, s[kb][r]);
            mx = sd_half_max(mx);
            const bool moved = (mx - m_run) * sl2 > kMaxSlack;
            const float m_new = moved ? mx : m_run;
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * sl2);
            m_run = m_new;
            l_run *= alpha;
            // O^T holds tiles 0 .. t - 1 here (their MFMA phases are over).  In
            // place, as asm with tied operands: written as o *= alpha the
            // compiler gives the rescaled O^T registers of its own and copies
            // all 64 accumulators on the common route.  (The MFMAs that wrote
            // O^T lie a whole row maximum behind: no hazard.)
            if (__builtin_amdgcn_ballot_w64(moved) != 0) {
  #pragma unroll
              for (int dt = 0; dt < kD / 32; ++dt)
  #pragma unroll
                for (int r = 0; r < 16; ++r) {
                  float x = o[dt][r];
                  asm volatile("v_mul_f32 %0, %1, %0" : "+v"(x) : "v"(alpha));
                  o[dt][r] = x;
                }
            }
          }
          psum = exps(m_run);
          if (full || __builtin_amdgcn_ballot_w64(!(psum <= kRedoSum)) == 0)
            break;
          full = true;
        }
        l_run += psum;
      } else {
        // Head dim 64, where this phase is the longer one: the same steps as
        // two straight-line copies (fast route, then the full one if needed).
        // The compiler copies registers around whichever form it likes less:
        // all of O^T on the fast route of this form at head dim 128, the
        // scores in the loop form at head dim 64.
        bool full = true;
        if constexpr (MASK == 0 && !FIRST) {
          const float psum = exps(m_run);
          full = __builtin_amdgcn_ballot_w64(!(psum <= kRedoSum)) != 0;
          if (!full)
            l_run += psum;
        }
        if (full) {
          float mx = s[0][0];
          asm volatile("" : "+v"(mx)); // (keeps the maximum off the fast route)
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              mx = fmaxf(mx, s[kb][r]);
          mx = sd_half_max(mx);
          const bool moved = (mx - m_run) * sl2 > kMaxSlack;
          const float m_new = moved ? mx : m_run;
          const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * sl2);
          m_run = m_new;
          const float psum = exps(m_new);
          l_run = l_run * alpha + psum;
          if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
              for (int r = 0; r < 16; ++r)
                o[dt][r] *= alpha;
          }
        }
      }
    }
    // wavefronts 0..3 end their round here
    if (!team) {
      wait_all_but_round();
      sd_barrier();
    }
    sl_prev = sl_cur;
    sl_cur = sl_next;
    sl_next = next_slot(sl_next);
  };
  round(0, std::integral_constant<int, 0>{});
#pragma clang loop unroll(disable)
  for (int t = 1; t < tiles; ++t)
    round(t, std::integral_constant<int, 1>{});
  round(tiles, std::integral_constant<int, 2>{});
  if (!team) // pairs with the last barrier of wavefronts 4..7
    __builtin_amdgcn_s_barrier();

  // ---- epilogue: O = O^T / l, through LDS for row-contiguous stores -----------
  __builtin_amdgcn_s_waitcnt(sd_wait_imm(0));
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  const float inv = 1.0f / sd_half_sum(l_run);
  const uint32_t band = lds0 + (uint32_t)wave * (32 * kOutPitch);
  // lane holds query lq, features 32*dt + 8*(r/4) + 4*half + r%4
#pragma unroll
  for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      u32x2 w2;
      w2.x = sd_pack<BF16>(o[dt][r4 * 4 + 0] * inv, o[dt][r4 * 4 + 1] * inv);
      w2.y = sd_pack<BF16>(o[dt][r4 * 4 + 2] * inv, o[dt][r4 * 4 + 3] * inv);
      *(SD_AS3 u32x2 *)(uintptr_t)(band + lq * kOutPitch +
                                   (dt * 32 + r4 * 8 + half * 4) * 2) = w2;
    }
  char *op = g.o + (b * g.o_sb + h * g.o_sh) * 2;
  // kChunks lanes cover one output row; 4 or 8 rows per pass
#pragma unroll
  for (int rows = 0; rows < 32; rows += C::kRowsPerLoad) {
    const int row = rows + l / C::kChunks;
    const int cb = (l % C::kChunks) * 16;
    const u32x4 v =
        *(const SD_AS3 u32x4 *)(uintptr_t)(band + row * kOutPitch + cb);
    const int qr = qw0 + row;
    if (qr < g.Sq)
      *(SD_AS1 u32x4 *)(op + (int64_t)qr * g.o_ss * 2 + cb) = v;
  }
  } // pass
}

struct SdpaPlan {
  bool ok = false;
  bool bf16 = true;
  int hd = 128;
  bool mask = false;
  bool mask_rows16 = false;       // every mask row starts and ends on 16 bytes
  int64_t m_st[4] = {0, 0, 0, 0}; // mask strides over [B, Hq, Sq, Skv]
  uint32_t m_bytes = 0;
};

// A mask the kernel can read: rank 4, boolean / f32 / bf16 / f16, unit key
// stride, and every run of 4 keys a load fetches whole and aligned (extents
// and the other strides multiples of 4), one (batch, head) slab below 2 GiB.
bool plan_mask(const fhip_sdpa_desc *d, SdpaPlan &p) {
  const fhip_tensor_desc &m = d->mask;
  if (d->is_causal || m.rank != 4)
    return false;
  if (m.dtype != FHIP_BOOLEAN && m.dtype != FHIP_FLOAT &&
      m.dtype != FHIP_BFLOAT16 && m.dtype != FHIP_HALF)
    return false;
  const int64_t dims[4] = {d->q.dim[0], d->q.dim[1], d->q.dim[2], d->k.dim[2]};
  if (!fhip_broadcast_strides(m, 4, dims, p.m_st))
    return false;
  const int64_t Sq = dims[2], Skv = dims[3];
  if (p.m_st[3] != 1 || Skv % 4 != 0)
    return false;
  for (int i = 0; i < 3; ++i)
    if (p.m_st[i] < 0 || p.m_st[i] % 4 != 0)
      return false;
  const int64_t bytes =
      ((Sq - 1) * p.m_st[2] + Skv) * (int64_t)fhip_dtype_size(m.dtype);
  if (bytes >= (1ll << 31))
    return false;
  p.m_bytes = (uint32_t)bytes;
  p.mask = true;
  const int64_t es = (int64_t)fhip_dtype_size(m.dtype);
  p.mask_rows16 = Skv * es % 16 == 0;
  for (int i = 0; i < 3; ++i)
    p.mask_rows16 = p.mask_rows16 && p.m_st[i] * es % 16 == 0;
  return true;
}

SdpaPlan make_plan(const fhip_sdpa_desc *d) {
  SdpaPlan p;
  if (d->mask.rank != 0 && !plan_mask(d, p))
    return p;
  const int dt = d->q.dtype;
  if (dt != FHIP_BFLOAT16 && dt != FHIP_HALF)
    return p;
  if (d->k.dtype != dt || d->v.dtype != dt || d->o.dtype != dt)
    return p;
  p.bf16 = dt == FHIP_BFLOAT16;
  if (d->q.rank != 4 || (d->q.dim[3] != 64 && d->q.dim[3] != 128) ||
      d->k.dim[3] != d->q.dim[3] || d->v.dim[3] != d->q.dim[3])
    return p;
  p.hd = (int)d->q.dim[3];
  const fhip_tensor_desc *ts[4] = {&d->q, &d->k, &d->v, &d->o};
  for (const fhip_tensor_desc *t : ts) {
    if (t->stride[3] != 1 && t->dim[3] != 1)
      return p;
    for (int i = 0; i < 3; ++i)
      if (t->dim[i] > 1 && (t->stride[i] < 0 || (t->stride[i] * 2) % 16 != 0))
        return p;
  }
  const int64_t Sq = d->q.dim[2], Skv = d->k.dim[2];
  if (Sq < 1 || Skv < 1 || Sq >= (1ll << 30) || Skv >= (1ll << 30))
    return p;
  // 32-bit lane offsets inside one (batch, head) slab of K / V
  if (Skv * d->k.stride[2] * 2 >= (1ll << 31) ||
      Skv * d->v.stride[2] * 2 >= (1ll << 31))
    return p;
  // grid: heads x batch x query tiles
  if (d->q.dim[0] > 65535 || (Sq + kBQ - 1) / kBQ > 65535)
    return p;
  // the running maximum is taken over raw scores: needs a positive scale
  if (d->has_scale && !(d->scale > 0.f))
    return p;
  p.ok = true;
  return p;
}

} // namespace

bool fhip_fast_sdpa_applicable(const fhip_sdpa_desc *d) {
  return make_plan(d).ok;
}

int fhip_fast_sdpa(fhip_ctx *ctx, const fhip_sdpa_desc *d, const void *q,
                   const void *k, const void *v, const void *mask, void *o) {
  const SdpaPlan p = make_plan(d);
  FHIP_REQUIRE(ctx, p.ok, "sdpa: descriptor not supported by the MFMA kernel");
  FHIP_REQUIRE(ctx,
               (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) &
                15) == 0,
               "sdpa: Q, K, V, O must be 16-byte aligned");
  bool staged_mask = false;
  SdpaArgs g{};
  g.q = (const char *)q;
  g.k = (const char *)k;
  g.v = (const char *)v;
  g.o = (char *)o;
  auto st = [](const fhip_tensor_desc &t, int i) {
    return t.dim[i] > 1 ? t.stride[i] : 0;
  };
  g.q_sb = st(d->q, 0), g.q_sh = st(d->q, 1), g.q_ss = st(d->q, 2);
  g.k_sb = st(d->k, 0), g.k_sh = st(d->k, 1), g.k_ss = st(d->k, 2);
  g.v_sb = st(d->v, 0), g.v_sh = st(d->v, 1), g.v_ss = st(d->v, 2);
  g.o_sb = st(d->o, 0), g.o_sh = st(d->o, 1), g.o_ss = st(d->o, 2);
  g.Sq = (int32_t)d->q.dim[2];
  g.Skv = (int32_t)d->k.dim[2];
  g.group = (int32_t)(d->q.dim[1] / d->k.dim[1]);
  g.causal = d->is_causal;
  if (p.mask) {
    FHIP_REQUIRE(ctx, mask != nullptr, "sdpa: mask descriptor without a mask");
    FHIP_REQUIRE(ctx,
                 ((uintptr_t)mask & (4 * fhip_dtype_size(d->mask.dtype) - 1)) == 0,
                 "sdpa: the mask must be aligned to four of its elements");
    staged_mask = p.mask_rows16 && ((uintptr_t)mask & 15) == 0;
    g.mask = (const char *)mask;
    g.m_sb = p.m_st[0], g.m_sh = p.m_st[1], g.m_sq = p.m_st[2];
    g.m_bytes = p.m_bytes;
    g.m_dt = d->mask.dtype;
  }
  const float scale =
      d->has_scale ? d->scale : 1.0f / sqrtf((float)d->q.dim[3]);
  g.scale_log2e = scale * 1.4426950408889634f;
  g.scale = scale;
  const int n_qtiles = (g.Sq + kBQ - 1) / kBQ;
  const int64_t groups = d->is_causal ? (n_qtiles + 1) / 2 : n_qtiles;
  const int64_t heads = d->q.dim[1] * d->q.dim[0];
  dim3 grid((unsigned)d->q.dim[1], (unsigned)d->q.dim[0], (unsigned)groups);
  if (heads % 8 == 0 && groups > 1 && heads * groups < (1ll << 31) &&
      std::getenv("FUSILLI_HIP_SDPA_GRID") == nullptr) {
    g.xcd_heads = (int32_t)d->q.dim[1];
    g.xcd_groups = (int32_t)groups;
    grid = dim3((unsigned)(heads * groups));
  }
  auto launch = [&](auto kernel, int lds_bytes, FhipOncePerDevice &configured) {
    if (!configured.done(ctx->device)) {
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              lds_bytes) != hipSuccess)
        return fhip_fail(ctx, "sdpa: cannot reserve LDS");
      configured.mark(ctx->device);
    }
    hipLaunchKernelGGL(kernel, grid, dim3(kWaves * 64), lds_bytes, ctx->stream,
                       g);
    FHIP_HIP_CHECK(ctx, hipGetLastError());
    return 0;
  };
  // one flag per kernel instance: [head dim][type][plain / causal / mask in
  // registers / mask staged in LDS]
  static FhipOncePerDevice configured[2][2][4];
  fhip_note_kernel(ctx, "sdpa_fwd d=%d causal=%d mask=%d", p.hd, (int)(d->is_causal != 0),
                   p.mask ? (staged_mask ? 2 : 1) : 0);
  auto pick = [&](auto hd) {
    constexpr int HD = decltype(hd)::value;
    FhipOncePerDevice(&cfg)[2][4] = configured[HD == 128];
    constexpr int lds = SdShape<HD>::kLdsB;
    constexpr int lds_mask = SdShape<HD>::kLdsMaskB;
    if (p.mask && staged_mask)
      return p.bf16
                 ? launch(sdpa_fwd_kernel<true, false, HD, 2>, lds_mask, cfg[1][3])
                 : launch(sdpa_fwd_kernel<false, false, HD, 2>, lds_mask, cfg[0][3]);
    if (p.mask)
      return p.bf16 ? launch(sdpa_fwd_kernel<true, false, HD, 1>, lds, cfg[1][2])
                    : launch(sdpa_fwd_kernel<false, false, HD, 1>, lds, cfg[0][2]);
    if (p.bf16)
      return d->is_causal
                 ? launch(sdpa_fwd_kernel<true, true, HD, 0>, lds, cfg[1][1])
                 : launch(sdpa_fwd_kernel<true, false, HD, 0>, lds, cfg[1][0]);
    return d->is_causal
               ? launch(sdpa_fwd_kernel<false, true, HD, 0>, lds, cfg[0][1])
               : launch(sdpa_fwd_kernel<false, false, HD, 0>, lds, cfg[0][0]);
  };
  return p.hd == 128 ? pick(std::integral_constant<int, 128>{})
                     : pick(std::integral_constant<int, 64>{});
}

// C[M, N] = A[M, K] * W[N, K]^T in bfloat16 with float32 sums, for row counts between the
// weight-streaming kernel's (gemm_bf16_stream.hip, up to 16 with its fused epilogues) and those at
// which the library's product is near the matrix cores' rate: a decode step of a larger batch, a
// short prompt portion beside decoded tokens.  There the product is bound by reading W once, and A
// no longer fits a block's registers.
//
// Persistent blocks of eight wavefronts.  A block computes a tile of C: a block of 64 or 128 rows by
// up to TL_GROUPS groups of 16 columns (above 128 rows: sixteen wavefronts, 256 rows by up to
// TL_TALL_GROUPS groups), in steps of TL_BK = 64 along K.  The step's pieces of W
// [columns][64 k] and of A [rows][64 k] reach LDS by direct loads (global_load_lds_dwordx4: lane l
// of a wavefront fills bytes 16 l .. 16 l + 15 after a uniform address), two or three steps ahead
// into three or four buffers, so a step costs no registers, no LDS writes and one barrier.  A row
// of a piece is 128 bytes = 8 pieces of 16; piece p of row r lies at piece p ^ ((r / 2) % 8), which
// spreads the 16 rows of one matrix-core operand read over all banks.  The loads and their waits
// are inline assembly: the compiler would wait for every load in flight before each LDS read (and
// it does so as soon as the kernel holds any load into registers, which is why there is no bias).
//
//   v_mfma_f32_16x16x32_bf16:  C^T[n, m] += W[n, k] * A[m, k]
//     A operand = W tile (lane 16 j + r: row r, k = 32 s + 8 j .. + 7), B operand = A^T (same)
//     result lane 16 j + r holds C[r][n0 + 4 j + i], i = 0..3
//
// The work is the list of all (tile, step) pairs, tiles in order and each tile's steps in order;
// block b takes the pairs [b * chunk, (b + 1) * chunk), and its loads run ahead across tile
// boundaries, so a block starts its pipeline once.  Two cuts (tile_plan):
//   whole tiles: N is wide enough for every block to get the same number of tiles of 6 to 12
//     groups; the result is written once, in its own type, and the gated epilogue
//     silu(gate) * up (cwm/fastgen/forward.py:776-781) can be applied to it;
//   shared tiles: tiles of 8 groups, the pairs dealt out evenly whatever the tiles' ends; the
//     block that is the s-th to touch a tile writes its float32 partial sum into slab s,
//     C[s][M][N], and the block that ends a tile zeroes the slabs it leaves unused, so the consumer
//     adds `slabs` slabs whatever the cut (as it adds the streaming kernel's partial sums).
// Cut and order of every sum are fixed by N, K, the block height (64, 128 or 256 rows) and
// the number of blocks; within one block height a row's result does not depend on the other rows.
//
// Replaces torch.nn.functional.linear at cwm/fastgen/forward.py:593-606,763,776-782,820 for such
// batches.  Needs K % 64 == 0, N % 16 == 0 and 16-byte aligned rows.
#include "common.h"

CWM_DEFINE_ERROR_API

#define TL_GROUPS 12        // groups of 16 columns in the widest tile
#ifndef TL_SHARED_GROUPS
#define TL_SHARED_GROUPS 8  // in a tile whose steps several blocks share
#endif
#define TL_MIN_GROUPS 6     // narrower whole tiles would load more of A than of W
#define TL_BK 64
#define TL_ROTATE_STEPS 128   // steps of K up to which the tiles walk K from different starts
#define TL_MAX_ROWS 512

extern "C" int cwm_gemm_bf16_tile_max_rows() { return TL_MAX_ROWS; }

#ifndef TL_WAVES_64
#define TL_WAVES_64 8  // wavefronts of a block of 64 rows
#endif
#ifndef TL_WAVES_128
#define TL_WAVES_128 8  // and of a block of 128 rows
#endif
// More than 128 rows: blocks of 256 rows and 16 wavefronts, so that W is still read once; its tiles are at most
// TL_TALL_GROUPS wide (three buffers of 256 rows and 128 columns fill the LDS)
#define TL_TALL_ROWS 256
#define TL_TALL_WAVES 16
#define TL_TALL_GROUPS 8

// G: groups of 16 columns that a step's piece of W holds (the widest tile of the cut)
template <int BM, int WAVES, int G, typename TC, bool GLU>
__global__ void __launch_bounds__(WAVES * 64)
gemm_tile_kernel(const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, long ldw, TC* __restrict__ C, long ldc,
                 long slab_stride, int M, int N, int steps, int n_groups, int n_col_tiles, int n_row_blocks, long total,
                 int chunk, int slabs) {
  constexpr int W_BYTES = G * 16 * TL_BK * 2;
  constexpr int A_BYTES = BM * TL_BK * 2;
  constexpr int STAGE = W_BYTES + A_BYTES;
  constexpr int STAGES = 4 * STAGE < 160 * 1024 ? 4 : 3;
  constexpr int WN = 4;                  // wavefronts along the columns: wavefront wn takes the groups wn, wn + WN, ...
  constexpr int WM = WAVES / WN;         // and along the rows
  constexpr int NT = G / WN;             // groups of a wavefront
  constexpr int MT = BM / (16 * WM);     // its tiles of 16 rows
  constexpr int W_DMA = W_BYTES / 1024 / WAVES;  // loads of a wavefront per step: each fills 1 KB = 8 rows
  constexpr int A_DMA = A_BYTES / 1024 / WAVES;
  static_assert(G % WN == 0 && BM % (16 * WM) == 0 && W_BYTES % (1024 * WAVES) == 0 && A_BYTES % (1024 * WAVES) == 0, "block shape");
  static_assert(TL_SHARED_GROUPS <= TL_TALL_GROUPS && STAGES * STAGE <= 160 * 1024, "a block's buffers must fit the LDS");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * STAGE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const long first = (long)blockIdx.x * chunk;
  const int count = (int)min((long)chunk, total - first);
  if (count <= 0) return;

  // tile t: row block t % n_row_blocks of the column tile t / n_row_blocks, whose groups of 16
  // columns are [ct * n_groups / n_col_tiles, (ct + 1) * n_groups / n_col_tiles)
  auto first_group = [&](int ct) -> int { return (int)(((long)ct * n_groups) / n_col_tiles); };

  // ---- the loads: where the next step to be fetched lies
  int i_tile = (int)(first / steps);
  int i_step = (int)(first - (long)i_tile * steps);
  int i_left = count;
  const bf16_t* wsrc;
  const bf16_t* asrc;
  uint32_t w_off[W_DMA], a_off[A_DMA];
  int rotation = 0;
  // this lane's pieces of a step: load q fills rows 8 q .. 8 q + 7; rows past the tile or the matrix read its last row
  auto enter_tile = [&](int tile) {
    const int ct = tile / n_row_blocks;
    const int n0 = 16 * first_group(ct);
    const int n_last = min(16 * first_group(ct + 1), N) - 1;
    const int m0 = (tile - ct * n_row_blocks) * BM;
#pragma unroll
    for (int i = 0; i < W_DMA; ++i) {
      const int row = 8 * (wave * W_DMA + i) + (lane >> 3);
      const int piece = (lane & 7) ^ ((row >> 1) & 7);
      w_off[i] = (uint32_t)(((size_t)(min(n0 + row, n_last) - n0) * ldw + 8 * piece) * 2);
    }
#pragma unroll
    for (int i = 0; i < A_DMA; ++i) {
      const int row = 8 * (wave * A_DMA + i) + (lane >> 3);
      const int piece = (lane & 7) ^ ((row >> 1) & 7);
      a_off[i] = (uint32_t)(((size_t)(min(m0 + row, M - 1) - m0) * lda + 8 * piece) * 2);
    }
    wsrc = W + (size_t)n0 * ldw;
    asrc = A + (size_t)m0 * lda;
    // Blocks that are at the same step of their tiles ask the L2 for the same lines of A at the same time (blocks
    // that own whole tiles all start at step 0).  With a short K, where A stays in the L2, that costs more than it
    // saves (gate/up of the 32B shape at 64 rows: 106 against 96 us; an 8,192 x 8,192 product 38 against 28), so a
    // tile's step j reads K at (j + rotation) mod steps, with a rotation of the tile's own.  With a long K the W that
    // streams through the L2 pushes A out between its uses, and blocks in step fetch a line once for all of them
    // (down, K = 21,504: 51 against 54 us), so there is no rotation.  A sum's order is fixed by its tile and the cut.
    rotation = steps <= TL_ROTATE_STEPS ? __builtin_amdgcn_readfirstlane((int)(((unsigned)tile * 37u) % (unsigned)steps)) : 0;
  };
  enter_tile(i_tile);
  const uint32_t lds0 = (uint32_t)(uintptr_t)(&lds[0]);
  auto issue = [&](int buf) {
    int k_step = __builtin_amdgcn_readfirstlane(i_step + rotation);  // where along K this step reads (uniform)
    if (k_step >= steps) k_step -= steps;
    const bf16_t* ws = wsrc + (size_t)k_step * TL_BK;
    const bf16_t* as = asrc + (size_t)k_step * TL_BK;
    const uint32_t dst = lds0 + buf * STAGE;
#pragma unroll
    for (int i = 0; i < W_DMA; ++i) dma16_once(ws, w_off[i], dst + (wave * W_DMA + i) * 1024);  // W is read once, 8 rows of 128 bytes a load
#pragma unroll
    for (int i = 0; i < A_DMA; ++i) dma16(as, a_off[i], dst + W_BYTES + (wave * A_DMA + i) * 1024);
    if (i_left > 1) {  // past the block's last pair: that pair again, into a buffer nobody reads
      --i_left;
      if (++i_step == steps) {
        i_step = 0;
        enter_tile(++i_tile);
      }
    }
  };

  // ---- the products
  const int wm = wave / WN;
  const int wn = wave - wm * WN;
  const int r = lane & 15;
  const int j = lane >> 4;
  const int key = (r >> 1) & 7;  // the same for every row this lane reads: they differ by multiples of 16
  const int w_row = (wn * 16 + r) * 128;
  const int a_row = (wm * 16 * MT + r) * 128;
  float4v acc[NT][MT];
  int c_tile = (int)(first / steps);
  int c_step = (int)(first - (long)c_tile * steps);
  int buf = 0;  // the buffer that holds the next pair to be multiplied

#pragma unroll
  for (int t = 0; t < STAGES - 1; ++t) issue(t);
  for (int left = count; left > 0;) {
    // this block's steps of one tile; the loop over them holds no store, so that the only waits for
    // memory in it are the ones written here
    const int seg = min(steps - c_step, left);
    const int ct = c_tile / n_row_blocks;
    const int g0 = first_group(ct);
    const int width = first_group(ct + 1) - g0;  // groups of this tile
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (float4v){0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < seg; ++it) {
      // this wavefront's loads of the pair have landed (those of the pairs after it may be in flight);
      // after the barrier so have everyone's, and everyone has left the buffer that is filled next
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"((STAGES - 2) * (W_DMA + A_DMA)) : "memory");
      issue((buf + STAGES - 1) % STAGES);
      const unsigned char* wt = lds + buf * STAGE;
      const unsigned char* at = wt + W_BYTES;
#pragma unroll
      for (int s = 0; s < TL_BK / 32; ++s) {
        const int piece = ((4 * s + j) ^ key) * 16;
        Frag8 xf[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xf[mt].u = *(const uint4*)(at + a_row + mt * 2048 + piece);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          if (wn + WN * nt < width) {  // uniform over the wavefront
            Frag8 wf;
            wf.u = *(const uint4*)(wt + w_row + nt * WN * 2048 + piece);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf.v, xf[mt].v, acc[nt][mt], 0, 0, 0);
          }
        }
      }
      buf = (buf + 1) % STAGES;
    }
    left -= seg;
    c_step += seg;

    // the tile's sum over this block's steps: slab s, s counting the blocks that touch the tile
    const int slab = (int)(blockIdx.x - ((long)c_tile * steps) / chunk);
    const int m0 = (c_tile - ct * n_row_blocks) * BM;
    TC* out = C + (size_t)slab * slab_stride;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int g = wn + WN * nt;
      if (g >= width) continue;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + wm * 16 * MT + mt * 16 + r;
        const float4v v = acc[nt][mt];
        if constexpr (GLU) {
          // a group holds 8 gate columns, then the 8 up columns of the same 8 outputs: lanes with
          // j = 0, 1 hold the gates, the lanes 32 further on the ups of the same columns
          float4v up;
#pragma unroll
          for (int e = 0; e < 4; ++e) up[e] = __shfl_xor(v[e], 32, 64);
          if (j < 2 && m < M) {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float gr = bf16_to_f32(f32_to_bf16(v[e])), ur = bf16_to_f32(f32_to_bf16(up[e]));
              o[e] = gr / (1.0f + expf(-gr)) * ur;
            }
            *(uint2*)((bf16_t*)out + (size_t)m * ldc + 8 * (g0 + g) + 4 * j) = make_uint2(pack2_bf16(o[0], o[1]), pack2_bf16(o[2], o[3]));
          }
        } else {
          if (m >= M) continue;
          const int n = 16 * (g0 + g) + 4 * j;
          if constexpr (sizeof(TC) == 4) {
            *(float4*)((float*)out + (size_t)m * ldc + n) = make_float4(v[0], v[1], v[2], v[3]);
          } else {
            *(uint2*)((bf16_t*)out + (size_t)m * ldc + n) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
          }
        }
      }
    }
    if (c_step == steps) {
      // the tile is complete: the slabs after this one hold nothing of it
      if constexpr (sizeof(TC) == 4 && !GLU) {
        const int quads = 4 * width;  // float4 pieces in a row of the tile
        for (int s = slab + 1; s < slabs; ++s) {
          float* z = (float*)C + (size_t)s * slab_stride;
          for (int e = tid; e < BM * quads; e += WAVES * 64) {
            const int m = m0 + e / quads;
            const int n = 16 * g0 + 4 * (e % quads);
            if (m < M) *(float4*)(z + (size_t)m * ldc + n) = make_float4(0.f, 0.f, 0.f, 0.f);
          }
        }
      }
      c_step = 0;
      ++c_tile;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // the loads past the last pair
}

struct TilePlan {
  int block_rows, n_row_blocks, n_groups, n_col_tiles, steps, n_blocks, chunk, slabs;
  long total;
};

// most blocks that touch one tile when the pairs are cut every `chunk`
static int most_sharers(long tiles, long steps, long chunk) {
  long most = 1;
  for (long t = 0; t < tiles; ++t) {
    const long touched = (t * steps + steps - 1) / chunk - (t * steps) / chunk + 1;
    if (touched > most) most = touched;
  }
  return (int)most;
}

static TilePlan tile_plan(int M, int N, int K, int units) {
  TilePlan p;
  p.block_rows = M <= 64 ? 64 : M <= 128 ? 128 : TL_TALL_ROWS;
  const int widest_whole = p.block_rows == TL_TALL_ROWS ? TL_TALL_GROUPS : TL_GROUPS;
  p.n_row_blocks = (M + p.block_rows - 1) / p.block_rows;
  p.n_groups = N / 16;
  p.steps = K / TL_BK;
  // whole tiles: the fewest tiles, a multiple of the blocks, that are at most TL_GROUPS wide
  for (int per_block = 1; per_block <= 64; ++per_block) {
    const long tiles = (long)per_block * units;
    if (tiles % p.n_row_blocks) continue;
    const long col_tiles = tiles / p.n_row_blocks;
    if (col_tiles > p.n_groups) break;
    const long widest = (p.n_groups + col_tiles - 1) / col_tiles;
    if (widest > widest_whole) continue;
    if (p.n_groups / col_tiles < TL_MIN_GROUPS) break;
    p.n_col_tiles = (int)col_tiles;
    p.total = tiles * p.steps;
    p.n_blocks = units;
    p.chunk = per_block * p.steps;
    p.slabs = 1;
    return p;
  }
  // shared tiles
  p.n_col_tiles = (p.n_groups + TL_SHARED_GROUPS - 1) / TL_SHARED_GROUPS;
  const long tiles = (long)p.n_col_tiles * p.n_row_blocks;
  p.total = tiles * p.steps;
  long per = (p.total + units - 1) / units;
  if (per < 8) per = p.total < 8 ? p.total : 8;  // a block's start costs a few steps
  p.n_blocks = (int)((p.total + per - 1) / per);
  p.chunk = (int)per;
  p.slabs = most_sharers(tiles, p.steps, per);
  return p;
}

// The slabs of partial results that the product of these sizes leaves on `units` blocks (1: the
// result itself, in any type and with the gated epilogue if asked).
extern "C" int cwm_gemm_bf16_tile_slabs(int M, int N, int K, int units) {
  if (M <= 0 || N <= 0 || K <= 0 || K % TL_BK || N % 16 || units <= 0) return -1;
  return tile_plan(M, N, K, units).slabs;
}

// `slabs` must be what cwm_gemm_bf16_tile_slabs answers for the same sizes and units; C holds
// [slabs][M][ldc] float32 if it is more than 1 (slab_stride elements apart), else [M][ldc] of
// c_dtype.  glu: W holds gate and up rows in alternating groups of 8 and C [M, N / 2] receives
// silu(gate) * up in bfloat16; only where slabs is 1.
extern "C" int cwm_gemm_bf16_tile(const void* A, long lda, const void* W, long ldw, void* C, int c_dtype, long ldc,
                                  long slab_stride, int M, int N, int K, int units, int slabs, int glu, hipStream_t stream) {
  CWM_REQUIRE(M >= 0 && N > 0 && K > 0 && units > 0, "gemm_bf16_tile: bad sizes M=%d N=%d K=%d units=%d", M, N, K, units);
  CWM_REQUIRE(M <= TL_MAX_ROWS, "gemm_bf16_tile: M=%d is more than %d rows", M, TL_MAX_ROWS);
  CWM_REQUIRE(K % TL_BK == 0, "gemm_bf16_tile: K=%d must be a multiple of %d", K, TL_BK);
  CWM_REQUIRE(N % 16 == 0, "gemm_bf16_tile: N=%d must be a multiple of 16", N);
  CWM_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && ldc % 4 == 0, "gemm_bf16_tile: row strides must be multiples of 8 elements (C: 4)");
  CWM_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)C % 16) == 0,
              "gemm_bf16_tile: operands must be 16-byte aligned");
  CWM_REQUIRE(lda >= K && ldw >= K && ldc >= (glu ? N / 2 : N), "gemm_bf16_tile: row strides shorter than rows");
  CWM_REQUIRE(lda < (1L << 22) && ldw < (1L << 22), "gemm_bf16_tile: row strides too long for 32-bit offsets");
  CWM_REQUIRE(c_dtype == CWM_F32 || c_dtype == CWM_BF16, "gemm_bf16_tile: unknown output dtype %d", c_dtype);
  if (M == 0) return 0;
  const TilePlan p = tile_plan(M, N, K, units);
  CWM_REQUIRE(slabs == p.slabs, "gemm_bf16_tile: these sizes leave %d slabs of partial results, not %d", p.slabs, slabs);
  CWM_REQUIRE(slabs == 1 || c_dtype == CWM_F32, "gemm_bf16_tile: partial sums are float32");
  CWM_REQUIRE(!glu || (slabs == 1 && c_dtype == CWM_BF16), "gemm_bf16_tile: the gated epilogue needs whole tiles and a bfloat16 result");
  dim3 grid((unsigned)p.n_blocks);
#define CWM_LAUNCH_TILE(BM, WAVES, G, TC, GLU)                                                                           \
  hipLaunchKernelGGL((gemm_tile_kernel<BM, WAVES, G, TC, GLU>), grid, dim3(WAVES * 64), 0, stream, (const bf16_t*)A, lda, \
                     (const bf16_t*)W, ldw, (TC*)C, ldc, slab_stride, M, N, p.steps, p.n_groups, p.n_col_tiles,           \
                     p.n_row_blocks, p.total, p.chunk, p.slabs)
#define CWM_LAUNCH_ROWS(BM, WAVES, WHOLE)                       \
  do {                                                         \
    if (glu)                                                   \
      CWM_LAUNCH_TILE(BM, WAVES, WHOLE, bf16_t, true);         \
    else if (slabs > 1)                                        \
      CWM_LAUNCH_TILE(BM, WAVES, TL_SHARED_GROUPS, float, false); \
    else if (c_dtype == CWM_F32)                               \
      CWM_LAUNCH_TILE(BM, WAVES, WHOLE, float, false);         \
    else                                                       \
      CWM_LAUNCH_TILE(BM, WAVES, WHOLE, bf16_t, false);        \
  } while (0)
  if (p.block_rows == 64)
    CWM_LAUNCH_ROWS(64, TL_WAVES_64, TL_GROUPS);
  else if (p.block_rows == 128)
    CWM_LAUNCH_ROWS(128, TL_WAVES_128, TL_GROUPS);
  else
    CWM_LAUNCH_ROWS(TL_TALL_ROWS, TL_TALL_WAVES, TL_TALL_GROUPS);
#undef CWM_LAUNCH_ROWS
#undef CWM_LAUNCH_TILE
  return cwm_launch_status("gemm_bf16_tile");
}

// out[M, N] = x[M, K] * W[N, K]^T for few rows (decode steps, the logits of a
// few positions): bf16 inputs, 32-bit accumulation on the matrix cores, bf16 or
// 32-bit output.  The time of such a product is the time to read W once, so the
// kernel is laid out around that read:
//
//   * a wave owns 16 rows of W; W is the A operand of MFMA 16x16x32 (16 rows x
//     32 k) and is read straight from memory in operand order, several steps
//     ahead of the products that use them.  From a matrix stored row by row a
//     load instruction takes 64 contiguous bytes of each of 16 rows.  A matrix
//     stored in tiles (rv_tile_weight: the 16 x 32 values of one product
//     contiguous in the order the lanes hold them, a wave's tiles one after
//     the other along K) is read as one contiguous stream per wave, 1 KB an
//     instruction: the memory then sees long runs instead of 64-byte pieces
//     5 KB apart, and a product takes a tenth to a quarter less time;
//   * the waves of a block own neighbouring rows and the same range of K, so
//     they share x: the block stages x through LDS in pieces of 512 columns
//     (double-buffered, rows padded against bank conflicts; beyond 32 rows of
//     x in pieces of 256; beyond 16 rows brought in by waves of their own into
//     three buffers)
//     and every wave reads its B operands from there; up to four column sets
//     of 16 rows of x share each read of W;
//   * a matrix with few rows is also split along K over blocks (grid.y) so
//     that every CU has work; each slice writes 32-bit partial sums and a
//     second kernel adds the slices in a fixed order.  A row of x therefore
//     gives the same bits whatever else is in the batch.
//
// The reference hands these products to cuBLASLt, with its own kernels for the
// one-row case (v3/crates/rvllm-cutlass/src/cublaslt.rs:184-277, kernels/fp8_gemv.cu);
// this is the bf16 counterpart of the latter for up to 64 rows.
#include <math.h>
#include <stdlib.h>

#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 sk_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float sk_f32x4;

union SkFrag {
  sk_bf16x8 v;
  uint4 u4;
};

// A wave keeps SK_DEPTH steps of 128 columns of W in flight (a ring of
// fragment sets in registers): with a memory latency of a few microseconds and
// a step worth 4 KB a wave, that is what it takes for some 1024 waves to draw
// the full bandwidth, and it lets a short slice issue all of its loads at once.
// x is staged a chunk of SK_CHUNK_STEPS steps at a time, two buffers.  Up to 32
// rows of x a chunk is the whole ring (512 columns); for more rows it is half
// the ring (256 columns), so that the buffers stay at 67 KB and two blocks fit
// a CU, and the loop is written out for two chunks so that every place of the
// ring is still named at compile time.  Rows of the staged x are padded by 8
// elements: the row stride is then 4 banks off a multiple of 64 banks, and the
// 16 lanes that read the same columns of 16 rows hit 64 different banks.
#define SK_DEPTH 4
#define SK_CHUNK_STEPS_OF(MT) ((MT) <= 2 ? 4 : 2)
#define SK_MAX_WAVES 8

template <typename TC>
__device__ __forceinline__ void sk_store1(TC* p, float a);
template <>
__device__ __forceinline__ void sk_store1<float>(float* p, float a) {
  p[0] = a;
}
template <>
__device__ __forceinline__ void sk_store1<uint16_t>(uint16_t* p, float a) {
  p[0] = rv_f32_to_bf16_bits(a);
}

// grid (row blocks, K slices); block = waves x 64.  With one slice the result
// goes to `out` as TC; with more, slice s writes 32-bit sums to part[s][M][N].
// ACT 0 or 1: W holds the rows of a gate and an up projection in fours, two
// gates and then their two ups; a lane's four sums are then two gates and
// their ups, and what an unsliced product stores is act(gate) * up, N / 2
// values a row (the sums rounded to bf16 first, exactly as the separate kernel
// for it would read them): a kernel and a pass over memory less, at no cost.
// A sliced product stores its partial sums as for ACT < 0.
// TILED: W is stored in tiles (see rv_tile_weight); ldw is then unused.
// A copy of 16 bytes a lane from memory straight into LDS: lane l's land at `to` + 16 l (`to` the same in all
// lanes).  Written as an instruction of its own, so the compiler knows of no read from memory and of no write
// to LDS: the wave that issues these issues no other reads from memory and counts them itself (sk_wait_copies).
__device__ __forceinline__ void sk_copy16_to_lds(const void* from, const uint16_t* to) {
  const uint32_t at = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint16_t*)to;
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(at) : "memory", "m0");
}
// Waits until at most N of this wave's reads from memory are on their way (they arrive in the order of asking).
template <int N>
__device__ __forceinline__ void sk_wait_copies() {
  static_assert(N >= 0 && N < 64, "the counter has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));  // vmcnt(N), nothing else
  asm volatile("" ::: "memory");
}
__device__ const uint4 sk_zeros16 = {0u, 0u, 0u, 0u};  // what a copy reads where x has nothing

// Beyond 16 rows of x a block has three waves more, which own no rows of W and only bring x in (SK_BRINGERS_OF):
// x is then half as many bytes as W or as many, and a wave that asks for both waits for its x behind the W it asked for earlier
// (reads come back in the order of asking) and, with the barrier that follows, for the W of the whole next chunk
// and of every wave of the block, which takes off the ring's depth; staging x also takes a quarter of such a
// product's time in loads, masks and stores.  The waves that bring x in ask for nothing else, copy straight from
// memory into LDS, a chunk ahead, and count their copies themselves; the others wait for W alone.  One such wave
// cannot keep up with four that multiply, two nearly; with four the widest products have too few blocks.
#define SK_BRINGERS_OF(MT) ((MT) >= 2 ? 3 : 0)
template <int MT, typename TC, int ACT = -1, bool TILED = false>
__global__ void __launch_bounds__(SK_MAX_WAVES * 64)
gemm_skinny_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, TC* __restrict__ out,
                   float* __restrict__ part, int M, int N, int K, long long ldx, long long ldw, long long ldc,
                   int slice_len) {
  constexpr int DEPTH = SK_DEPTH;
  constexpr int CH = SK_CHUNK_STEPS_OF(MT);  // steps of 128 columns in a chunk of x
  constexpr int UNROLL = DEPTH / CH;         // chunks a pass of the main loop takes
  constexpr int SK_KC = CH * 128;
  constexpr int SK_ROW = SK_KC + 8;
  // With waves that only bring x in, three buffers take turns: a chunk's x is on its way into one while the
  // chunk before it is multiplied from another and the third still holds the one before that.  A copy fills
  // 64 pieces of 16 bytes at a time, so a buffer has room behind its last row for the last copy's overhang.
  constexpr int BUFS = SK_BRINGERS_OF(MT) > 0 ? 3 : 2;
  constexpr int ROWS_ROOM = SK_BRINGERS_OF(MT) > 0 ? MT * 16 + 2 : MT * 16;
  __shared__ __attribute__((aligned(16))) uint16_t xs[BUFS][ROWS_ROOM][SK_ROW];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in all lanes, and known to be
  constexpr int BRINGERS = SK_BRINGERS_OF(MT);
  const int waves = (int)(blockDim.x >> 6) - BRINGERS;  // the waves that own rows of W
  const bool brings_x = BRINGERS > 0 && wave >= waves;
  const int r16 = lane & 15;
  const int kb = lane >> 4;
  const int n0 = (blockIdx.x * waves + (brings_x ? 0 : wave)) * 16;
  const bool wave_has_rows = n0 < N;
  const int row = n0 + r16 < N ? n0 + r16 : N - 1;
  const int kbeg = blockIdx.y * slice_len;
  const int kend = kbeg + slice_len < K ? kbeg + slice_len : K;
  const int chunks = (kend - kbeg + SK_KC - 1) / SK_KC;

  // Every read from memory below is unconditional, from an address clamped
  // into the operand: a read under a branch makes the compiler wait for all
  // earlier reads before the next product, which would undo the ring.  What a
  // clamped read brings in is thrown away (x) or meets zeros of x (W).

  // staging: the block copies x[0 : MT*16, chunk] into LDS, 16 bytes a thread and turn
  constexpr int PIECES = MT * 16 * (SK_KC / 8);  // 16-byte pieces in a chunk
  // a thread holds at most PIECES / 256 pieces (blocks have at least 4 waves)
  constexpr int MAX_REGS = BRINGERS > 0 ? 1 : (PIECES + 255) / 256;
  const int stagers = (int)blockDim.x;  // threads that stage x
  const int sid = tid;
  // One set of registers per chunk of a pass: a set that is loaded at two places of the loop gets copied by the
  // compiler right after the second load, and the copy waits for every read asked for before it, the ring's too.
  uint4 staged_sets[UNROLL][MAX_REGS];
  const int last_k = kend - 8;  // the last 16-byte piece of this slice (slices are multiples of 8 long)
  auto stage_load = [&](int c, uint4 (&staged)[MAX_REGS]) {
#pragma unroll
    for (int n = 0; n < MAX_REGS; ++n) {
      int p = sid + n * stagers;
      p = p < PIECES ? p : PIECES - 1;
      int m = p / (SK_KC / 8);
      int k = kbeg + c * SK_KC + (p % (SK_KC / 8)) * 8;
      m = m < M ? m : M - 1;
      k = k < last_k ? k : last_k;
      staged[n] = *(const uint4*)(x + (size_t)m * ldx + k);
    }
  };
  auto stage_store = [&](int c, int buf, uint4 (&staged)[MAX_REGS]) {
#pragma unroll
    for (int n = 0; n < MAX_REGS; ++n) {
      int p = sid + n * stagers;
      p = p < PIECES ? p : PIECES - 1;  // threads past the end repeat the last piece: the same bytes to the same place
      const int m = p / (SK_KC / 8);
      const int col = (p % (SK_KC / 8)) * 8;
      // Columns past the slice's end become zeros, by a mask and not by a choice
      // (a choice would let the compiler put the read under a branch again).
      // Rows past M repeat row M - 1; their sums are never stored.
      const unsigned keep = 0u - (unsigned)(kbeg + c * SK_KC + col < kend);
      uint4 v = staged[n];
      // The staged values count as used only from here on: otherwise the masking
      // drifts up between the products, and its wait for x drains the ring.
      asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
      v.x &= keep, v.y &= keep, v.z &= keep, v.w &= keep;
      *(uint4*)(&xs[buf][m][col]) = v;
    }
  };

  sk_f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (sk_f32x4){0.f, 0.f, 0.f, 0.f};
  const uint16_t* wrow = w + (size_t)row * ldw + kbeg;
  const int last_off = kend - 8 - kbeg;
  // tiled: this lane's 16 bytes of the wave's tile at K step 0 (a wave past the last rows reads the last tile),
  // and the steps of 32 a row of tiles has
  const int k32 = (K + 31) >> 5;
  const uint16_t* wtile = w + ((size_t)(wave_has_rows ? n0 >> 4 : (N - 1) >> 4) * k32 << 9) + lane * 8;
  const int step0 = kbeg >> 5;  // slices begin at multiples of 128

  SkFrag ring[DEPTH][4];
  auto load_w = [&](int koff, SkFrag* a) {  // koff: offset inside the slice of the 128 columns to read
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (TILED) {
        const int ks = step0 + (koff >> 5) + j;
        a[j].u4 = *(const uint4*)(wtile + ((size_t)(ks < k32 ? ks : k32 - 1) << 9));
      } else {
        const int off = koff + j * 32 + kb * 8;
        a[j].u4 = *(const uint4*)(wrow + (off < last_off ? off : last_off));
      }
    }
  };
  if constexpr (BRINGERS > 0) {
    if (brings_x) {
      // A buffer is rows of SK_ROW / 8 pieces of 16 bytes, the last of them padding; a copy fills 64 pieces in a
      // row, wherever rows begin and end, and each lane reads the piece of x that belongs where its 16 bytes
      // land: row min(m, M - 1), or zeros for the padding, for columns past the slice's end and behind the last row.
      constexpr int ROW_PIECES = SK_ROW / 8;
      constexpr int COPIES = (MT * 16 * ROW_PIECES + 63) / 64;        // copy instructions a chunk
      constexpr int MY_COPIES = (COPIES + BRINGERS - 1) / BRINGERS;  // of one bringing wave
      const int me = wave - waves;
      auto bring = [&](int c, int buf) {
#pragma unroll
        for (int n = 0; n < MY_COPIES; ++n) {
          int i = me + n * BRINGERS;
          i = i < COPIES ? i : COPIES - 1;  // the last one once more: the same bytes to the same place
          const int q = i * 64 + lane;
          const int m = q / ROW_PIECES;
          const int cp = q - m * ROW_PIECES;
          const int k = kbeg + c * SK_KC + cp * 8;
          const bool there = cp < SK_KC / 8 && k < kend && m < MT * 16;
          const int mm = m < M ? m : M - 1;
          const uint16_t* src = x + (size_t)mm * ldx + (k < last_k ? k : last_k);
          sk_copy16_to_lds(there ? (const void*)src : (const void*)&sk_zeros16, &xs[buf][0][0] + i * 512);
        }
      };
      // As many barriers as the waves that multiply: one after the first chunk, one after every chunk of the loop
      // (which takes its chunks UNROLL at a time, a chunk past the slice's end included).  While chunk cc is
      // multiplied, chunk cc + 1 arrives and chunk cc + 2 is asked for.
      bring(0, 0);
      bring(1, 1);
      sk_wait_copies<MY_COPIES>();  // chunk 0 is there
      __syncthreads();
      const int rounds = (chunks + UNROLL - 1) / UNROLL * UNROLL;
      int into = 2;
      for (int cc = 0; cc < rounds; ++cc) {
        bring(cc + 2, into);  // that buffer was last read in chunk cc - 1
        into = into == 2 ? 0 : into + 1;
        sk_wait_copies<MY_COPIES>();  // chunk cc + 1 is there
        __syncthreads();
      }
      sk_wait_copies<0>();  // nothing lands in LDS after the block has given it back
      return;
    }
  }
  // The first chunk of x and the whole ring are requested together.  The order
  // (x, then the ring's places in turn) is the one every pass of the loop below
  // leaves behind, so the compiler's count of reads in flight is exact there.
  if constexpr (BRINGERS == 0) stage_load(0, staged_sets[0]);
  asm volatile("" ::: "memory");
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    load_w(d * 128, ring[d]);
    asm volatile("" ::: "memory");
  }
  if constexpr (BRINGERS == 0) stage_store(0, 0, staged_sets[0]);
  __syncthreads();

  int turn = 0;  // with three buffers: the one the next chunk lies in
  int c = 0;
  do {  // a slice has at least one chunk; a loop that may run zero times lets the first reads sink below the barrier
    // the x of the chunks after this pass's: asked for here, all of it, before the ring's reads, so that waiting
    // for it leaves those in flight; in flight while this pass's chunks are multiplied
    if constexpr (BRINGERS == 0) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) stage_load(c + u + 1, staged_sets[u]);
    }
    asm volatile("" ::: "memory");
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      // chunk c + u: its x lies in buffer `buf`, its W in the ring's places u * CH .. u * CH + CH - 1.  A chunk
      // past the slice's end (an odd number of chunks, two a pass) meets zeros of x.
      const int cc = c + u;
      const int buf = BUFS == 3 ? turn : (UNROLL == 1 ? (c & 1) : (u & 1));
      turn = turn == 2 ? 0 : turn + 1;
#pragma unroll
      for (int st = 0; st < CH; ++st) {
        const int d = u * CH + st;
        // The operands from x of several products are asked for before the first of them: a read from LDS takes
        // some hundred cycles, and one or two in flight make sixteen of them a step longer than the step's share
        // of the memory's time.  A whole step's at once up to 32 rows of x; beyond, half a step's (registers).
        constexpr int JG = MT <= 2 ? 4 : 2;  // 128-column quarters whose operands are in flight together
#pragma unroll
        for (int j0 = 0; j0 < 4; j0 += JG) {
          SkFrag b[JG][MT];
#pragma unroll
          for (int j = 0; j < JG; ++j) {
            const int col = st * 128 + (j0 + j) * 32 + kb * 8;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) b[j][mt].u4 = *(const uint4*)(&xs[buf][mt * 16 + r16][col]);
          }
          __builtin_amdgcn_sched_barrier(0);  // or the compiler puts each read back before its product
#pragma unroll
          for (int j = 0; j < JG; ++j) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[d][j0 + j].v, b[j][mt].v, acc[mt], 0, 0, 0);
          }
        }
        load_w((cc + UNROLL) * SK_KC + st * 128, ring[d]);  // the same place of the ring, a ring's length on
        asm volatile("" ::: "memory");                     // here, and not gathered at the chunk's end
      }
      // that buffer was last read in chunk cc - 1, before the barrier below
      if constexpr (BRINGERS == 0) stage_store(cc + 1, buf ^ 1, staged_sets[u]);
      __syncthreads();
    }
    c += UNROLL;
  } while (c < chunks);

  if (!wave_has_rows) return;
  // a lane holds the sums for x row m = mt*16 + r16 and W rows n0 + kb*4 .. + 3
  const int nb = n0 + kb * 4;
  const bool sliced = gridDim.y > 1;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r16;
    if (m >= M) continue;
    if (sliced) {
      float* o = part + ((size_t)blockIdx.y * M + m) * N + nb;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (nb + i < N) o[i] = acc[mt][i];
    } else if constexpr (ACT >= 0) {
      if (nb < N) {  // N is a multiple of 4
        auto as_stored = [](float v) { return __uint_as_float((uint32_t)rv_f32_to_bf16_bits(v) << 16); };
        TC* o = out + (size_t)m * ldc + nb / 2;
        sk_store1<TC>(o, rv_gated<bf16_t, ACT>(as_stored(acc[mt][0]), as_stored(acc[mt][2])));
        sk_store1<TC>(o + 1, rv_gated<bf16_t, ACT>(as_stored(acc[mt][1]), as_stored(acc[mt][3])));
      }
    } else {
      TC* o = out + (size_t)m * ldc + nb;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (nb + i < N) sk_store1<TC>(o + i, acc[mt][i]);
    }
  }
}

// out[m][n] = sum over slices of part[s][m][n], slices in order.
template <typename TC>
__global__ void sk_reduce_kernel(const float* __restrict__ part, TC* __restrict__ out, int slices, int M, int N,
                                 long long ldc) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)M * N) return;
  const int m = (int)(idx / N);
  const int n = (int)(idx - (long long)m * N);
  float s = 0.f;
  for (int i = 0; i < slices; ++i) s += part[(size_t)i * M * N + idx];
  sk_store1<TC>(out + (size_t)m * ldc + n, s);
}

// The plan for a shape: waves a block, K slices, columns a slice (a multiple of
// 128).  The chip runs all blocks at once, a few per CU, so the time is set by
// the CU with the most blocks: the plan looks for a number of blocks that
// fills the CUs evenly (close below a multiple of their number), with about
// 2048 waves in all and slices that are not too short.
#define SK_NUM_CUS 256
// For measurements: a plan that replaces the model's for every shape (0, 0 = the model's again).
static int sk_forced_waves = 0, sk_forced_units = 0;
extern "C" void rv_gemm_skinny_force_plan(int waves, int units_per_slice) {
  sk_forced_waves = waves >= 4 && waves <= SK_MAX_WAVES ? waves : 0;
  sk_forced_units = units_per_slice > 0 ? units_per_slice : 0;
}

extern "C" void rv_gemm_skinny_plan(int N, int K, int* waves, int* slices, int* slice_len) {
  const int tiles = rv_div_up(N, 16);
  const int units = rv_div_up(K, 128);
  if (sk_forced_waves && sk_forced_units) {
    const int per = sk_forced_units < units ? sk_forced_units : units;
    *waves = sk_forced_waves;
    *slice_len = per * 128;
    *slices = rv_div_up(units, per);
    return;
  }
  // The constants are fitted to the measured times of every plan for the twelve products of the 4B-, 12B- and
  // 27B-sized layers at 8 rows (matrices in tiles): the chosen plans lie 2 % above the best ones on average.
  double best_time = 1e300;
  int best_w = 4, best_len = units * 128, best_s = 1;
  const double w_bytes = 2.0 * N * K;
  for (int wv = 4; wv <= SK_MAX_WAVES; ++wv) {
    const int row_blocks = rv_div_up(tiles, wv);
    for (int s = 1; s <= units && s <= 64; ++s) {
      const int per = rv_div_up(units, s);        // 128-column units a slice, the slices as even as they come
      if (rv_div_up(units, per) != s) continue;   // the same plan as with fewer slices
      // a model of the time, in bytes moved at full speed
      const double part_bytes = s > 1 ? 64.0 * s * 16.0 * N : 0.0;  // what partial sums cost, written and read again
      const long long blocks = (long long)row_blocks * s;
      const long long rounds = (blocks + SK_NUM_CUS - 1) / SK_NUM_CUS;
      const double fill = pow((double)blocks / (double)(rounds * SK_NUM_CUS), 0.25);  // evenness over the CUs
      const double total_waves = (double)blocks * wv;
      const double in_flight = total_waves >= 768.0 ? 1.0 : total_waves / 768.0;  // enough loads in flight
      const double rows_used = (double)tiles / (double)(row_blocks * wv);          // waves without rows
      const double startup = (per + 1.0) / per;  // a wave's start costs about one step
      const double time = (w_bytes + part_bytes) / (fill * in_flight * rows_used) * startup;
      if (time < best_time * (1.0 - 1e-9)) {
        best_time = time;
        best_w = wv;
        best_len = per * 128;
        best_s = s;
      }
    }
  }
  *waves = best_w;
  *slice_len = best_len;
  *slices = best_s;
}

// Floats of workspace that rv_gemm_skinny needs for this shape (0 when unsliced).
extern "C" long long rv_gemm_skinny_workspace(int M, int N, int K) {
  int waves, slices, len;
  rv_gemm_skinny_plan(N, K, &waves, &slices, &len);
  return slices > 1 ? (long long)slices * M * N : 0;
}

// Number of K slices of this shape (1 = unsliced).
extern "C" int rv_gemm_skinny_slices(int N, int K) {
  int waves, slices, len;
  rv_gemm_skinny_plan(N, K, &waves, &slices, &len);
  return slices;
}

template <int MT, typename TC, int ACT = -1>
static int sk_launch(hipStream_t stream, const uint16_t* x, const uint16_t* w, TC* out, float* part, int M, int N,
                     int K, long long ldx, long long ldw, long long ldc, int do_reduce, int tiled) {
  int waves, slices, len;
  rv_gemm_skinny_plan(N, K, &waves, &slices, &len);
  if (slices > 1 && part == nullptr) return rv_fail("gemm_skinny: this shape needs a workspace");
  // a block holds SK_MAX_WAVES waves at most (two per SIMD, for their registers), the one that brings x in included
  if (waves + SK_BRINGERS_OF(MT) > SK_MAX_WAVES) waves = SK_MAX_WAVES - SK_BRINGERS_OF(MT);
  dim3 grid(rv_div_up(rv_div_up(N, 16), waves), slices);
  const dim3 block((waves + SK_BRINGERS_OF(MT)) * 64);  // the waves that own rows of W, and those that only bring x in
  if (tiled)
    gemm_skinny_kernel<MT, TC, ACT, true><<<grid, block, 0, stream>>>(x, w, out, part, M, N, K, ldx, ldw, ldc, len);
  else
    gemm_skinny_kernel<MT, TC, ACT, false><<<grid, block, 0, stream>>>(x, w, out, part, M, N, K, ldx, ldw, ldc, len);
  RV_LAUNCH_CHECK("gemm_skinny");
  if (slices > 1 && do_reduce) {
    const long long total = (long long)M * N;
    sk_reduce_kernel<TC><<<dim3(rv_div_up(total, 256)), dim3(256), 0, stream>>>(part, out, slices, M, N, ldc);
    RV_LAUNCH_CHECK("gemm_skinny_reduce");
  }
  return 0;
}

// With `do_reduce` 0 a sliced product leaves its 32-bit partial sums in `part`
// ([slices][M][N]) for a consumer that adds them itself, and `out` is not
// written; an unsliced product always writes `out`.
// `tiled` != 0: W is what rv_tile_weight made of the [N, K] matrix, and ldw is not used.
extern "C" int rv_gemm_skinny(hipStream_t stream, const void* x, const void* w, void* out, int out_dtype, float* part,
                              int M, int N, int K, long long ldx, long long ldw, long long ldc, int do_reduce,
                              int tiled) {
  RV_CHECK(M >= 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: M=%d must be at most 64 (N=%d K=%d)", M, N, K);
  RV_CHECK(K % 8 == 0 && ldx % 8 == 0 && (tiled || ldw % 8 == 0),
           "gemm_skinny: K and the row strides must be multiples of 8");
  RV_CHECK(ldx >= K && (tiled || ldw >= K) && ldc >= N, "gemm_skinny: leading dimensions too small");
  RV_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_skinny: operands must be 16-byte aligned");
  if (M == 0) return 0;
  const int mt = rv_div_up(M, 16);
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)w;
#define SK_CASE(MTV)                                                                                  \
  case MTV:                                                                                           \
    if (out_dtype == RV_F32)                                                                          \
      return sk_launch<MTV, float>(stream, xp, wp, (float*)out, part, M, N, K, ldx, ldw, ldc, do_reduce, tiled);        \
    if (out_dtype == RV_BF16)                                                                         \
      return sk_launch<MTV, uint16_t>(stream, xp, wp, (uint16_t*)out, part, M, N, K, ldx, ldw, ldc, do_reduce, tiled);  \
    break;
  switch (mt) {
    SK_CASE(1)
    SK_CASE(2)
    SK_CASE(3)
    SK_CASE(4)
  }
#undef SK_CASE
  return rv_fail("gemm_skinny: unsupported output dtype %d", out_dtype);
}

// act(x W_gate^T) * (x W_up^T) in one kernel: W [N, K] holds the rows of the two projections in fours (gates
// 2q, 2q + 1, then ups 2q, 2q + 1), `out` is [M, N / 2].  Only for shapes whose plan has one slice
// (rv_gemm_skinny_slices); act 0: gelu in its tanh form, 1: silu.  Otherwise as rv_gemm_skinny.
extern "C" int rv_gemm_skinny_gate_up(hipStream_t stream, const void* x, const void* w, void* out, int out_dtype,
                                      int M, int N, int K, long long ldx, long long ldw, long long ldc, int act,
                                      int tiled) {
  RV_CHECK(M >= 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny_gate_up: M=%d must be at most 64 (N=%d K=%d)", M, N, K);
  RV_CHECK(N % 4 == 0, "gemm_skinny_gate_up: N=%d must be a multiple of 4 (two gates, two ups)", N);
  RV_CHECK(K % 8 == 0 && ldx % 8 == 0 && (tiled || ldw % 8 == 0),
           "gemm_skinny_gate_up: K and the row strides must be multiples of 8");
  RV_CHECK(ldx >= K && (tiled || ldw >= K) && ldc >= N / 2, "gemm_skinny_gate_up: leading dimensions too small");
  RV_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_skinny_gate_up: operands must be 16-byte aligned");
  RV_CHECK(act == 0 || act == 1, "gemm_skinny_gate_up: unknown activation %d", act);
  RV_CHECK(rv_gemm_skinny_slices(N, K) == 1, "gemm_skinny_gate_up: the plan for N=%d K=%d has slices", N, K);
  if (M == 0) return 0;
  const int mt = rv_div_up(M, 16);
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)w;
#define SK_CASE(MTV)                                                                                                \
  case MTV:                                                                                                         \
    if (out_dtype == RV_F32)                                                                                        \
      return act == 0 ? sk_launch<MTV, float, 0>(stream, xp, wp, (float*)out, nullptr, M, N, K, ldx, ldw, ldc, 1, tiled)   \
                      : sk_launch<MTV, float, 1>(stream, xp, wp, (float*)out, nullptr, M, N, K, ldx, ldw, ldc, 1, tiled);  \
    if (out_dtype == RV_BF16)                                                                                       \
      return act == 0                                                                                               \
                 ? sk_launch<MTV, uint16_t, 0>(stream, xp, wp, (uint16_t*)out, nullptr, M, N, K, ldx, ldw, ldc, 1, tiled)  \
                 : sk_launch<MTV, uint16_t, 1>(stream, xp, wp, (uint16_t*)out, nullptr, M, N, K, ldx, ldw, ldc, 1, tiled); \
    break;
  switch (mt) {
    SK_CASE(1)
    SK_CASE(2)
    SK_CASE(3)
    SK_CASE(4)
  }
#undef SK_CASE
  return rv_fail("gemm_skinny_gate_up: unsupported output dtype %d", out_dtype);
}

// W [N, K] (row stride ldw) into tiles: tile (n / 16, k / 32) holds 16 rows x 32 columns as the 64 lanes of a
// product's A operand hold them, lane (k % 32 / 8) * 16 + n % 16 eight consecutive columns, 1 KB a tile, a row of
// tiles (all of K) contiguous.  Rows past N and columns past K are zeros.  `out` has
// ceil(N / 16) * ceil(K / 32) * 512 elements.
__global__ void sk_tile_weight_kernel(const uint16_t* __restrict__ w, uint16_t* __restrict__ out, int N, int K,
                                      long long ldw, int k32, long long pieces) {
  const long long p = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // one 16-byte piece of the output
  if (p >= pieces) return;
  const int lane = (int)(p & 63);
  const long long tile = p >> 6;
  const int ks = (int)(tile % k32);
  const long long nt = tile / k32;
  const long long n = nt * 16 + (lane & 15);
  const int k0 = ks * 32 + (lane >> 4) * 8;
  uint16_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (n < N && k0 + i < K) ? w[n * ldw + k0 + i] : (uint16_t)0;
  *(uint4*)(out + p * 8) = *(const uint4*)v;
}

extern "C" long long rv_tile_weight_elements(int N, int K) {
  return (long long)rv_div_up(N, 16) * rv_div_up(K, 32) * 512;
}

extern "C" int rv_tile_weight(hipStream_t stream, const void* w, void* out, int N, int K, long long ldw) {
  RV_CHECK(N > 0 && K > 0 && ldw >= K && w && out, "tile_weight: bad arguments N=%d K=%d", N, K);
  RV_CHECK(((uintptr_t)out % 16) == 0, "tile_weight: the output must be 16-byte aligned");
  const int k32 = rv_div_up(K, 32);
  const long long pieces = rv_tile_weight_elements(N, K) / 8;
  sk_tile_weight_kernel<<<dim3(rv_div_up(pieces, 256)), dim3(256), 0, stream>>>((const uint16_t*)w, (uint16_t*)out, N, K,
                                                                              ldw, k32, pieces);
  RV_LAUNCH_CHECK("tile_weight");
  return 0;
}

// out[m][n] (bf16 or 32-bit) = sum over slices of part[s][m][n].
extern "C" int rv_reduce_slices(hipStream_t stream, const float* part, void* out, int out_dtype, int slices, int M,
                                int N) {
  RV_CHECK(slices >= 1 && M >= 0 && N > 0 && part && out, "reduce_slices: bad arguments");
  if (M == 0) return 0;
  const long long total = (long long)M * N;
  if (out_dtype == RV_F32)
    sk_reduce_kernel<float><<<dim3(rv_div_up(total, 256)), dim3(256), 0, stream>>>(part, (float*)out, slices, M, N, N);
  else if (out_dtype == RV_BF16)
    sk_reduce_kernel<uint16_t><<<dim3(rv_div_up(total, 256)), dim3(256), 0, stream>>>(part, (uint16_t*)out, slices, M,
                                                                                    N, N);
  else
    return rv_fail("reduce_slices: unsupported output dtype %d", out_dtype);
  RV_LAUNCH_CHECK("reduce_slices");
  return 0;
}

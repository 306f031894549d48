// Mask preprocessing: elementwise mask -> block mask -> kept-tile lists.
// Integer/byte work bound by HBM bandwidth; output is bit-identical to the reference's
// build_groups_from_block_mask (fa2_custom_mask/fa2_custom_mask.py:15-38).
#include "common.h"

namespace bsattn {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// 16 bool bytes (each 0 or 1) -> 16 bits: a dot product of four bytes with (1, 2, 4, 8) or (16, 32, 64, 128)
// places four bits at once
__device__ __forceinline__ unsigned bools16(const u32x4& d) {
  const unsigned lo = __builtin_amdgcn_udot4(d[1], 0x80402010u, __builtin_amdgcn_udot4(d[0], 0x08040201u, 0u, false), false);
  const unsigned hi = __builtin_amdgcn_udot4(d[3], 0x80402010u, __builtin_amdgcn_udot4(d[2], 0x08040201u, 0u, false), false);
  return lo | (hi << 8);
}

// ---------------------------------------------------------------------------------------
// dense [.,.,N,N] bool -> block [.,.,nb,nb] bool (tile kept iff any element set).
// One wavefront owns 64 rows x 1024 columns (16 tiles): every lane ORs its 16-byte column
// slice over the 64 rows, then a ballot folds 4 lanes into one tile flag.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void reduce_dense_kernel(const uint8_t* __restrict__ dense, int N,
                                                           int nb, int H, int64_t sb, int64_t sh,
                                                           int64_t sm, uint8_t* __restrict__ block) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rb = blockIdx.x;
  const int col0 = (blockIdx.y * 4 + wave) * 1024;
  if (col0 >= N) return;
  const int bh = blockIdx.z;
  const int b = bh / H, h = bh % H;
  const int col = col0 + lane * 16;
  const bool in = col < N;
  const uint8_t* p = dense + b * sb + h * sh + (int64_t)rb * 64 * sm + (in ? col : 0);
  typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));
  uintx4 acc = {0u, 0u, 0u, 0u};
#pragma unroll 16
  for (int r = 0; r < 64; ++r) acc |= __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(p + r * sm));
  const bool nz = in && ((acc[0] | acc[1] | acc[2] | acc[3]) != 0u);
  const unsigned long long bal = __ballot(nz);
  if (lane < 16) {
    const int t = (col0 >> 6) + lane;
    if (t < nb) block[((int64_t)bh * nb + rb) * nb + t] = ((bal >> (4 * lane)) & 0xFull) ? 1 : 0;
  }
}

// one wavefront per mask row: number of kept tiles
__global__ __launch_bounds__(256) void count_rows_kernel(const uint8_t* __restrict__ block, int rows,
                                                         int nb, int H, int64_t sb, int64_t sh,
                                                         int64_t sm, int64_t sn,
                                                         int32_t* __restrict__ cnt) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int m = row % nb, bh = row / nb;
  const uint8_t* p = block + (bh / H) * sb + (bh % H) * sh + (int64_t)m * sm;
  int c = 0;
  for (int n0 = 0; n0 < nb; n0 += 64) {
    const int n = n0 + lane;
    const bool keep = n < nb && p[(int64_t)n * sn] != 0;
    c += __popcll(__ballot(keep));
  }
  if (lane == 0) cnt[row] = c;
}

// single workgroup: exclusive scan of the per-row counts (row_ptr) and of the non-empty
// flags (position of each row in `groups`); totals to counts[0..1].
__global__ __launch_bounds__(1024) void scan_rows_kernel(const int32_t* __restrict__ cnt, int rows,
                                                         int32_t* __restrict__ row_ptr,
                                                         int32_t* __restrict__ gidx,
                                                         int32_t* __restrict__ counts) {
  __shared__ int s_t[1024];
  __shared__ int s_g[1024];
  const int tid = threadIdx.x;
  const int per = (rows + 1023) / 1024;
  const int r0 = min(rows, tid * per), r1 = min(rows, r0 + per);
  int t = 0, g = 0;
  for (int r = r0; r < r1; ++r) { const int c = cnt[r]; t += c; g += c > 0; }
  s_t[tid] = t; s_g[tid] = g;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {   // Hillis-Steele inclusive scan
    int at = 0, ag = 0;
    if (tid >= off) { at = s_t[tid - off]; ag = s_g[tid - off]; }
    __syncthreads();
    s_t[tid] += at; s_g[tid] += ag;
    __syncthreads();
  }
  int bt = s_t[tid] - t, bg = s_g[tid] - g;    // exclusive prefix of this thread's span
  for (int r = r0; r < r1; ++r) {
    const int c = cnt[r];
    row_ptr[r] = bt; gidx[r] = bg;
    bt += c; bg += c > 0;
  }
  if (tid == 1023) { row_ptr[rows] = s_t[1023]; counts[0] = s_g[1023]; counts[1] = s_t[1023]; }
}

// one wavefront per mask row: ordered fill of col_idx and the row's `groups` entry
__global__ __launch_bounds__(256) void fill_rows_kernel(const uint8_t* __restrict__ block, int rows,
                                                        int nb, int H, int64_t sb, int64_t sh,
                                                        int64_t sm, int64_t sn,
                                                        const int32_t* __restrict__ row_ptr,
                                                        const int32_t* __restrict__ gidx,
                                                        int32_t* __restrict__ col_idx,
                                                        int32_t* __restrict__ groups) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int m = row % nb, bh = row / nb;
  const uint8_t* p = block + (bh / H) * sb + (bh % H) * sh + (int64_t)m * sm;
  const int start = row_ptr[row];
  int pos = start;
  for (int n0 = 0; n0 < nb; n0 += 64) {
    const int n = n0 + lane;
    const bool keep = n < nb && p[(int64_t)n * sn] != 0;
    const unsigned long long bal = __ballot(keep);
    if (keep) col_idx[pos + __popcll(bal & ((1ull << lane) - 1ull))] = n;
    pos += __popcll(bal);
  }
  if (groups != nullptr && lane == 0 && pos > start) {
    int32_t* g = groups + (int64_t)gidx[row] * 5;
    g[0] = bh / H; g[1] = bh % H; g[2] = m; g[3] = start; g[4] = pos - start;
  }
}


// ---------------------------------------------------------------------------------------
// Counting and scanning in one workgroup, for contiguous block masks of up to 1023 rows and 256 KB (one launch
// less: at 274 rows the launches and the gaps between them are nearly all of the 12 us the three steps take).
// In row-major order the kept tiles of a contiguous mask are a stream compaction of its bytes: thread t owns
// the `seg` consecutive bytes from t * seg (16-byte loads, held in registers), the block-wide exclusive scan of
// the threads' counts gives the number of kept tiles in front of a thread's segment, and the segments stay in
// LDS with one bit per byte: thread r then finds the start of row r as the count in front of the segment that
// holds byte r * nb plus the set bits of that segment below it.  Lengths and the rows' positions in `groups`
// follow from the starts after a second scan over the non-empty flags.
// The same launch writes col_idx and groups: one workgroup writing 75 000 scattered entries would take 36-50 us, so
// for masks of more than LISTS_FILL_MAX tiles the launch has LISTS_FILL_WGS workgroups, each of which counts and scans the
// whole mask for itself (75 KB from the L2) and fills its share of the entries.
// ---------------------------------------------------------------------------------------
constexpr int LISTS_ONE_MAX_ROWS = 1023, LISTS_ONE_MAX_SEG = 256;

// inclusive sum over the 1024 threads of the workgroup; s_w: 16 ints of LDS; returns the sum, *total = all
__device__ __forceinline__ int block_inclusive_sum(int v, int* s_w, int* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(v, off);
    if (lane >= off) v += o;
  }
  __syncthreads();                      // s_w may still be read from the previous use
  if (lane == 63) s_w[wave] = v;
  __syncthreads();
  int before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const int t = s_w[w];
    if (w < wave) before += t;
    all += t;
  }
  *total = all;
  return v + before;
}

// The kernel also writes col_idx and groups, every thread the entries of its own segment: with one workgroup for
// masks of up to LISTS_FILL_MAX tiles, with several for larger ones (see below).
constexpr int LISTS_FILL_MAX = 16384;
constexpr int LISTS_FILL_WGS = 32;
__global__ __launch_bounds__(1024) void count_scan_kernel(const uint8_t* __restrict__ block, int rows, int nb,
                                                          int seg, int32_t* __restrict__ row_ptr,
                                                          int32_t* __restrict__ gidx, int32_t* __restrict__ counts,
                                                          int H, int32_t* __restrict__ col_idx,
                                                          int32_t* __restrict__ groups) {
  constexpr int CH = LISTS_ONE_MAX_SEG / 16, WORDS = (CH + 1) / 2;
  __shared__ int s_w[16];
  __shared__ int s_off[1024];                   // kept tiles in front of a thread's segment
  __shared__ unsigned s_bits[1024][WORDS];      // a thread's segment, one bit per byte
  __shared__ int s_start[LISTS_ONE_MAX_ROWS + 1];
  const int tid = threadIdx.x;
  const int total = rows * nb, base = tid * seg;
  unsigned bits[WORDS];
#pragma unroll
  for (int w = 0; w < WORDS; ++w) bits[w] = 0u;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int off = base + 16 * c;
    if (16 * c < seg && off < total) {
      u32x4 d = {0u, 0u, 0u, 0u};
      if (off + 16 <= total) {
        d = *reinterpret_cast<const u32x4*>(block + off);
      } else {                            // the last, incomplete chunk of the mask: byte by byte
#pragma unroll
        for (int b = 0; b < 16; ++b)
          if (off + b < total) d[b >> 2] |= (unsigned)block[off + b] << (8 * (b & 3));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {       // every byte -> 0 / 1 (any non-zero byte counts as set)
        unsigned t = d[i];
        t |= t >> 4; t |= t >> 2; t |= t >> 1;
        d[i] = t & 0x01010101u;
      }
      bits[c >> 1] |= bools16(d) << (16 * (c & 1));
    }
  }
  int cnt = 0;
#pragma unroll
  for (int w = 0; w < WORDS; ++w) { cnt += __popc(bits[w]); s_bits[tid][w] = bits[w]; }
  int kept;
  s_off[tid] = block_inclusive_sum(cnt, s_w, &kept) - cnt;
  __syncthreads();
  // thread r: start of row r = kept tiles in front of byte r * nb
  if (tid <= rows) {
    int start = kept;
    if (tid < rows) {
      const int idx = tid * nb, t = idx / seg, k = idx - t * seg;
      start = s_off[t];
#pragma unroll
      for (int w = 0; w < WORDS; ++w) {
        const int below = k - 32 * w;     // bits of this word in front of the row's first byte
        const unsigned m = below <= 0 ? 0u : below >= 32 ? ~0u : (1u << below) - 1u;
        start += __popc(s_bits[t][w] & m);
      }
      if (blockIdx.x == 0) row_ptr[tid] = start;
    } else if (blockIdx.x == 0) {
      row_ptr[rows] = kept; counts[1] = kept;
    }
    s_start[tid] = start;
  }
  __syncthreads();
  const int len = tid < rows ? s_start[tid + 1] - s_start[tid] : 0;
  int ngroups;
  const int gi = block_inclusive_sum(len > 0 ? 1 : 0, s_w, &ngroups) - (len > 0 ? 1 : 0);
  if (blockIdx.x == 0) {
    if (tid < rows) gidx[tid] = gi;
    if (tid == 0) counts[0] = ngroups;
  }
  if (gridDim.x == 1) {
    // entry number s_off[tid] + k of the list is the k-th set byte of this thread's segment: its column block
    int pos = s_off[tid];
    int col = base % nb;                          // column block of the segment's first byte
#pragma unroll
    for (int w = 0; w < WORDS; ++w) {
      unsigned b = bits[w];
      int at = 0;                                 // bit position that `col` belongs to
      while (b != 0u) {
        const int bit = __ffs(b) - 1;
        b &= b - 1u;
        col += bit - at; at = bit;
        while (col >= nb) col -= nb;
        col_idx[pos++] = col;
      }
      col += 32 - at;
      while (col >= nb) col -= nb;
    }
    if (groups != nullptr && len > 0) {
      const int bh = tid / nb;
      int32_t* g = groups + (int64_t)gi * 5;
      g[0] = bh / H; g[1] = bh % H; g[2] = tid % nb; g[3] = s_start[tid]; g[4] = len;
    }
  } else {
    // Larger masks: several workgroups, each of which has counted and scanned the whole mask for itself (it sits in
    // the L2) and now fills its share of the rows, one wavefront per row (ballot and rank, as fill_rows_kernel):
    // one workgroup alone would spend 36 us on the scattered stores of 75 000 entries.
    if (tid < rows) s_off[tid] = gi;              // (the segments' offsets are no longer needed)
    __syncthreads();
    const int lane = tid & 63, nw = (int)gridDim.x * 16;
    for (int row = (int)blockIdx.x * 16 + (tid >> 6); row < rows; row += nw) {
      const uint8_t* p = block + (int64_t)row * nb;
      const int start = s_start[row];
      int pos = start;
      for (int n0 = 0; n0 < nb; n0 += 64) {
        const int n = n0 + lane;
        const bool keep = n < nb && p[n] != 0;
        const unsigned long long bal = __ballot(keep);
        if (keep) col_idx[pos + __popcll(bal & ((1ull << lane) - 1ull))] = n;
        pos += __popcll(bal);
      }
      if (groups != nullptr && lane == 0 && pos > start) {
        const int bh = row / nb;
        int32_t* g = groups + (int64_t)s_off[row] * 5;
        g[0] = bh / H; g[1] = bh % H; g[2] = row % nb; g[3] = start; g[4] = pos - start;
      }
    }
  }
}


// ---------------------------------------------------------------------------------------
// The 64 x 64 bit matrix whose row r is the word of lane r, transposed: six rounds of block swaps between lanes
// l and l ^ j (j = 32 ... 1), each exchanging the off-diagonal j x j blocks of every 2j x 2j block.
__device__ __forceinline__ unsigned long long transpose64(unsigned long long word, int lane) {
  unsigned long long keep = 0x00000000ffffffffull;     // columns c with (c & j) == 0
#pragma unroll
  for (int j = 32; j >= 1; j >>= 1) {
    const unsigned lo = __shfl_xor((unsigned)word, j), hi = __shfl_xor((unsigned)(word >> 32), j);
    const unsigned long long other = ((unsigned long long)hi << 32) | lo;
    word = (lane & j) ? (word & (keep << j)) | ((other & (keep << j)) >> j)
                      : (word & keep) | ((other & keep) << j);
    keep ^= keep << (j >> 1);        // 0x0000ffff0000ffff, 0x00ff00ff..., ..., 0x5555...
  }
  return word;
}

// ---------------------------------------------------------------------------------------
// Elementwise masks: the 64 x 64 bools of every kept tile packed into 64 words of 64 bits
// (word r = row r of the tile, bit c = column c), plus a flag per kept tile saying whether the
// tile is only partly set.  Slot t of `bits` / `partial` belongs to entry t of the kept-tile
// list.  `split` workgroups of 4 wavefronts per mask row block, their wavefronts striding over
// the row block's kept tiles; lane l packs row l of the tile.  A wavefront has one turn's loads in
// flight at a time, so the kernel lives on the number of wavefronts: `split` is chosen so that even
// a full row gives every wavefront a single turn (every tile of a 17536 x 17536 mask kept: 64 us
// against 72 us with 8 workgroups per row).  With the row and
// column strides of the mask and the lists both transposed, the words describe the columns (what the
// dK/dV pass needs).
// ---------------------------------------------------------------------------------------
constexpr int PACK_SPLIT_MAX = 32;
// workgroups per mask row block: a full row of nb tiles gives every wavefront one turn of `per_turn` tiles
static int pack_split(int nb, int per_turn) {
  const int s = (nb + 4 * per_turn - 1) / (4 * per_turn);
  return s < 1 ? 1 : s > PACK_SPLIT_MAX ? PACK_SPLIT_MAX : s;
}
constexpr int PACK_G = 4;     // measured against 8 and 16: fewer, longer wavefronts lose more than longer runs gain


// MODE 0: columns are contiguous in memory (sn == 1); MODE 1: rows are (sm == 1: the call for the column
// lists, with the mask's strides swapped); MODE 2: neither (one byte per load, one tile per wavefront).
// MODE 0 / 1: a tile is 64 memory rows of 64 contiguous bytes, half a 128-byte line of the L2, whose other
// half belongs to the neighbouring tile, and a small piece of a DRAM page.  A wavefront therefore takes G
// consecutive entries of the list at a time (in a dense stretch of a row list: 64 G contiguous bytes per
// memory row): one load instruction covers 16 / G memory rows of the G tiles, 16 bytes per lane.  The four
// lanes that share a memory row of a tile put their bits together, the words go through LDS so that lane l
// ends up with the word of memory row l of each tile.  In MODE 1 that is bit r of the words to come for
// column l: the 64 x 64 bit matrix is transposed between the lanes (transpose64).
template <int MODE, int G>
__global__ __launch_bounds__(256) void pack_tiles_kernel(const uint8_t* __restrict__ dense, int nb, int H,
                                                         int64_t sb, int64_t sh, int64_t sm, int64_t sn,
                                                         const int32_t* __restrict__ row_ptr,
                                                         const int32_t* __restrict__ col_idx,
                                                         uint8_t* __restrict__ partial,
                                                         unsigned long long* __restrict__ bits, int split) {
  __shared__ unsigned long long stage[MODE == 2 ? 1 : 4][MODE == 2 ? 1 : G][64];      // [wavefront][tile of the group][memory row]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // (row blocks from the last to the first: with causal masks the long lists then start first)
  const int rb = nb - 1 - blockIdx.x / split, bh = blockIdx.y;
  // Workgroups go to the 8 XCDs round-robin.  With a split that is a multiple of 8 an unrotated share index ties
  // every XCD, and its L2, to the same byte ranges of all memory rows of the mask; rotating the shares by the row
  // block spreads them (measured at N = 17536, token-causal mask: 28.7 against 32.9 us with 8 shares; without the
  // rotation 14, 18 and 20 shares were fast and 8 and 16 slow).  The transposing mode measured the other way round
  // (8, 16, 24 shares unrotated: 41-44 us; 12, 18, 32: 51-56 us) and keeps the tie.
  const int sub = MODE == 1 ? blockIdx.x % split : (blockIdx.x + rb) % split;
  const int32_t* rp = row_ptr + (int64_t)bh * nb;
  const int t0 = rp[rb], t1 = rp[rb + 1];
  const uint8_t* head = dense + (bh / H) * sb + (bh % H) * sh + (int64_t)rb * 64 * sm;
  if constexpr (MODE == 2) {
    for (int t = t0 + sub * 4 + wave; t < t1; t += 4 * split) {
      const uint8_t* p = head + (int64_t)col_idx[t] * 64 * sn + lane * sm;
      unsigned long long word = 0ull;
      for (int c = 0; c < 64; ++c) word |= (unsigned long long)(p[(int64_t)c * sn] != 0) << c;
      bits[(int64_t)t * 64 + lane] = word;
      const bool full = __ballot(word == ~0ull) == ~0ull;
      if (lane == 0) partial[t] = full ? 0 : 1;
    }
  } else {
    constexpr int RPI = 16 / G;                      // memory rows per load instruction
    const int64_t S = MODE == 0 ? sm : sn;           // stride between memory rows (the other stride is 1)
    const int64_t step = 64 * sn;                    // offset of a tile = its column block times this
    const int sub_row = lane / (4 * G), j = (lane >> 2) % G, chunk = lane & 3;
    unsigned long long (*my)[64] = stage[wave];
    for (int tg = t0 + G * (sub * 4 + wave); tg < t1; tg += 4 * G * split) {
      const int tj = tg + j < t1 ? tg + j : t1 - 1;               // (a group past the end repeats the last tile)
      const uint8_t* p = head + (int64_t)col_idx[tj] * step + (int64_t)sub_row * S + 16 * chunk;
#pragma unroll 1
      for (int r0 = 0; r0 < 64; r0 += 16 * RPI) {                 // 16 loads in flight
        u32x4 d[16];
#pragma unroll
        for (int it = 0; it < 16; ++it)
          d[it] = *reinterpret_cast<const u32x4*>(p + (r0 + RPI * it) * S);   // (cached: a neighbour wants the other half line)
#pragma unroll
        for (int it = 0; it < 16; ++it) {
          // the 16 bits of the four lanes that share the memory row, side by side (lane 4k + c holds bits 16c ..)
          const unsigned h = bools16(d[it]);
          const unsigned h0 = __builtin_amdgcn_mov_dpp(h, 0x00, 0xf, 0xf, true), h1 = __builtin_amdgcn_mov_dpp(h, 0x55, 0xf, 0xf, true);
          const unsigned h2 = __builtin_amdgcn_mov_dpp(h, 0xaa, 0xf, 0xf, true), h3 = __builtin_amdgcn_mov_dpp(h, 0xff, 0xf, 0xf, true);
          const unsigned long long x = (unsigned long long)(h0 | (h1 << 16)) | ((unsigned long long)(h2 | (h3 << 16)) << 32);
          if (chunk == 0) my[j][r0 + RPI * it + sub_row] = x;    // word of that memory row of tile j
        }
      }
      // (the LDS operations of one wavefront complete in order: the reads below see the writes above)
#pragma unroll 1
      for (int jj = 0; jj < G; ++jj) {
        if (tg + jj >= t1) break;
        unsigned long long word = my[jj][lane];
        if constexpr (MODE == 1) word = transpose64(word, lane);
        bits[(int64_t)(tg + jj) * 64 + lane] = word;
        const bool full = __ballot(word == ~0ull) == ~0ull;
        if (lane == 0) partial[tg + jj] = full ? 0 : 1;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Elementwise masks in one pass over the mask: block mask, "partly set" flags and the packed words of every
// tile that has a set element, all indexed by the tile's position in the grid ((mask head * nb + row block) * nb
// + column block), since the lists do not exist yet.  gather_tiles_kernel then moves the words of the kept
// tiles to their list positions, for the row lists as they are and for the column lists transposed, so the
// mask itself (Bm Hm N^2 bytes) is read once, in whole rows, whatever is made of it afterwards.
// As reduce_dense_kernel, one wavefront owns 64 rows x 1024 columns (16 tiles): a lane reads its 16-byte
// column slice of every row (16 rows in flight), turns it into 16 bits, the four lanes of a tile put theirs
// together, and the words wait in LDS until the 64 rows are through; then lane l holds the word of row l of
// each tile and the wavefront writes 512 contiguous bytes per tile.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void reduce_pack_kernel(const uint8_t* __restrict__ dense, int N, int nb, int H,
                                                          int64_t sb, int64_t sh, int64_t sm,
                                                          uint8_t* __restrict__ block, uint8_t* __restrict__ grid_partial,
                                                          unsigned long long* __restrict__ grid_bits) {
  __shared__ unsigned long long stage[4][16][64];      // [wavefront][tile][row]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rb = blockIdx.x;
  const int col0 = (blockIdx.y * 4 + wave) * 1024;
  if (col0 >= N) return;
  const int bh = blockIdx.z;
  const int b = bh / H, h = bh % H;
  const int col = col0 + lane * 16;
  const bool in = col < N;
  const uint8_t* p = dense + b * sb + h * sh + (int64_t)rb * 64 * sm + (in ? col : 0);
  const int j = lane >> 2, chunk = lane & 3;
  unsigned long long (*my)[64] = stage[wave];
#pragma unroll 1
  for (int r0 = 0; r0 < 64; r0 += 16) {
    u32x4 d[16];
#pragma unroll
    for (int it = 0; it < 16; ++it) d[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + (r0 + it) * sm));
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const unsigned hbits = in ? bools16(d[it]) : 0u;
      const unsigned h0 = __builtin_amdgcn_mov_dpp(hbits, 0x00, 0xf, 0xf, true), h1 = __builtin_amdgcn_mov_dpp(hbits, 0x55, 0xf, 0xf, true);
      const unsigned h2 = __builtin_amdgcn_mov_dpp(hbits, 0xaa, 0xf, 0xf, true), h3 = __builtin_amdgcn_mov_dpp(hbits, 0xff, 0xf, 0xf, true);
      const unsigned long long x = (unsigned long long)(h0 | (h1 << 16)) | ((unsigned long long)(h2 | (h3 << 16)) << 32);
      if (chunk == 0) my[j][r0 + it] = x;
    }
  }
  // (the LDS operations of one wavefront complete in order: the reads below see the writes above)
  const int t0 = col0 >> 6;
#pragma unroll 1
  for (int jj = 0; jj < 16; ++jj) {
    const int t = t0 + jj;
    if (t >= nb) break;
    const unsigned long long word = my[jj][lane];
    const bool any = __ballot(word != 0ull) != 0ull;
    const bool full = __ballot(word == ~0ull) == ~0ull;
    const int64_t tile = ((int64_t)bh * nb + rb) * nb + t;
    if (any) grid_bits[tile * 64 + lane] = word;        // (tiles without a set element are never looked at)
    if (lane == 0) { block[tile] = any ? 1 : 0; grid_partial[tile] = any && !full ? 1 : 0; }
  }
}

// Words of the kept tiles from their grid positions to their list positions.  TRANSPOSE: the lists are the column
// lists (list row = column block a, entries = row blocks), and the words are wanted per key with one bit per
// query: the 64 x 64 bit matrix is transposed between the lanes (transpose64).  One workgroup of four wavefronts per
// `split`-th of a list row, a wavefront per entry, four entries of a wavefront in flight; as in pack_tiles_kernel
// the shares are as many as give every wavefront of a full list one turn, and rotated by the list row.
constexpr int GATHER_FLY = 4;
template <bool TRANSPOSE>
__global__ __launch_bounds__(256) void gather_tiles_kernel(const uint8_t* __restrict__ grid_partial,
                                                           const unsigned long long* __restrict__ grid_bits, int nb,
                                                           const int32_t* __restrict__ row_ptr,
                                                           const int32_t* __restrict__ col_idx,
                                                           uint8_t* __restrict__ partial,
                                                           unsigned long long* __restrict__ bits, int split) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int a = blockIdx.x / split, sub = (blockIdx.x + a) % split, mh = blockIdx.y;
  const int32_t* rp = row_ptr + (int64_t)mh * nb;
  const int t0 = rp[a], t1 = rp[a + 1];
  // four entries of the wavefront in flight: their words are asked for before the first is written
  constexpr int FLY = GATHER_FLY;
  const int STEP = 4 * split;
  for (int t = t0 + sub * 4 + wave; t < t1; t += STEP * FLY) {
    unsigned long long word[FLY];
    uint8_t part[FLY];
#pragma unroll
    for (int f = 0; f < FLY; ++f) {
      const int tt = t + f * STEP;
      if (tt < t1) {
        const int other = col_idx[tt];
        const int64_t tile = TRANSPOSE ? ((int64_t)mh * nb + other) * nb + a : ((int64_t)mh * nb + a) * nb + other;
        word[f] = grid_bits[tile * 64 + lane];
        part[f] = grid_partial[tile];
      }
    }
#pragma unroll
    for (int f = 0; f < FLY; ++f) {
      const int tt = t + f * STEP;
      if (tt < t1) {
        bits[(int64_t)tt * 64 + lane] = TRANSPOSE ? transpose64(word[f], lane) : word[f];
        if (lane == 0) partial[tt] = part[f];
      }
    }
  }
}

int launch_reduce_pack(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh, int64_t sm,
                       uint8_t* block_out, uint8_t* grid_partial, unsigned long long* grid_bits, hipStream_t st) {
  const int nb = N / 64;
  dim3 grid(nb, (N + 4095) / 4096, Bm * Hm);
  hipLaunchKernelGGL(reduce_pack_kernel, grid, dim3(256), 0, st, dense, N, nb, Hm, sb, sh, sm, block_out, grid_partial,
                     grid_bits);
  return launch_status();
}

int launch_gather_tiles(const uint8_t* grid_partial, const unsigned long long* grid_bits, int Bm, int Hm, int nb,
                        int transposed, const int32_t* row_ptr, const int32_t* col_idx, uint8_t* partial,
                        unsigned long long* bits, hipStream_t st) {
  const int split = pack_split(nb, GATHER_FLY);
  const dim3 grid(nb * split, Bm * Hm);
  if (transposed)
    hipLaunchKernelGGL(gather_tiles_kernel<true>, grid, dim3(256), 0, st, grid_partial, grid_bits, nb, row_ptr, col_idx, partial, bits, split);
  else
    hipLaunchKernelGGL(gather_tiles_kernel<false>, grid, dim3(256), 0, st, grid_partial, grid_bits, nb, row_ptr, col_idx, partial, bits, split);
  return launch_status();
}

int launch_reduce_dense_mask(const uint8_t* dense, int Bm, int Hm, int N, int64_t sb, int64_t sh,
                             int64_t sm, uint8_t* block_out, hipStream_t st) {
  const int nb = N / 64;
  dim3 grid(nb, (N + 4095) / 4096, Bm * Hm);
  hipLaunchKernelGGL(reduce_dense_kernel, grid, dim3(256), 0, st, dense, N, nb, Hm, sb, sh, sm,
                     block_out);
  return launch_status();
}

int launch_block_mask_to_lists(const uint8_t* block, int Bm, int Hm, int nb, int64_t sb, int64_t sh,
                               int64_t sm, int64_t sn, int32_t* row_ptr, int32_t* col_idx,
                               int32_t* groups, int32_t* counts, int32_t* ws, hipStream_t st) {
  const int rows = Bm * Hm * nb;
  const int64_t total = (int64_t)rows * nb;
  const bool contiguous = sn == 1 && sm == nb && (Hm == 1 || sh == (int64_t)nb * nb) &&
                          (Bm == 1 || sb == (int64_t)Hm * nb * nb) && ((uintptr_t)block & 15) == 0;
  int32_t* cnt = ws;
  int32_t* gidx = ws + rows;
  const dim3 grid((rows + 3) / 4);
  if (contiguous && rows <= LISTS_ONE_MAX_ROWS && total <= 1024 * LISTS_ONE_MAX_SEG) {
    const int seg = (((int)total + 1023) / 1024 + 15) / 16 * 16;
    // the whole call in one launch: one workgroup for small masks, LISTS_FILL_WGS for larger ones (each counts and
    // scans for itself and fills its share)
    hipLaunchKernelGGL(count_scan_kernel, dim3(total <= LISTS_FILL_MAX ? 1 : LISTS_FILL_WGS), dim3(1024), 0, st, block,
                       rows, nb, seg, row_ptr, gidx, counts, Hm, col_idx, groups);
    return launch_status();
  } else {
    hipLaunchKernelGGL(count_rows_kernel, grid, dim3(256), 0, st, block, rows, nb, Hm, sb, sh, sm, sn, cnt);
    hipLaunchKernelGGL(scan_rows_kernel, dim3(1), dim3(1024), 0, st, cnt, rows, row_ptr, gidx, counts);
  }
  hipLaunchKernelGGL(fill_rows_kernel, grid, dim3(256), 0, st, block, rows, nb, Hm, sb, sh, sm, sn,
                     row_ptr, gidx, col_idx, groups);
  return launch_status();
}

// Sequence lengths that are not a multiple of 64: the last column block holds only `valid` keys.
// One workgroup per list row (mask head, block a); for each of its kept tiles the flag and the 64
// words in the format of pack_tiles_kernel: all ones, except in the last column block, where
// (row lists) every word keeps its low `valid` bits or (column lists: word = key, bit = query)
// only the first `valid` words are set.
__global__ __launch_bounds__(256) void tail_tiles_kernel(const int32_t* __restrict__ row_ptr,
                                                         const int32_t* __restrict__ col_idx, int nb, int valid,
                                                         int transpose, uint8_t* __restrict__ partial,
                                                         unsigned long long* __restrict__ bits) {
  const int r = blockIdx.x, a = r % nb;
  const int t0 = row_ptr[r], t1 = row_ptr[r + 1];
  const unsigned long long ones = ~0ull, low = valid >= 64 ? ones : ((1ull << valid) - 1ull);
  for (int i = threadIdx.x; i < (t1 - t0) * 64; i += 256) {
    const int t = t0 + (i >> 6), w = i & 63;
    const bool last = transpose ? a == nb - 1 : col_idx[t] == nb - 1;
    unsigned long long word = ones;
    if (last) word = transpose ? (w < valid ? ones : 0ull) : low;
    bits[(int64_t)t * 64 + w] = word;
    if (w == 0) partial[t] = last && valid < 64 ? 1 : 0;
  }
}

int launch_tail_tiles(int Bm, int Hm, int nb, int valid, int transpose, const int32_t* row_ptr,
                      const int32_t* col_idx, uint8_t* partial, unsigned long long* bits, hipStream_t st) {
  hipLaunchKernelGGL(tail_tiles_kernel, dim3(Bm * Hm * nb), dim3(256), 0, st, row_ptr, col_idx, nb, valid, transpose,
                     partial, bits);
  return launch_status();
}

int launch_pack_tiles(const uint8_t* dense, int Bm, int Hm, int nb, int64_t sb, int64_t sh, int64_t sm,
                      int64_t sn, const int32_t* row_ptr, const int32_t* col_idx, uint8_t* partial,
                      unsigned long long* bits, hipStream_t st) {
  // the wide loads need 16-byte aligned memory rows
  const bool wide = (((uintptr_t)dense | (uintptr_t)sb | (uintptr_t)sh) & 15) == 0;
  if (wide && sn == 1 && sm % 16 == 0) {
    const int split = pack_split(nb, PACK_G);
    hipLaunchKernelGGL((pack_tiles_kernel<0, PACK_G>), dim3(nb * split, Bm * Hm), dim3(256), 0, st, dense, nb, Hm, sb, sh, sm, sn, row_ptr, col_idx, partial, bits, split);
  } else if (wide && sm == 1 && sn % 16 == 0) {
    const int split = 8;      // (see the kernel)
    hipLaunchKernelGGL((pack_tiles_kernel<1, 4>), dim3(nb * split, Bm * Hm), dim3(256), 0, st, dense, nb, Hm, sb, sh, sm, sn, row_ptr, col_idx, partial, bits, split);
  } else {
    const int split = 8;
    hipLaunchKernelGGL((pack_tiles_kernel<2, 1>), dim3(nb * split, Bm * Hm), dim3(256), 0, st, dense, nb, Hm, sb, sh, sm, sn, row_ptr, col_idx, partial, bits, split);
  }
  return launch_status();
}

}  // namespace bsattn

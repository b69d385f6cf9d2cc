// Device-side parameter blocks shared by the convolution plan builder (host)
// and the implicit-GEMM kernels.
#pragma once

#include <hip/hip_runtime.h>

namespace mg {

// Division of a non-negative n < 2^31 by a divisor fixed at plan time:
// q = umulhi(n, mul) >> shr  (mul = ceil(2^(31+ceil_log2(d)) / d)); d == 1 is
// special-cased because its multiplier does not fit 32 bits.
struct FastDiv {
  unsigned mul, shr, d, pad_;
#ifdef __HIPCC__
  __device__ __forceinline__ unsigned div(unsigned n) const { return d == 1u ? n : __umulhi(n, mul) >> shr; }
#endif
};

inline FastDiv make_fastdiv(unsigned d) {
  FastDiv f{0u, 0u, d, 0u};
  if (d > 1u) {
    unsigned lg = 0;
    while ((1ull << lg) < d) ++lg;  // ceil(log2(d))
    const unsigned p = 31u + lg;
    f.mul = (unsigned)(((1ull << p) + d - 1ull) / d);
    f.shr = p - 32u;
  }
  return f;
}

// One row of the contraction table.  For the forward pass a row is one (c, tap);
// for the data gradient one (f, tap) of a stride phase.  `off` is the element
// offset that the row adds to a position's base offset inside one batch item of
// the gathered tensor; d[k] is what it adds to the position's coordinate on axis
// k, which must land in [0, Q[k]) for the element to exist (otherwise it is a
// padding zero).
struct TabEntry {
  int off;
  int d0, d1, d2;
};

// One K tile of the tap-major gather-GEMM: BK consecutive channels (forward) or
// filters (data gradient) under one filter tap.  Rows a_row0.. of the packed
// filter matrix multiply the gathered elements at `coff` + i * channel stride;
// all of them share the tap's coordinate offsets d[k], hence one validity test.
struct KTile {
  int a_row0;
  int coff;
  int d0, d1, d2;
  int pad0_, pad1_, pad2_;
};

// Sixteen consecutive columns of the filter-gradient matrix as the tap-major kernel
// lays it out: one tap, channels c0..c0+15 (c0 a multiple of 16); the groups of one
// channel block follow each other, one per tap.  `coff` = c0 * channel stride + the
// tap's element offset.
struct WGroup {
  int coff;
  int d0, d1, d2;
  int valid;
  int pad0_, pad1_, pad2_;
};

// A stride phase of the data gradient (the forward pass has exactly one phase).
// Positions of a phase are (n, j0, j1, j2), j_k in [0, J[k]); position j maps to
// the destination coordinate o0[k] + j_k * oj[k].
struct Phase {
  int J[3];
  int o0[3];
  int k_begin, k_count;  // rows [k_begin, k_begin + k_count) of the table
  int blk_begin;         // first block (along positions) that works on this phase
  int npos;              // N * J0 * J1 * J2
  FastDiv by_jvol, by_j12, by_j2;  // divisions that turn a position into (n, j0, j1, j2)
  int pad_[2];                     // 96 bytes: three 32-byte scalar loads
};
static_assert(sizeof(Phase) == 96, "Phase is read as three 32-byte rows");

// A slice of a tile's K tiles that one block computes (see GemmParams::share_first), and a tile
// whose slices the fix-up pass adds: its partial sums lie in consecutive slots, in K order.
struct ShareSlice {
  int tile, kt_begin, kt_end;
  int slot;  // of the partial sums; -1: all of the tile's K tiles, stored directly
};
struct ShareFix {
  int tile, first_slot, slots, pad_;
};

// Gather-GEMM:  dst[n, m, pos] = sum_k A(k, m) * src[n, row k, pos]
// The tap-major kernels read A from packed filters, [rows][a_ld] with the M values of a row
// contiguous; the table-driven kernel reads the filter bank where it lies:
// A(k, m) = A[arow[k] + m * a_mstride].
struct GemmParams {
  const void *A;
  const void *src;
  void *dst;
  const TabEntry *tab;
  const int *arow;  // table row -> offset of its m = 0 element in the filter bank
  int a_mstride;    // elements between consecutive m in the filter bank
  const Phase *phases;
  int nphases;
  int M;
  int Q[3];   // extents of the gathered tensor's spatial axes
  int sj[3];  // source coordinate advance per position step
  int qs[3];  // source element strides of the spatial axes
  int oj[3];  // destination coordinate advance per position step
  int os[3];  // destination element strides of the spatial axes
  int dst_mstride;
  long long src_nstride, dst_nstride;
  // tap-major kernels only
  const KTile *ktiles;  // Phase::k_begin / k_count index this table
  const void *zeros;    // a few zero elements in device memory
  unsigned a_bytes, src_bytes;  // sizes of A and src (each below 2 GiB)
  int a_ld;                     // values per row of A (M rounded up to a multiple of 4)
  int src_cstride;      // element stride between consecutive channels of the gathered tensor
  int vec_store;        // positions are contiguous in dst: a lane may store its TN positions as one vector
  int run_store;        // positions run through each sample of dst in order, rows not 16-byte aligned: a lane whose
                        // TN positions lie in one sample stores them as one vector of element alignment
  int m_tiles;          // row tiles per position block
  int items;            // work items: full_tiles whole tiles, then tail_split K slices of each remaining tile
  int full_tiles;       // tiles computed whole by one block each
  int tail_split;       // blocks that share each remaining tile (K slices), >= 1
  void *partial;        // [tail tile][slice][phase][BM][BN] partial sums of the shared tiles
  // Even shares of the last, partial round (persistent blocks): the K tiles of the tiles beyond
  // full_tiles, laid end to end, are cut into one run per block; a run is a few slices (a tile's
  // end, whole tiles, a tile's beginning).  share_first != nullptr switches this on; tail_split is
  // then not used.  After its whole tiles b, b + grid, ... block b takes the slices
  // share_first[b] .. share_first[b + 1] - 1.
  const int *share_first;     // [grid + 1]
  const ShareSlice *share_slices;
  const ShareFix *share_fix;  // the tiles that were cut, one thread block row of tail_fixup_kernel each
  // Fused stride phases (data gradient with a stride, tap-major kernel with NPH > 1): the phase
  // table holds ONE phase, the coarse grid J[k] = ceil(X[k] / stride[k]); every tile computes all
  // nph stride phases of its coarse positions, one accumulator set each, and writes them together,
  // so that the interleaved elements of dx leave the block as whole runs.
  int nph;              // 1 (not fused), 2 or 4; phases 2q and 2q+1 alternate along the last axis (po0[.][2] = 0, 1)
  int kcut[4];          // a tile's K tiles run filter block by filter block, kcut[nph-1] tiles each (the taps of all
                        // phases); tiles [kcut[f-1], kcut[f]) of a block belong to phase f (kcut[-1] = 0)
  int po0[4][3];        // destination coordinate of coarse position (0,0,0) in phase f
  int pJ[4][3];         // coarse positions j_k < pJ[f][k] exist in phase f
  // Taps of the last axis folded into the rows (tap-major kernel with FOLD): row 3*m + t of a tile
  // holds the sum over the taps of the other axes only, for tap t of the last axis, at the
  // position's own place along that axis; the epilogue adds the three rows of an m, each shifted
  // by its tap's offset along the last axis (+1, 0, -1 positions), into the one row of dst.
  int fold_row;         // 0: not folded; else the length of a row of positions (a power of two, 4 .. 64)
  // Stride phases as rows (data gradient of a few channels under a stride): the positions are the
  // coarse grid J[k] = ceil(X[k] / stride[k]) and row m of the GEMM is stride phase m % phase_count
  // of channel m / phase_count, so that every gathered element of grad serves all phases of its
  // coarse position (the packed filters hold a zero where a phase has no tap for it) and the
  // rows of an MFMA tile are channels x phases instead of channels alone.  po0 / pJ above say
  // where a phase's elements lie in dst and which exist; phases 2q and 2q + 1 are rows next to
  // each other and, with a stride of two along the last axis, elements next to each other.
  // Row tiles of one position block on one XCD (persistent blocks without even shares): blocks are
  // handed to the 8 XCDs round-robin, each with its own L2, and the m_tiles row tiles of a position
  // block gather the same elements.  With xcd_chunk = c > 1 the j-th block of an XCD starts on tile
  // ((j / c) * 8 + xcd) * c + j % c instead of on its own number: c consecutive tiles meet in one L2
  // (c divides 32, so that the two blocks of a compute unit still take tiles 256 apart).
  int xcd_chunk;
  int phase_count;      // 0: off; else the number of stride phases (2 or 4)
  int phase_pairs;      // phases 2q, 2q + 1 are neighbours along the last axis of dst
};

// Gather-GEMM with one position per lane, for few rows (the data gradient of a layer with a
// handful of channels, the forward pass of one with a handful of filters or of a first layer):
//   dst[n, m, pos of phase f] = sum over groups kg, entries e of  A(kg, e, f, m) * src[n, base(pos) + kg * group_stride + off_e]
// `tab` holds the entries in chunks of 16 / nph: entry e adds `off` elements to the
// position's base offset and d[k] to its source coordinate on axis k, which must land in
// [0, Q[k]) (else the element is a padding zero).  The packed operand holds, for chunk q and
// group kg, 64 values [entry within chunk][phase][row group][row within group]: zero where the
// entry feeds no tap of that phase, or the row is beyond M.
struct ThinParams {
  const float *A;
  const float *src;
  float *dst;
  const TabEntry *tab;
  int chunks;           // chunks of 16 / (nph * rg) entries
  int kgroups;          // groups of source channels: chunks * kgroups steps in all
  int kblock;           // groups per block: all chunks run under one block of groups before the next block
  unsigned group_bytes; // bytes of src between consecutive groups
  unsigned a_bytes, src_bytes;
  int M;
  int npos;             // N * J0 * J1 * J2 (coarse) positions
  int J[3];
  FastDiv by_jvol, by_j12, by_j2;
  int Q[3];    // extents of the gathered tensor's spatial axes
  int sj[3];   // source coordinate advance per position step
  int qs[3];   // source element strides of the spatial axes
  int oj[3];   // destination coordinate advance per position step
  int os[3];   // destination element strides of the spatial axes
  int dst_mstride;
  long long src_nstride, dst_nstride;
  int nph;          // 1, 2 or 4 stride phases per position
  int rg;           // groups of four rows per pass, nph * rg <= 16
  int passes;       // blocks of 4 * rg rows (grid.y); M <= 4 * rg * passes.  Pass y reads the packed filters
                    // from A + y * pass_floats and writes rows 4 * rg * y ...
  long long pass_floats;
  int po0[4][3];    // destination coordinate of position (0,0,0) in phase f
  int pJ[4][3];     // positions j_k < pJ[f][k] exist in phase f
  int pair_store;   // phases 2q and 2q+1 are neighbours along the last axis of dst, stored as one 8-byte piece
};

// conv_thin.hip
int launch_thin_pack(const float *w, float *packed, const int *arow, int chunks, int kgroups, long long group_stride, int m_stride, int M,
                     int rg, int passes, hipStream_t s);
int launch_thin_gemm(const ThinParams &p, hipStream_t s);
bool thin_gemm_has(int nph, int rg);

// Filter gradient:  out[split][f][col] = sum over the split's positions (n, g) of
//   grad[n, f, g] * x[n, column col at g]
struct WgradParams {
  const void *grad;
  const void *x;
  void *out;            // dw itself when splits == 1, else the partial-sum workspace
  const TabEntry *tab;  // one row per column (c, tap): the forward table
  int F, CT;            // rows and columns of dw viewed as a matrix
  int G[3], Q[3], sj[3], qs[3];
  int gvol;
  long long x_nstride, g_nstride;
  int kpos;    // N * gvol, the length of the sum
  int kchunk;  // positions per split (multiple of the K tile)
  int splits;
  FastDiv by_gvol, by_g12, by_g2;  // divisions that turn a position into (n, g0, g1, g2)
  // tap-major kernel only
  const WGroup *groups;
  const void *zeros;
  int x_cstride;
  unsigned grad_bytes, x_bytes;  // sizes of grad and x (each below 2 GiB)
  int col_tiles, row_tiles;  // tiles of the output matrix along columns / filters
  // One row of four 32-bit words per position (n, g), or null: the byte offset into x of the
  // position's window origin (without the padding shift, which the column groups' offsets carry),
  // the taps whose element exists there as a bit mask (64 taps at most, row-major), and what the
  // position's sample adds to the byte offset of grad[0][f][position]: n * (F - 1) * gvol elements.
  const void *pos_tab;
  int wvol;  // taps of the window
};

}  // namespace mg

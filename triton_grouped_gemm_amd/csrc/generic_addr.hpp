// Address arithmetic of the shape-agnostic kernel (gemm_generic.hip), kept apart from the kernel so that the library
// can also run it on the host: tgg_debug_generic_extents walks every tile of a launch with the scheduler's own
// functions and reports the lowest and highest element each operand would be touched at, which a CPU test compares
// with the operand shapes.  Everything here is index arithmetic on GemmParams and a Tile; no memory is accessed.
#pragma once
#include "common.hpp"
#include "sched.hpp"

namespace tgg {

constexpr int kGenericBM = 128, kGenericBN = 128, kGenericBK = 32;

// Where a tile's operand windows start (element offsets from the operand pointers) and how many rows / columns
// of the 128 x 128 tile exist.
struct GenericTileIo {
  int64_t a_elem;  // element (tile row 0, k = 0) of A
  int a_lim;       // rows of the tile that may be read
  int64_t b_elem;  // element (tile column 0, k = 0) of the group's B
  int b_lim;       // columns of the tile that may be read
  int64_t c_elem;  // element (tile row 0, column 0 of the output matrix) of C
};

TGG_HD bool generic_kmode(const GemmParams& p) { return p.mode == MODE_KG || p.mode == MODE_KG_COUNT; }

template <bool A_KMAJOR>
TGG_HD GenericTileIo generic_tile_io(const GemmParams& p, const Tile& t) {
  GenericTileIo io;
  // K-grouped: the rows of a tile are columns m of A[Ktot, Mdim] (or rows of x[M, Ktot] when A is K-contiguous)
  io.a_elem = generic_kmode(p) ? (A_KMAJOR ? t.row0 * p.a_sm : t.row0) : t.row0 * p.a_sm;
  io.a_lim = t.rows;
  io.b_elem = (int64_t)t.g * p.b_sg + (int64_t)t.n0 * p.b_sn;
  io.b_lim = (p.N - t.n0) < kGenericBN ? (p.N - t.n0) : kGenericBN;
  io.c_elem = generic_kmode(p) ? ((int64_t)t.g * p.c_sg + t.row0 * p.N) : t.row0 * (int64_t)p.N;
  return io;
}

// Element offset, from an operand window's start, of (row, k): rows K-contiguous (row stride s_row) ...
TGG_HD int64_t generic_elem_kmajor(int row, int64_t s_row, int64_t k) { return (int64_t)row * s_row + k; }
// ... or k rows that are contiguous along the tile's rows / columns (stride s_k between k rows)
TGG_HD int64_t generic_elem_mnmajor(int64_t k, int64_t s_k, int mn) { return k * s_k + mn; }

// Block-scaled epilogue: the 128-deep scale block that ends with K slab kt (slabs are kGenericBK deep)
TGG_HD int generic_scale_block_of_slab(int kt) { return (int)((((int64_t)(kt + 1) * kGenericBK) - 1) >> 7); }
TGG_HD int64_t generic_sb_index(const GemmParams& p, const Tile& t, int kb) {
  const int kblocks = (p.K + 127) >> 7, nblocks = (p.N + 127) >> 7;
  return ((int64_t)t.g * nblocks + (t.n0 >> 7)) * kblocks + kb;
}
TGG_HD int64_t generic_sa_index(const GemmParams& p, const Tile& t, int m, int kb) {
  return (t.row0 + m) * p.sa_rs + kb * p.sa_ks;
}
// Per-channel epilogue: scale of tile row m and of output column n
TGG_HD int64_t generic_scale_m_index(const GemmParams& p, const Tile& t, int m) {
  return generic_kmode(p) ? (int64_t)t.g * p.scale_m_sg + t.row0 + m : t.row0 + m;
}
TGG_HD int64_t generic_scale_n_index(const GemmParams& p, const Tile& t, int n) { return (int64_t)t.g * p.N + n; }

}  // namespace tgg

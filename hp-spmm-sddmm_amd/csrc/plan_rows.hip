// Rows strategy: construction of the row tiles.
#include "host.hpp"

#include "rank_kernels.hpp"
#include "routed_plan_kernels.hpp"
#include "rowtile_kernels.hpp"

namespace hpspmm_host {

// Row tiles (rows strategy): every row cut into slots of 8 nonzeros, 8 slots to a tile, a row's
// slots adjacent in one tile (1 / 2 / 4 / 8 of them for up to 8 / 16 / 32 / 64 nonzeros, tiles
// sorted by that class), longer rows over consecutive tiles, those that get a whole workgroup
// first.  Built on the device (0.2 ms at 100k nonzeros, 0.5 ms at 12 M; on the host it took about
// 3 ms per million nonzeros, after copying the column indices over).  Skipped (the kernel then walks the
// CSR arrays) when padding would blow the layout up, which is what a matrix of mostly empty rows
// does, and beyond kRowTileMaxNnz (rows strategy forced on a very large matrix).
namespace {
constexpr int64_t kRowTilePadFactor = 8;
}  // namespace

// The rows sorted by group (one radix pass over the group numbers, stable: rows of a group stay in
// row order), the tile ranges from the group sizes, then one thread per record of the layout.
int build_row_tiles(hpspmm_plan* p, const int32_t* d_rowptr, const int32_t* d_col, hipStream_t st) {
  using hpspmm::kSlotsPerTile;
  constexpr int kTile = hpspmm::kRowTile;
  constexpr int kGroups = hpspmm::kRowTileGroups;
  const int64_t rows = p->rows, nnz = p->nnz;
  if (rows <= 0) return HPSPMM_OK;

  DeviceTemps tmp;
  const int64_t n_tiles = ceil_div(rows, hpspmm::kSortTile);
  const size_t scan_words = (size_t)std::max(scan_scratch_words(256 * n_tiles), scan_scratch_words(rows + 1));
  for (int i = 0; i < 2; ++i) {
    tmp.room<uint32_t>((size_t)rows);
    tmp.room<int32_t>((size_t)rows);
  }
  tmp.room<uint32_t>((size_t)(256 * n_tiles + 1));
  tmp.room<uint32_t>(scan_words);
  tmp.room<uint32_t>(kGroups + 2);
  tmp.room<uint32_t>((size_t)rows + 1);
  if (int rc = tmp.reserve()) return rc;
  uint32_t* d_keys[2];
  int32_t* d_ids[2];
  for (int i = 0; i < 2; ++i) {
    d_keys[i] = tmp.take<uint32_t>((size_t)rows);
    d_ids[i] = tmp.take<int32_t>((size_t)rows);
  }
  uint32_t* d_hist = tmp.take<uint32_t>((size_t)(256 * n_tiles + 1));
  uint32_t* d_scan = tmp.take<uint32_t>(scan_words);
  uint32_t* d_count = tmp.take<uint32_t>(kGroups + 2);
  uint32_t* d_long = tmp.take<uint32_t>((size_t)rows + 1);  // tiles of the rows with tiles of their own, then their scan

  HPSPMM_HIP(hipMemsetAsync(d_count, 0, (kGroups + 2) * sizeof(uint32_t), st));
  hipLaunchKernelGGL(hpspmm::rowtile_classify_kernel, dim3((unsigned)ceil_div(rows, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                     0, st, rows, nnz, d_rowptr, d_keys[0], d_ids[0], d_count);
  int sorted = 0;
  if (int rc = radix_sort_pairs(rows, d_keys, d_ids, d_hist, d_scan, 8, st, &sorted)) return rc;
  const int32_t* d_order = d_ids[sorted];
  uint32_t cnt[kGroups + 2];
  HPSPMM_HIP(hipMemcpyAsync(cnt, d_count, sizeof cnt, hipMemcpyDeviceToHost, st));
  HPSPMM_HIP(hipStreamSynchronize(st));
  // an unchecked rowptr (HPSPMM_PLAN_NO_VALIDATE) that is not monotone or runs past nnz: no tiles,
  // the CSR kernel is left to the caller's arrays as they are
  if (cnt[kGroups + 1] != 0) return HPSPMM_OK;

  hpspmm::RowTileLayout lay{};
  lay.count[4] = (int64_t)cnt[0] + cnt[1];
  lay.count[3] = cnt[2];
  lay.count[2] = cnt[3];
  lay.count[1] = cnt[4];
  lay.count[0] = 0;
  for (int g = 5; g < kGroups; ++g) lay.count[0] += cnt[g];
  lay.loop_tiles = cnt[kGroups];
  lay.start[4] = 0;
  lay.start[3] = lay.count[4];
  lay.start[2] = lay.start[3] + lay.count[3];
  lay.start[1] = lay.start[2] + lay.count[2];
  lay.start[0] = lay.start[1] + lay.count[1];
  // tile ranges: long rows, then the classes from 8 slots a row down to 1
  const int64_t t3 = lay.count[3], t2 = ceil_div(lay.count[2], 2), t1 = ceil_div(lay.count[1], 4),
                t0 = ceil_div(lay.count[0], 8);
  lay.first[3] = lay.loop_tiles;
  lay.first[2] = lay.loop_tiles + t3;
  lay.first[1] = lay.loop_tiles + t3 + t2;
  lay.first[0] = lay.loop_tiles + t3 + t2 + t1;
  lay.tiles = lay.loop_tiles + t3 + t2 + t1 + t0;
  const int64_t tiles = lay.tiles;
  if (tiles * kTile > kRowTilePadFactor * nnz + (1 << 20) || tiles >= (1 << 24)) return HPSPMM_OK;  // not worth it

  const int64_t n_loop = lay.count[4];
  const size_t bytes_ent = (size_t)tiles * kTile * sizeof(int2);
  const size_t bytes_loop = (size_t)std::max<int64_t>(n_loop, 1) * sizeof(int2);
  if (hipMalloc(&p->d_tent, bytes_ent) != hipSuccess || hipMalloc(&p->d_ldesc, bytes_loop) != hipSuccess ||
      hipMalloc(&p->d_zrow, 36 * sizeof(float)) != hipSuccess) {
    (void)hipGetLastError();
    return fail(HPSPMM_ERR_ALLOC, "device allocation of %zu bytes for the row tiles failed", bytes_ent + bytes_loop);
  }
  p->workspace_bytes += (int64_t)(bytes_ent + bytes_loop + 36 * sizeof(float));
  if (n_loop > 0) {
    hipLaunchKernelGGL(hpspmm::rowtile_long_tiles_kernel, dim3((unsigned)ceil_div(n_loop + 1, hpspmm::kBlock)),
                       dim3(hpspmm::kBlock), 0, st, n_loop, d_order, d_rowptr, d_long);
    if (int rc = exclusive_scan_u32(d_long, d_long, n_loop + 1, st, d_scan)) return rc;
    hipLaunchKernelGGL(hpspmm::rowtile_ldesc_kernel, dim3((unsigned)ceil_div(n_loop, hpspmm::kBlock)), dim3(hpspmm::kBlock),
                       0, st, n_loop, d_long, p->d_ldesc);
  }
  if (tiles > 0)
    hipLaunchKernelGGL(hpspmm::rowtile_fill_kernel, dim3((unsigned)ceil_div(tiles * kTile, hpspmm::kBlock)),
                       dim3(hpspmm::kBlock), 0, st, lay, d_order, p->d_ldesc, d_rowptr, d_col, p->d_tent);
  HPSPMM_HIP(hipMemsetAsync(p->d_zrow, 0, 36 * sizeof(float), st));
  hipError_t e = hipStreamSynchronize(st);  // the temporaries go out of scope
  if (e == hipSuccess) e = hipGetLastError();
  if (e != hipSuccess) return fail(HPSPMM_ERR_HIP, "row tiles: %s", hipGetErrorString(e));
  p->rt_tiles = (int32_t)tiles;
  p->rt_loop = (int32_t)n_loop;
  p->rt_wg = (int32_t)cnt[0];
  p->rt_loop_tiles = (int32_t)lay.loop_tiles;
  p->rt_waves = (int32_t)(n_loop + (tiles - lay.loop_tiles));
  return HPSPMM_OK;
}

}  // namespace hpspmm_host

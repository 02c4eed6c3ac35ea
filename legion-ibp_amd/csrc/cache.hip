// Feature caches: static hot-set, LRU dynamic, int8-compressed; the id->slot
// lookup; and the row gather (HBM rows on hits, zero-copy pinned host rows on
// misses, dequantisation fused for int8 rows).
//
// Reference semantics (Legion-IBP, sampling_server/src):
//   cache/cache_impl.cuh:239-303        gather: row i of the output belongs to ids[i];
//                                       hit -> cache row, miss -> host row of the id
//   cache/cache.cu:314-338              FindFeat: id -> slot for one frontier segment
//   cache/cache.cu:559-656              FillUp: choose rows, copy them, build the map
//   comp_cache/static_cache_kernel.cuh:6-29,185-266   set = id mod n_sets, ways contiguous
// What differs on purpose: hot set = top rows by (out-degree desc, id asc) found
// with a threshold search and two scans (no sort, no presampling); our own
// open-addressing table (or a direct map) instead of the vendored cuckoo table;
// a batch-synchronous LRU (the reference's LRU source is absent); int8 + per-row
// scale instead of the un-vendored lossless codec; one lane moves 16 bytes and
// several rows are in flight per lane instead of one float per thread.
#include <algorithm>
#include <vector>

#include <hip/hip_ext.h>

#include "scan.hpp"

namespace lmi {

// ------------------------------------------------------------------ gather
// Generic row mover over work items j in [*first_ptr, *n_ptr).  Entry j of the work
// list is a pair (output row i, source row); without a list i = j.  With SRC_FROM_LIST the source row is the pair's
// second word, so the only dependent load in front of the row itself is the pair;
// otherwise it is src_index[i] (or i).  The destination row is dst_index[i] (or
// i); a negative source or destination skips the row.  LPR lanes cooperate on a
// row, each moving sizeof(V) bytes per step, with U rows in flight per lane.
// HOSTLINK only names the instantiation that reads over the host link, so that
// profiles list the HBM gather and the host-link gather as two kernels.
// One launch can serve several pipes (output buffers): their blocks interleave over
// blockIdx.x like those of the sampling kernels, and the source table is shared.
struct MoveRow {
  const int2 *list;
  const int32_t *first_ptr, *n_ptr, *src_index, *dst_index;
  uint8_t *dst;
};
struct MoveGroup {
  MoveRow p[LMI_MAX_GROUP];
  int n;
};

template <typename V, int LPR, int U, bool NT, bool HOSTLINK>
static __global__ __launch_bounds__(256) void move_rows_kernel(
    MoveGroup g, int src_from_list, const uint8_t *src, int chunks, int64_t src_row_bytes, int64_t dst_row_bytes,
    unsigned long long *row_counter) {
  LMI_GRID_ROW(g.n);
  const MoveRow &r = g.p[row];
  const int2 *list = r.list;
  const int32_t *src_index = r.src_index, *dst_index = r.dst_index;
  uint8_t *dst = r.dst;
  const int n = *r.n_ptr;
  const int first = r.first_ptr ? *r.first_ptr : 0;
  if (row_counter && bx == 0 && threadIdx.x == 0 && n > first)
    atomicAdd(row_counter, (unsigned long long)(n - first));  // work items offered to this launch (profiling)
  const int lane = threadIdx.x & (LPR - 1);
  const int group = (bx * blockDim.x + threadIdx.x) / LPR;
  const int n_groups = gx * blockDim.x / LPR;
  for (int j0 = first + group; j0 < n; j0 += n_groups * U) {
    int64_t so[U], dofs[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = j0 + u * n_groups;
      so[u] = -1;
      dofs[u] = -1;
      if (j < n) {
        int i = j, si;
        if (list) {
          const int2 pr = list[j];
          i = pr.x;
          si = pr.y;
        }
        if (!list || !src_from_list) si = src_index ? src_index[i] : i;
        const int di = dst_index ? dst_index[i] : i;
        if (si >= 0 && di >= 0) {
          so[u] = (int64_t)si * src_row_bytes;
          dofs[u] = (int64_t)di * dst_row_bytes;
        }
      }
    }
    for (int c = lane; c < chunks; c += LPR) {
      V v[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (so[u] >= 0) v[u] = __builtin_nontemporal_load(reinterpret_cast<const V *>(src + so[u] + (int64_t)c * sizeof(V)));
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (so[u] >= 0) {
          V *d = reinterpret_cast<V *>(dst + dofs[u] + (int64_t)c * sizeof(V));
          if (NT) __builtin_nontemporal_store(v[u], d);
          else *d = v[u];
        }
    }
  }
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));  // a 16-byte access at a 4-byte-aligned address

// Row mover for rows that a power-of-two lane group does not fit: 400-byte rows (25 chunks of
// 16 bytes would leave 7 of 32 lanes idle), rows that are no multiple of 16 bytes, rows whose
// start is only 4-byte aligned.  A row is `cpr` 16-byte units followed by `tail` 4-byte units.
// A block takes a tile of TILE consecutive work items in two steps.  Staging: one thread per
// work item resolves it (list entry, source row, destination row: the only dependent loads)
// and the items that have something to move -- cache hits, when the source index is the
// cache slot -- are compacted into LDS by ballot + prefix popcount, as (source offset,
// destination offset) pairs.  Moving: the 256 threads walk the units of the staged rows in
// flat order, unit f = staged row f / units, place f % units inside it, offsets from LDS, so
// every lane of every pass but the last has a unit, misses cost no lanes, and the row loads
// of a pass depend on nothing but LDS.  Consecutive lanes touch consecutive bytes of a row,
// and of the next row when the destination rows are contiguous.  V16 says whether the 16-byte
// accesses may assume 16-byte alignment.  Work items, lists and index arrays mean what they
// mean in move_rows_kernel.
constexpr int kTileWaves = 4;  // wavefronts of a 256-thread block
template <typename V16, int TILE, int U, bool NT, bool HOSTLINK>
static __global__ __launch_bounds__(256) void move_rows_tiled_kernel(
    MoveGroup g, int src_from_list, const uint8_t *src, int cpr, int tail, int tile_rows, int64_t src_row_bytes,
    int64_t dst_row_bytes, unsigned long long *row_counter) {
  static_assert(TILE == 64 || TILE == 256, "a tile is at most one work item per lane of one wavefront, or of the block");
  __shared__ int64_t s_src[TILE], s_dst[TILE];
  __shared__ int s_cnt[kTileWaves];
  LMI_GRID_ROW(g.n);
  const MoveRow &r = g.p[row];
  const int2 *list = r.list;
  const int32_t *src_index = r.src_index, *dst_index = r.dst_index;
  uint8_t *dst = r.dst;
  const int n = *r.n_ptr;
  const int first = r.first_ptr ? *r.first_ptr : 0;
  if (row_counter && bx == 0 && threadIdx.x == 0 && n > first)
    atomicAdd(row_counter, (unsigned long long)(n - first));  // work items offered to this launch (profiling)
  const int units = cpr + tail;
  const int dq = 256 / units, dr = 256 % units;  // what 256 units further means in (row, place)
  const int r0 = (int)threadIdx.x / units, u0 = (int)threadIdx.x % units;
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
  const int n_tiles = (n - first + tile_rows - 1) / tile_rows;  // tile_rows <= TILE
  for (int tile = bx; tile < n_tiles; tile += gx) {
    // ---- staging
    bool ok = false;
    int64_t so = 0, dof = 0;
    if ((int)threadIdx.x < tile_rows) {
      const int j = first + tile * tile_rows + (int)threadIdx.x;
      if (j < n) {
        int i = j, si;
        if (list) {
          const int2 pr = list[j];
          i = pr.x;
          si = pr.y;
        }
        if (!list || !src_from_list) si = src_index ? src_index[i] : i;
        const int di = dst_index ? dst_index[i] : i;
        ok = si >= 0 && di >= 0;
        so = (int64_t)si * src_row_bytes;
        dof = (int64_t)di * dst_row_bytes;
      }
    }
    int n_rows;
    if (TILE == 64) {
      if (wid == 0) {
        const uint64_t m = __ballot(ok);
        if (ok) {
          const int pos = __popcll(m & lanemask_lt());
          s_src[pos] = so;
          s_dst[pos] = dof;
        }
        if (lane == 0) s_cnt[0] = __popcll(m);
      }
      __syncthreads();
      n_rows = s_cnt[0];
    } else {
      const uint64_t m = __ballot(ok);
      if (lane == 0) s_cnt[wid] = __popcll(m);
      __syncthreads();
      int base = 0, total = 0;
#pragma unroll
      for (int w = 0; w < kTileWaves; ++w) {
        const int c = s_cnt[w];
        if (w < wid) base += c;
        total += c;
      }
      if (ok) {
        const int pos = base + __popcll(m & lanemask_lt());
        s_src[pos] = so;
        s_dst[pos] = dof;
      }
      __syncthreads();
      n_rows = total;
    }
    // ---- moving
    const int lim = n_rows * units;
    int rr = r0, uu = u0;
    for (int f0 = threadIdx.x; f0 < lim; f0 += 256 * U) {
      int64_t sa[U], da[U];
      int kind[U];  // 0: nothing, 1: 16 bytes, 2: 4 bytes
#pragma unroll
      for (int q = 0; q < U; ++q) {
        kind[q] = 0;
        if (f0 + q * 256 < lim) {
          const int off = uu < cpr ? 16 * uu : 16 * cpr + 4 * (uu - cpr);
          sa[q] = s_src[rr] + off;
          da[q] = s_dst[rr] + off;
          kind[q] = uu < cpr ? 1 : 2;
        }
        uu += dr;
        rr += dq;
        if (uu >= units) {
          uu -= units;
          ++rr;
        }
      }
      V16 v[U];
      uint32_t w[U];
#pragma unroll
      for (int q = 0; q < U; ++q) {
        if (kind[q] == 1) v[q] = __builtin_nontemporal_load(reinterpret_cast<const V16 *>(src + sa[q]));
        else if (kind[q] == 2) w[q] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(src + sa[q]));
      }
#pragma unroll
      for (int q = 0; q < U; ++q) {
        if (kind[q] == 1) {
          V16 *d = reinterpret_cast<V16 *>(dst + da[q]);
          if (NT) __builtin_nontemporal_store(v[q], d);
          else *d = v[q];
        } else if (kind[q] == 2) {
          uint32_t *d = reinterpret_cast<uint32_t *>(dst + da[q]);
          if (NT) __builtin_nontemporal_store(w[q], d);
          else *d = w[q];
        }
      }
    }
    __syncthreads();  // the next tile's staging overwrites the offsets
  }
}

// The HBM gather of cache hits, for fp32 / fp16 rows of every size from 16 bytes up.  Output rows [first, n)
// directly, source row = src_index[row] (a cache slot; negative = a miss, skipped).  A block takes a
// tile of consecutive rows and its 256 threads walk the tile's 16-byte units in flat order -- unit f is
// piece f % upr of row f / upr -- U units per lane and pass: the U slots (lanes of one row read the
// same word: one cache line per wavefront), then the U row pieces, then the U stores, each step
// issued whole before the next waits.  Lanes without a unit, or whose row is a miss, issue nothing
// (every access they would make costs the memory pipeline a cycle whether or not HBM sees it).
// Nothing else stands between a block and its bytes: no LDS, no barrier.  Measured against the same
// loop with computed source rows on one output buffer, this shape keeps 90 % of its rate; staging a
// tile's rows through LDS first kept 70 %.  A row that is no multiple of 16 bytes ends with a unit
// that overlaps the one before it (both write the same bytes), so every access is 16 bytes wide, at
// 4-byte alignment when the row length demands it (V16 says which).
// rows_seen (pinned host memory, or null): the launch leaves each pipe's row count there for the host
// to size later grids by (see launch_gather_flat).
template <typename V16, int U, bool NT>
static __global__ __launch_bounds__(256) void gather_rows_flat_kernel(MoveGroup g, const uint8_t *__restrict__ src,
                                                                      int upr, int last_off, int rows_per_tile,
                                                                      int64_t src_pitch, int64_t dst_pitch,
                                                                      unsigned long long *row_counter,
                                                                      int32_t *rows_seen) {
  LMI_GRID_ROW(g.n);
  const MoveRow &r = g.p[row];
  const int32_t *__restrict__ src_index = r.src_index;
  uint8_t *__restrict__ dst = r.dst;
  const int n = *r.n_ptr;
  const int first = r.first_ptr ? *r.first_ptr : 0;
  if (bx == 0 && threadIdx.x == 0) {
    if (row_counter && n > first) atomicAdd(row_counter, (unsigned long long)(n - first));  // profiling
    if (rows_seen) rows_seen[row] = n - first;
  }
  const int dq = (256 * 1) / upr, dr = 256 % upr;  // what 256 units further means in (row, piece)
  const int r0 = (int)threadIdx.x / upr, u0 = (int)threadIdx.x % upr;
  const int n_tiles = (n - first + rows_per_tile - 1) / rows_per_tile;
  for (int tile = bx; tile < n_tiles; tile += gx) {
    const int row0 = first + tile * rows_per_tile;
    const int nr = n - row0 < rows_per_tile ? n - row0 : rows_per_tile;
    const int lim = nr * upr;
    int rr = r0, uu = u0;
    for (int f0 = threadIdx.x; f0 < lim; f0 += 256 * U) {
      int slot[U], off[U];
      int64_t da[U];
      V16 v[U];
#pragma unroll
      for (int k = 0; k < U; ++k) {
        const int i = row0 + rr;
        slot[k] = f0 + 256 * k < lim ? src_index[i] : -1;
        off[k] = (uu == upr - 1) ? last_off : 16 * uu;
        da[k] = (int64_t)i * dst_pitch + off[k];
        uu += dr;
        rr += dq;
        if (uu >= upr) {
          uu -= upr;
          ++rr;
        }
      }
#pragma unroll
      for (int k = 0; k < U; ++k)
        if (slot[k] >= 0)
          v[k] = __builtin_nontemporal_load(reinterpret_cast<const V16 *>(src + (int64_t)slot[k] * src_pitch + off[k]));
#pragma unroll
      for (int k = 0; k < U; ++k)
        if (slot[k] >= 0) {
          V16 *d = reinterpret_cast<V16 *>(dst + da[k]);
          if (NT) __builtin_nontemporal_store(v[k], d);
          else *d = v[k];
        }
    }
  }
}

// Grid of a gather whose real row count only the device knows.  The worst case of a batch is about
// ten times what a batch holds, and a block that finds no tile is not free: the device starts about one
// workgroup per clock, so the 8 000 idle blocks of a worst-case grid cost a 40 us launch a seventh of
// its time.  The gather kernels leave the row count of every launch in pinned host memory
// (rows_seen); the largest of the last launch, with an eighth on top, sizes the next grid.  The
// kernels stride over their tiles by the grid, so a grid that turns out small is slower, not wrong.
static int64_t hinted_rows(Server *s, int64_t n_max) {
  if (!s->rows_seen_host || !s->gather_adaptive) return n_max;
  int32_t seen = 0;
  for (int k = 0; k < LMI_MAX_GROUP; ++k) {
    const int32_t v = s->rows_seen_host[k];
    seen = v > seen ? v : seen;
  }
  if (seen <= 0) return n_max;  // nothing seen yet
  return std::min<int64_t>(n_max, (int64_t)seen + seen / 8 + 64);
}

struct MoveArgs {
  MoveGroup g;     // per pipe: work list, bounds, index arrays, destination
  int src_from_list;
  int max_blocks;  // per pipe; 0 = fill the device
  int unroll;      // 0 = the server's gather_unroll
  int host_link;   // the source is pinned host memory read over the host link
  unsigned long long *row_counter;  // device counter that receives the number of work items, or null
  hipEvent_t ev_start, ev_stop;     // stamped with the kernel's begin and end when not null (profiling)
  const uint8_t *src;
  int64_t src_row_bytes, dst_row_bytes, row_bytes;  // row_bytes = bytes moved per row
  int64_t n_max;   // per pipe
};

template <typename V, int LPR, int U>
static void launch_move_vlu(hipStream_t st, const MoveArgs &a, int grid, bool nt) {
  const int chunks = (int)(a.row_bytes / sizeof(V));
  // with profiling on, the launch carries its own start / stop events
#define LMI_MOVE(NT_, HL_)                                                                                      \
  if (a.ev_start)                                                                                               \
    hipExtLaunchKernelGGL((move_rows_kernel<V, LPR, U, NT_, HL_>), dim3(grid * a.g.n), dim3(256), 0, st,         \
                          a.ev_start, a.ev_stop, 0, a.g, a.src_from_list, a.src, chunks, a.src_row_bytes,        \
                          a.dst_row_bytes, a.row_counter);                                                       \
  else                                                                                                          \
    hipLaunchKernelGGL((move_rows_kernel<V, LPR, U, NT_, HL_>), dim3(grid * a.g.n), dim3(256), 0, st, a.g,       \
                       a.src_from_list, a.src, chunks, a.src_row_bytes, a.dst_row_bytes, a.row_counter)
  if (a.host_link) {
    LMI_MOVE(true, true);
  } else if (nt) {
    LMI_MOVE(true, false);
  } else {
    LMI_MOVE(false, false);
  }
#undef LMI_MOVE
}

template <typename V, int LPR>
static void launch_move_vl(hipStream_t st, const MoveArgs &a, int grid, bool nt, int unroll) {
  switch (unroll) {
    case 1: launch_move_vlu<V, LPR, 1>(st, a, grid, nt); break;
    case 2: launch_move_vlu<V, LPR, 2>(st, a, grid, nt); break;
    case 8: launch_move_vlu<V, LPR, 8>(st, a, grid, nt); break;
    default: launch_move_vlu<V, LPR, 4>(st, a, grid, nt); break;
  }
}

template <typename V>
static void launch_move_v(hipStream_t st, const MoveArgs &a, int grid, bool nt, int unroll, int lpr) {
  switch (lpr) {
    case 1: launch_move_vl<V, 1>(st, a, grid, nt, unroll); break;  // thread per row (measurement only)
    case 4: launch_move_vl<V, 4>(st, a, grid, nt, unroll); break;
    case 8: launch_move_vl<V, 8>(st, a, grid, nt, unroll); break;
    case 16: launch_move_vl<V, 16>(st, a, grid, nt, unroll); break;
    case 32: launch_move_vl<V, 32>(st, a, grid, nt, unroll); break;
    default: launch_move_vl<V, 64>(st, a, grid, nt, unroll); break;
  }
}

// Grid of an HBM gather whose worst case needs `want` blocks: a sixteenth of that, between 8
// and 64 blocks per CU.
static int64_t auto_gather_blocks(const Server *s, int64_t want) {
  return std::min<int64_t>(std::max<int64_t>(want / 16, (int64_t)s->n_cu * 8), (int64_t)s->n_cu * 64);
}

template <typename V16, int TILE, int U>
static void launch_tiled_vtu(hipStream_t st, const MoveArgs &a, int grid, bool nt, int cpr, int tail, int tile_rows) {
#define LMI_TILED(NT_, HL_)                                                                                         \
  if (a.ev_start)                                                                                                   \
    hipExtLaunchKernelGGL((move_rows_tiled_kernel<V16, TILE, U, NT_, HL_>), dim3(grid * a.g.n), dim3(256), 0, st,    \
                          a.ev_start, a.ev_stop, 0, a.g, a.src_from_list, a.src, cpr, tail, tile_rows,              \
                          a.src_row_bytes, a.dst_row_bytes, a.row_counter);                                          \
  else                                                                                                              \
    hipLaunchKernelGGL((move_rows_tiled_kernel<V16, TILE, U, NT_, HL_>), dim3(grid * a.g.n), dim3(256), 0, st, a.g,  \
                       a.src_from_list, a.src, cpr, tail, tile_rows, a.src_row_bytes, a.dst_row_bytes, a.row_counter)
  if (a.host_link) {
    LMI_TILED(true, true);
  } else if (nt) {
    LMI_TILED(true, false);
  } else {
    LMI_TILED(false, false);
  }
#undef LMI_TILED
}

template <typename V16, int TILE>
static void launch_tiled_vt(hipStream_t st, const MoveArgs &a, int grid, bool nt, int cpr, int tail, int tile_rows,
                            int unroll) {
  if (unroll >= 4) launch_tiled_vtu<V16, TILE, 4>(st, a, grid, nt, cpr, tail, tile_rows);
  else if (unroll >= 2) launch_tiled_vtu<V16, TILE, 2>(st, a, grid, nt, cpr, tail, tile_rows);
  else launch_tiled_vtu<V16, TILE, 1>(st, a, grid, nt, cpr, tail, tile_rows);
}

// Rows of a tile of the tiled movers: about 8 KB of rows, so that a batch of long rows still
// makes thousands of tiles and short tiles even out the blocks that run beside host-link reads;
// between 2 and 64 (a wavefront stages them), or the block's 256 when rows are so short that 64
// of them do not give every thread a unit.  Measured, share of HBM peak: 400-byte rows 16 rows
// 47 %, 32 44 %, 64 42 %; 5 732-byte rows 2 rows 52 %, 4 48 %, 8 49 %, 16 41 %.
static int tiled_tile_rows(Server *s, int64_t row_bytes) {
  if (s->gather_tile_rows > 0) return std::min(s->gather_tile_rows, row_bytes < 128 ? 256 : 64);
  if (row_bytes < 128) return 256;
  int t = 64;
  while (t > 2 && (int64_t)t * row_bytes > 8192) t >>= 1;
  return t;
}

// Rows per tile of the flat gather: about 8 KB worth of rows, two at least.
static int launch_gather_flat(Server *s, hipStream_t st, const MoveArgs &a, bool nt, bool aligned16) {
  const int upr = (int)((a.row_bytes + 15) / 16);
  const int last_off = (int)a.row_bytes - 16;
  const int u_want = s->gather_unroll > 0 ? s->gather_unroll : 2;
  const int U = u_want >= 4 ? 4 : u_want >= 2 ? 2 : 1;
  int rpt = (int)std::max<int64_t>(2, std::min<int64_t>(64, 8192 / a.row_bytes));
  if (s->gather_tile_rows > 0) rpt = std::min(s->gather_tile_rows, 256);
  const int64_t want = ceil_div(hinted_rows(s, a.n_max), rpt);
  const int64_t cap = a.max_blocks > 0 ? a.max_blocks : s->gather_blocks > 0 ? s->gather_blocks : (int64_t)s->n_cu * 64;
  const int grid = (int)std::max<int64_t>(1, std::min(want, cap));
#define LMI_FLAT(V_, U_, NT_)                                                                                          \
  if (a.ev_start)                                                                                                      \
    hipExtLaunchKernelGGL((gather_rows_flat_kernel<V_, U_, NT_>), dim3(grid * a.g.n), dim3(256), 0, st, a.ev_start,     \
                          a.ev_stop, 0, a.g, a.src, upr, last_off, rpt, a.src_row_bytes, a.dst_row_bytes,              \
                          a.row_counter, s->rows_seen_dev);                                                            \
  else                                                                                                                 \
    hipLaunchKernelGGL((gather_rows_flat_kernel<V_, U_, NT_>), dim3(grid * a.g.n), dim3(256), 0, st, a.g, a.src, upr,   \
                       last_off, rpt, a.src_row_bytes, a.dst_row_bytes, a.row_counter, s->rows_seen_dev)
#define LMI_FLAT_U(V_, NT_)                 \
  if (U == 4) { LMI_FLAT(V_, 4, NT_); }     \
  else if (U == 2) { LMI_FLAT(V_, 2, NT_); } \
  else { LMI_FLAT(V_, 1, NT_); }
  if (aligned16 && nt) { LMI_FLAT_U(u32x4, true) }
  else if (aligned16) { LMI_FLAT_U(u32x4, false) }
  else if (nt) { LMI_FLAT_U(u32x4_a4, true) }
  else { LMI_FLAT_U(u32x4_a4, false) }
#undef LMI_FLAT_U
#undef LMI_FLAT
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

static int launch_move_rows_tiled(Server *s, hipStream_t st, const MoveArgs &a, bool nt, bool aligned16) {
  const int cpr = (int)(a.row_bytes / 16), tail = (int)(a.row_bytes % 16) / 4;
  const int tile = tiled_tile_rows(s, a.row_bytes);
  const int64_t want = ceil_div(a.n_max, tile);
  const int64_t cap = a.max_blocks > 0 ? a.max_blocks : s->gather_blocks > 0 ? s->gather_blocks : auto_gather_blocks(s, want);
  const int grid = (int)std::max<int64_t>(1, std::min(want, cap));
  // two units in flight per lane unless the caller or the knob says otherwise (400-byte rows: 1 -> 42 %
  // of HBM peak, 2 -> 44 %, 4 -> 34 %)
  const int unroll = a.unroll > 0 ? a.unroll : s->gather_unroll > 0 ? s->gather_unroll : 2;
  if (aligned16 && tile <= 64) launch_tiled_vt<u32x4, 64>(st, a, grid, nt, cpr, tail, tile, unroll);
  else if (aligned16) launch_tiled_vt<u32x4, 256>(st, a, grid, nt, cpr, tail, tile, unroll);
  else if (tile <= 64) launch_tiled_vt<u32x4_a4, 64>(st, a, grid, nt, cpr, tail, tile, unroll);
  else launch_tiled_vt<u32x4_a4, 256>(st, a, grid, nt, cpr, tail, tile, unroll);
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

// Picks the widest vector that divides the row and all base addresses, and a
// power-of-two lane group that covers one row when possible; rows such a group does not
// fit exactly go to the tiled mover.
static int launch_move_rows(Server *s, hipStream_t st, const MoveArgs &a, bool nt) {
  if (a.n_max <= 0 || a.row_bytes <= 0) return LMI_OK;
  if (a.g.n < 1 || a.g.n > LMI_MAX_GROUP) LMI_FAIL(LMI_ERR_ARG, "a row move serves 1..LMI_MAX_GROUP pipes");
  uintptr_t align = (uintptr_t)a.src | (uintptr_t)a.src_row_bytes | (uintptr_t)a.dst_row_bytes | (uintptr_t)a.row_bytes;
  for (int k = 0; k < a.g.n; ++k) align |= (uintptr_t)a.g.p[k].dst;
  int vec = (align % 16 == 0) ? 16 : (align % 8 == 0) ? 8 : 4;
  if (align % 4 != 0) LMI_FAIL(LMI_ERR_ARG, "feature rows must be 4-byte aligned");
  {
    // a lane group fits exactly when the row is 8, 16, 32 or 64 aligned 16-byte chunks (128 .. 1024 bytes)
    const int64_t c16 = a.row_bytes / 16;
    const bool exact = vec == 16 && (c16 == 8 || c16 == 16 || c16 == 32 || c16 == 64);
    const bool knobs = s->gather_vec != 0 || (s->gather_lpr != 0 && !a.host_link);  // measurement knobs of the lane-group mover
    // HBM gather (gather_flat): 0 or 3 the flat gather, 1 the LDS-tiled mover, 2 lane groups; host-link
    // gather (miss_flat): the LDS-tiled mover 0 when no lane group fits, 1 always, 2 never
    const int flat = a.host_link ? s->miss_flat : s->gather_flat;
    bool direct = !a.host_link && a.row_bytes >= 16;  // rows walked directly, source row = src_index[row]: the hits
    for (int k = 0; k < a.g.n; ++k) direct = direct && !a.g.p[k].list && a.g.p[k].src_index && !a.g.p[k].dst_index;
    if (direct && !knobs && (flat == 0 || flat == 3)) return launch_gather_flat(s, st, a, nt, vec == 16);
    if (a.row_bytes >= 16 && (flat == 1 || (flat == 0 && !exact && !knobs)))
      return launch_move_rows_tiled(s, st, a, nt, vec == 16);
  }
  if (s->gather_vec == 4 || (s->gather_vec == 8 && vec == 16)) vec = s->gather_vec;  // narrower on request
  const int64_t chunks = a.row_bytes / vec;
  int lpr = a.host_link ? 0 : s->gather_lpr;  // the knob is about the HBM gather
  if (lpr != 1 && lpr != 4 && lpr != 8 && lpr != 16 && lpr != 32 && lpr != 64) {
    lpr = 8;
    while (lpr < chunks && lpr < 64) lpr <<= 1;
  }
  const int unroll = a.unroll > 0 ? a.unroll : s->gather_unroll > 0 ? s->gather_unroll : 1;
  const int64_t groups_per_block = 256 / lpr;
  int64_t want = ceil_div(a.n_max, groups_per_block * (unroll > 0 ? unroll : 1));
  // Many small blocks rather than one resident wave of them: blocks that run beside host-link reads
  // are slowed unevenly, and the dispatcher evens that out (paper100m-shaped, 4 batches per launch:
  // 8 blocks per CU and pipe 62 % of HBM peak, 32 66 %, 64 67 %, 128 66 %, 256 57 %).  A batch holds
  // about a tenth of its worst-case rows, and blocks without rows are not free (products-shaped:
  // 40 % of peak on 2048 blocks per pipe, 36 % on 16384), hence the sixteenth.
  int64_t cap = a.max_blocks > 0 ? a.max_blocks : s->gather_blocks > 0 ? s->gather_blocks : auto_gather_blocks(s, want);
  const int grid = (int)std::max<int64_t>(1, std::min(want, cap));
  if (vec == 16) launch_move_v<u32x4>(st, a, grid, nt, unroll, lpr);
  else if (vec == 8) launch_move_v<u32x2>(st, a, grid, nt, unroll, lpr);
  else launch_move_v<uint32_t>(st, a, grid, nt, unroll, lpr);
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

// ------------------------------------------------------------- int8 codec
__device__ __forceinline__ float load_elem(const uint8_t *row, int i, int dtype) {
  if (dtype == LMI_F16) return __half2float(reinterpret_cast<const __half *>(row)[i]);
  return reinterpret_cast<const float *>(row)[i];
}

// One wavefront per row: absmax over the row, scale = absmax / 127,
// q = clamp(rint(x / scale), -127, 127).  Build-time only, so the source row
// (usually in pinned host memory) is read twice rather than staged.
static __global__ __launch_bounds__(256) void quantize_rows_kernel(
    const int32_t *row_ids, int64_t n_rows, const uint8_t *feat, int dim, int dtype, int64_t row_bytes,
    int8_t *q, float *scale) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
  const int64_t n_waves = (int64_t)gridDim.x * blockDim.x / kWave;
  for (int64_t r = wave; r < n_rows; r += n_waves) {
    const uint8_t *row = feat + (int64_t)row_ids[r] * row_bytes;
    float a = 0.0f;
    for (int i = lane; i < dim; i += kWave) a = fmaxf(a, fabsf(load_elem(row, i, dtype)));
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) a = fmaxf(a, __shfl_xor(a, d, kWave));
    const float sc = a / 127.0f;
    if (lane == 0) scale[r] = sc;
    for (int i = lane; i < dim; i += kWave) {
      float v = (a == 0.0f) ? 0.0f : rintf(load_elem(row, i, dtype) / sc);
      v = fminf(127.0f, fmaxf(-127.0f, v));
      q[r * dim + i] = (int8_t)v;
    }
  }
}

// y = float(q) * scale for the four int8 values packed in `w`, bit for bit what
// __fmul_rn((float)q, scale) gives, in two instructions per element instead of three:
// the byte, biased by 128, converts as an unsigned byte in one instruction, and one fused
// multiply-add takes the bias out again -- (q + 128) * scale - 128 * scale is q * scale
// exactly before the single rounding, because 128 * scale is exact (a power of two; the
// caller takes the plain path when it would overflow).
__device__ __forceinline__ void dequant4(uint32_t w, float sc, float bias /* -128 * sc */, bool plain, float y[4]) {
  if (plain) {
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = __fmul_rn((float)(int8_t)((w >> (e * 8)) & 0xFF), sc);
    return;
  }
  const uint32_t u = w ^ 0x80808080u;
  y[0] = __fmaf_rn((float)(u & 0xFFu), sc, bias);
  y[1] = __fmaf_rn((float)((u >> 8) & 0xFFu), sc, bias);
  y[2] = __fmaf_rn((float)((u >> 16) & 0xFFu), sc, bias);
  y[3] = __fmaf_rn((float)(u >> 24), sc, bias);
}

// Dequantising gather for hits of the int8 cache, 16 elements per lane:
// y = float(q) * scale, rounded to the output type (RNE for fp16).
// Like the row mover, one launch serves several pipes (MoveGroup: src_index = slot per row,
// dst = the pipe's output rows).
template <typename OUT, int LPR>
static __global__ __launch_bounds__(256) void gather_int8_kernel(MoveGroup g, const int8_t *q, const float *scale,
                                                                 int dim, unsigned long long *row_counter) {
  LMI_GRID_ROW(g.n);
  const int32_t *cache_index = g.p[row].src_index;
  OUT *out = reinterpret_cast<OUT *>(g.p[row].dst);
  const int n = *g.p[row].n_ptr;
  const int first = g.p[row].first_ptr ? *g.p[row].first_ptr : 0;
  if (row_counter && bx == 0 && threadIdx.x == 0 && n > first)
    atomicAdd(row_counter, (unsigned long long)(n - first));
  const int lane = threadIdx.x & (LPR - 1);
  const int group = (bx * blockDim.x + threadIdx.x) / LPR;
  const int n_groups = gx * blockDim.x / LPR;
  const int chunks = dim / 16;
  for (int i = first + group; i < n; i += n_groups) {
    const int slot = cache_index[i];
    if (slot < 0) continue;
    const float sc = scale[slot];
    const bool plain = !(sc < 1.0e30f);  // 128 * scale must stay finite (also catches a NaN scale)
    const float bias = -128.0f * sc;
    const int8_t *src = q + (int64_t)slot * dim;
    OUT *dst = out + (int64_t)i * dim;
    for (int c = lane; c < chunks; c += LPR) {
      const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c * 16));
      union alignas(16) {
        OUT y[16];
        u32x4 v[sizeof(OUT)];
      } pk;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float f[4];
        dequant4(w[k], sc, bias, plain, f);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (sizeof(OUT) == 2) pk.y[4 * k + e] = __float2half_rn(f[e]);
          else pk.y[4 * k + e] = f[e];
        }
      }
      u32x4 *d4 = reinterpret_cast<u32x4 *>(dst + c * 16);
#pragma unroll
      for (int k = 0; k < (int)sizeof(OUT); ++k) __builtin_nontemporal_store(pk.v[k], d4 + k);
    }
  }
}

// The same gather in the shape of move_rows_tiled_kernel: the hits of a tile of 64 rows are
// staged in LDS as (output row, slot, scale), then the block walks their EPL-element units in
// flat order.  EPL = 16 / sizeof(OUT) makes every lane's output one 16-byte store and a
// wavefront's store one contiguous kilobyte.  U units in flight per lane.
template <int BYTES> struct RawVec;
template <> struct RawVec<16> { typedef u32x4 type; };
template <> struct RawVec<8> { typedef u32x2 type; };
template <> struct RawVec<4> { typedef uint32_t type; };

template <typename OUT, int EPL, int U>
static __global__ __launch_bounds__(256) void gather_int8_tiled_kernel(MoveGroup g, const int8_t *q, const float *scale,
                                                                       int dim, int tile_rows,
                                                                       unsigned long long *row_counter,
                                                                       int32_t *rows_seen) {
  typedef typename RawVec<EPL>::type IN;
  constexpr int OUT_VECS = EPL * (int)sizeof(OUT) / 16;
  constexpr int TILE = 64;
  __shared__ int s_row[TILE], s_slot[TILE];
  __shared__ float s_scale[TILE];
  __shared__ int s_cnt;
  LMI_GRID_ROW(g.n);
  const int32_t *cache_index = g.p[row].src_index;
  OUT *out = reinterpret_cast<OUT *>(g.p[row].dst);
  const int n = *g.p[row].n_ptr;
  const int first = g.p[row].first_ptr ? *g.p[row].first_ptr : 0;
  if (bx == 0 && threadIdx.x == 0) {
    if (row_counter && n > first) atomicAdd(row_counter, (unsigned long long)(n - first));
    if (rows_seen) rows_seen[row] = n - first;  // for the host to size the next grids by (hinted_rows)
  }
  const int units = dim / EPL;
  const int dq = 256 / units, dr = 256 % units;
  const int r0 = (int)threadIdx.x / units, u0 = (int)threadIdx.x % units;
  const int n_tiles = (n - first + tile_rows - 1) / tile_rows;  // tile_rows <= TILE
  for (int tile = bx; tile < n_tiles; tile += gx) {
    if (threadIdx.x < TILE) {
      const int i = first + tile * tile_rows + (int)threadIdx.x;
      const int slot = ((int)threadIdx.x < tile_rows && i < n) ? cache_index[i] : -1;
      const uint64_t m = __ballot(slot >= 0);
      if (slot >= 0) {
        const int pos = __popcll(m & lanemask_lt());
        s_row[pos] = i;
        s_slot[pos] = slot;
        s_scale[pos] = scale[slot];
      }
      if (threadIdx.x == 0) s_cnt = __popcll(m);
    }
    __syncthreads();
    const int lim = s_cnt * units;
    int rr = r0, uu = u0;
    for (int f0 = threadIdx.x; f0 < lim; f0 += 256 * U) {
      int at[U], c[U];
      bool on[U];
#pragma unroll
      for (int k = 0; k < U; ++k) {
        on[k] = f0 + k * 256 < lim;
        at[k] = rr;
        c[k] = uu;
        uu += dr;
        rr += dq;
        if (uu >= units) {
          uu -= units;
          ++rr;
        }
      }
      union {
        IN v;
        uint32_t w[EPL / 4];
      } in[U];
#pragma unroll
      for (int k = 0; k < U; ++k)
        if (on[k])
          in[k].v = __builtin_nontemporal_load(reinterpret_cast<const IN *>(q + (int64_t)s_slot[at[k]] * dim + c[k] * EPL));
#pragma unroll
      for (int k = 0; k < U; ++k)
        if (on[k]) {
          union alignas(16) {
            OUT y[EPL];
            u32x4 v[OUT_VECS];
          } pk;
          const float sc = s_scale[at[k]];
          const bool plain = !(sc < 1.0e30f);
          const float bias = -128.0f * sc;
#pragma unroll
          for (int e4 = 0; e4 < EPL / 4; ++e4) {
            float f[4];
            dequant4(in[k].w[e4], sc, bias, plain, f);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if constexpr (sizeof(OUT) == 2) pk.y[4 * e4 + e] = __float2half_rn(f[e]);
              else pk.y[4 * e4 + e] = f[e];
            }
          }
          u32x4 *d4 = reinterpret_cast<u32x4 *>(out + (int64_t)s_row[at[k]] * dim + c[k] * EPL);
#pragma unroll
          for (int e = 0; e < OUT_VECS; ++e) __builtin_nontemporal_store(pk.v[e], d4 + e);
        }
    }
    __syncthreads();
  }
}

// Element-wise fallback for row lengths that are not a multiple of 16.
template <typename OUT>
static __global__ __launch_bounds__(256) void gather_int8_generic_kernel(MoveGroup g, const int8_t *q,
                                                                         const float *scale, int dim,
                                                                         unsigned long long *row_counter) {
  LMI_GRID_ROW(g.n);
  const int32_t *cache_index = g.p[row].src_index;
  OUT *out = reinterpret_cast<OUT *>(g.p[row].dst);
  const int n = *g.p[row].n_ptr;
  const int first = g.p[row].first_ptr ? *g.p[row].first_ptr : 0;
  if (row_counter && bx == 0 && threadIdx.x == 0 && n > first)
    atomicAdd(row_counter, (unsigned long long)(n - first));
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = (bx * blockDim.x + threadIdx.x) / kWave;
  const int n_waves = gx * blockDim.x / kWave;
  for (int i = first + wave; i < n; i += n_waves) {
    const int slot = cache_index[i];
    if (slot < 0) continue;
    const float sc = scale[slot];
    for (int c = lane; c < dim; c += kWave) {
      const float f = __fmul_rn((float)q[(int64_t)slot * dim + c], sc);
      if constexpr (sizeof(OUT) == 2) out[(int64_t)i * dim + c] = __float2half_rn(f);
      else out[(int64_t)i * dim + c] = f;
    }
  }
}

// ------------------------------------------------------------------ lookup
struct LookupArgs {
  const int32_t *ids;
  int64_t n_nodes;
  int kind, table_kind;
  const HashSlot *slots;
  int log2cap;
  const int32_t *slot_of;
  const uint4 *rank_tab;
  const int32_t *lru_keys;
  int32_t *lru_use;
  int64_t lru_sets;
  int lru_ways;
  int32_t *cache_index, *lru_fill;
  int2 *miss_list;
  DevState *st;
  int seg_first, seg_last, seg;
  const HashSlot *dedup;  // the batch's dedup table: value of a seed id = its first row
  int dedup_log2cap;
  int lookup_blocks;  // blocks [0, lookup_blocks) look rows up, the rest carry `fill`
  FillArgs fill;      // last step of the hop sampled just before (hop -1: none)
};

// Bitmap + rank table: the slot of a cached node is the number of cached nodes
// with a smaller id = rank at the start of its 64-id word + set bits below it.
__device__ __forceinline__ int32_t rank_find(const uint4 *tab, int32_t id) {
  const uint4 e = tab[id >> 6];
  const uint64_t bits = (uint64_t)e.x | ((uint64_t)e.y << 32);
  const int b = id & 63;
  if (!((bits >> b) & 1ull)) return -1;
  return (int32_t)e.z + __popcll(bits & ((1ull << b) - 1ull));
}

__device__ __forceinline__ int32_t static_find(int table_kind, const HashSlot *slots, int log2cap,
                                               const int32_t *slot_of, const uint4 *rank_tab, int32_t id) {
  if (table_kind == LMI_TABLE_RANK) return rank_find(rank_tab, id);
  if (table_kind == LMI_TABLE_DIRECT) return slot_of[id];
  return table_find(slots, log2cap, id);
}

// id -> slot for rows [first, last) of the batch -> cache_index[].  Rows that
// miss are appended to the segment's miss list as (row, id) pairs: ballot +
// prefix popcount inside each wavefront, one LDS pass over the 16 wavefronts of
// the block, one atomic per block.  The HBM gather needs no list: it walks the
// rows directly and skips the misses.  List order is arbitrary; it only
// schedules the host-link gather.
constexpr int kLookupBlock = 1024;
struct LookupGroup {  // blocks interleave over the pipes, as in the sampling kernels
  LookupArgs p[LMI_MAX_GROUP];
  int n;
};

static __global__ __launch_bounds__(kLookupBlock) void lookup_kernel(LookupGroup g) {
  LMI_GRID_ROW(g.n);
  const LookupArgs &a = g.p[row];
  __shared__ int wave_cnt[kLookupBlock / kWave];
  __shared__ int block_base;
  if (bx >= a.lookup_blocks) {
    fill_local_ids(a.fill, (int64_t)(bx - a.lookup_blocks) * blockDim.x + threadIdx.x,
                   (int64_t)(gx - a.lookup_blocks) * blockDim.x);
    return;
  }
  const int first = (a.seg_first == 0) ? 0 : a.st->node_counter[9 + a.seg_first - 1];
  const int last = a.st->node_counter[9 + a.seg_last];
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
  const int stride = a.lookup_blocks * blockDim.x;
  for (int b = first + bx * blockDim.x; b < last; b += stride) {
    const int i = b + threadIdx.x;
    bool miss = false;
    int32_t id = -1;
    if (i < last) {
      id = a.ids[i];
      int slot = -1;
      if (id >= 0 && id < a.n_nodes) {
        if (a.kind == LMI_CACHE_LRU) {
          // a set's record is its keys followed by its ticks (one 64-byte line for 8 ways), so the
          // tick of a hit is written into the line its key was just read from
          const int set = (int)((uint32_t)id % (uint32_t)a.lru_sets);
          const int64_t rec = (int64_t)set * 2 * a.lru_ways;
          int way = -1;
          if ((a.lru_ways & 3) == 0) {  // a set's keys start on a 16-byte boundary: four ways per load
            for (int w = 0; w < a.lru_ways; w += 4) {
              const int4 k = *reinterpret_cast<const int4 *>(a.lru_keys + rec + w);
              if (k.x == id) way = w;
              if (k.y == id) way = w + 1;
              if (k.z == id) way = w + 2;
              if (k.w == id) way = w + 3;
            }
          } else {
            for (int w = 0; w < a.lru_ways; ++w)
              if (a.lru_keys[rec + w] == id) way = w;
          }
          if (way >= 0) {
            slot = set * a.lru_ways + way;  // sets * ways < 2^31
            a.lru_use[rec + way] = a.st->lru_tick;
          }
          // a repeated seed keeps both rows, but the id is offered for insertion once, by its first row
          const bool repeat = i < a.st->n_seeds &&
                              table_find(a.dedup, a.dedup_log2cap, id, a.st->table_tag, a.st->table_mask) != i;
          a.lru_fill[i] = repeat ? -2 : -1;
        } else if (a.kind != LMI_CACHE_NONE) {
          slot = static_find(a.table_kind, a.slots, a.log2cap, a.slot_of, a.rank_tab, id);
        }
        miss = slot < 0;
      }
      a.cache_index[i] = slot;
    }
    const uint64_t mm = __ballot(miss);
    if (lane == 0) wave_cnt[wid] = __popcll(mm);
    __syncthreads();
    if (threadIdx.x == 0) {
      int t = 0;
#pragma unroll
      for (int w = 0; w < kLookupBlock / kWave; ++w) {
        const int c = wave_cnt[w];
        wave_cnt[w] = t;
        t += c;
      }
      block_base = t ? atomicAdd(&a.st->n_miss[a.seg], t) : 0;
    }
    __syncthreads();
    if (miss) a.miss_list[block_base + wave_cnt[wid] + __popcll(mm & lanemask_lt())] = make_int2(i, id);
    __syncthreads();
  }
}

static inline int64_t seg_list_base(const Server *s, int seg) { return seg == 0 ? 0 : s->node_cap[seg - 1]; }

int launch_lookup(Server *s, Pipe *const *pp, int n, hipStream_t st, int seg_first, int seg_last) {
  LookupGroup g{};
  g.n = n;
  const int64_t n_max = s->node_cap[seg_last];
  const int lookup_blocks = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(n_max, kLookupBlock), (int64_t)s->n_cu * 2));
  int grid = lookup_blocks;
  const int pending = pp[0]->fill_pending;  // the hop sampled last left its local ids to this kernel
  if (pending >= 0) grid += fill_blocks(s->edge_cap[pending], kLookupBlock);
  for (int k = 0; k < n; ++k) {
    Pipe &p = *pp[k];
    LookupArgs &a = g.p[k];
    a.ids = p.ids;
    a.n_nodes = s->n_nodes;
    a.kind = s->cache_kind;
    a.table_kind = s->table_kind;
    a.slots = s->id_table.slots;
    a.log2cap = s->id_table.log2cap;
    a.slot_of = s->slot_of;
    a.rank_tab = s->rank_tab;
    a.lru_keys = s->lru_keys;
    a.lru_use = s->lru_use;
    a.lru_sets = s->lru_sets;
    a.lru_ways = s->lru_ways;
    a.cache_index = p.cache_index;
    a.miss_list = p.miss_list + seg_list_base(s, seg_first);
    a.lru_fill = p.lru_fill;
    a.dedup = p.dedup.slots;
    a.dedup_log2cap = p.dedup.log2cap;
    a.st = p.st;
    a.seg_first = seg_first;
    a.seg_last = seg_last;
    a.seg = seg_first;
    a.lookup_blocks = lookup_blocks;
    a.fill.hop = -1;
    if (pending >= 0) a.fill = fill_args(p, pending);
    p.fill_pending = -1;
  }
  hipLaunchKernelGGL(lookup_kernel, dim3(grid * n), dim3(kLookupBlock), 0, st, g);
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

// Orders `st` behind the pipe's last batch.  Its side-stream work ends with the event `join_of`; a
// wait on another queue's event holds a stream up for about 10 us even when the event fired long
// ago, so that wait is only queued when the host cannot already see the event as complete.  Work
// of the batch that `join_of` does not cover sits on the caller's stream that carried the batch:
// the same stream orders itself, another one is put behind an event recorded there now (at that
// stream's present tail, which is at or behind the batch's last kernel).
int pipe_handover(Pipe &p, hipStream_t st) {
  if (p.tail_unjoined && p.last_stream != st && p.handover) {
    LMI_HIP(hipEventRecord(p.handover, p.last_stream));
    LMI_HIP(hipStreamWaitEvent(st, p.handover, 0));
    p.last_stream = st;  // `st` now carries the order
  }
  return LMI_OK;
}

int pipe_join(Pipe &p, hipStream_t st) {
  LMI_TRY(pipe_handover(p, st));
  if (!p.side_pending || (p.join_waited && p.join_waiter == st)) return LMI_OK;
  if (hipEventQuery(p.join_of) == hipSuccess) {
    p.side_pending = false;  // complete: no stream has to wait any more
    return LMI_OK;
  }
  (void)hipGetLastError();  // "not ready" is an answer, not a failure
  LMI_HIP(hipStreamWaitEvent(st, p.join_of, 0));
  p.join_waited = true;  // this stream is in order; another one that names the pipe later still has to wait
  p.join_waiter = st;
  return LMI_OK;
}

// A join event was just recorded for the pipe on the side stream.
static void pipe_side_owes(Pipe &p, hipEvent_t join_of) {
  p.join_of = join_of;
  p.side_pending = true;
  p.join_waited = false;
}

int pipes_join(Pipe *const *pp, int n, hipStream_t st) {
  hipEvent_t seen[LMI_MAX_GROUP];
  bool done[LMI_MAX_GROUP];
  int n_seen = 0;
  for (int k = 0; k < n; ++k) {
    Pipe &p = *pp[k];
    LMI_TRY(pipe_handover(p, st));
    if (!p.side_pending) continue;
    int dup = -1;
    for (int j = 0; j < n_seen; ++j)
      if (seen[j] == p.join_of) dup = j;
    if (dup >= 0) {  // `st` already waits for this event, or has seen it complete
      if (done[dup]) p.side_pending = false;
      else p.join_waited = true, p.join_waiter = st;
      continue;
    }
    LMI_TRY(pipe_join(p, st));
    if (n_seen < LMI_MAX_GROUP) {
      seen[n_seen] = p.join_of;
      done[n_seen++] = !p.side_pending;
    }
  }
  return LMI_OK;
}

// int8 rows: dequantised inside the gather.
static int launch_hits_int8(Server *s, const MoveGroup &g, hipStream_t st, int seg_last) {
  const int64_t n_max = s->node_cap[seg_last];
  const int dim = s->cfg.feat_dim;
  const int64_t want = ceil_div(n_max, 4);
  const int64_t cap = s->gather_blocks > 0 ? s->gather_blocks : auto_gather_blocks(s, want);
  const int grid = g.n * (int)std::max<int64_t>(1, std::min<int64_t>(want, cap));
  const int8_t *q = (const int8_t *)s->cache_data;
  unsigned long long *rc = s->prof_on ? s->d_prof_rows : nullptr;
  hipEvent_t e0, e1;
  prof_kernel_events(s, PROF_GATHER_HIT, &e0, &e1);
#define LMI_INT8(KERN)                                                                                   \
  if (e0)                                                                                                \
    hipExtLaunchKernelGGL((KERN), dim3(grid), dim3(256), 0, st, e0, e1, 0, g, q, s->cache_scale, dim, rc); \
  else                                                                                                   \
    hipLaunchKernelGGL((KERN), dim3(grid), dim3(256), 0, st, g, q, s->cache_scale, dim, rc)
  const bool half = s->cfg.feat_dtype == LMI_F16;
  if (dim % 16 == 0 && s->gather_flat != 2) {
    // elements per lane: by default as many as make one 16-byte store (8 fp16, 4 fp32)
    int epl = s->int8_epl > 0 ? s->int8_epl : (half ? 8 : 4);
    if (epl != 16 && epl != 8 && epl != 4) epl = half ? 8 : 4;
    if (half && epl == 4) epl = 8;  // fewer than 16 output bytes per lane are not offered
    // 768-element fp16 rows, share of HBM peak: 8 rows per tile 45 %, 16 51 %, 32 54 %, 64 52 %
    const int tile_rows = s->gather_tile_rows > 0 ? std::min(64, s->gather_tile_rows) : 32;
    // sized by the rows the last launches held (hinted_rows): a block without a tile is not free
    const int64_t want_f = ceil_div(hinted_rows(s, n_max), tile_rows);
    const int64_t cap_f = s->gather_blocks > 0 ? s->gather_blocks
                          : s->gather_adaptive ? (int64_t)s->n_cu * 64 : auto_gather_blocks(s, want_f);
    const int grid_f = g.n * (int)std::max<int64_t>(1, std::min<int64_t>(want_f, cap_f));
#define LMI_INT8_FLAT(KERN)                                                                                   \
  if (e0)                                                                                                     \
    hipExtLaunchKernelGGL((KERN), dim3(grid_f), dim3(256), 0, st, e0, e1, 0, g, q, s->cache_scale, dim,        \
                          tile_rows, rc, s->rows_seen_dev);                                                   \
  else                                                                                                        \
    hipLaunchKernelGGL((KERN), dim3(grid_f), dim3(256), 0, st, g, q, s->cache_scale, dim, tile_rows, rc,       \
                       s->rows_seen_dev)
#define LMI_INT8_FLAT_U(OUT_, EPL_)                                    \
  if (s->gather_unroll >= 4) {                                         \
    LMI_INT8_FLAT((gather_int8_tiled_kernel<OUT_, EPL_, 4>));           \
  } else if (s->gather_unroll != 1) {                                  \
    LMI_INT8_FLAT((gather_int8_tiled_kernel<OUT_, EPL_, 2>));           \
  } else {                                                             \
    LMI_INT8_FLAT((gather_int8_tiled_kernel<OUT_, EPL_, 1>));           \
  }
    if (half && epl == 16) {
      LMI_INT8_FLAT_U(__half, 16)
    } else if (half) {
      LMI_INT8_FLAT_U(__half, 8)
    } else if (epl == 16) {
      LMI_INT8_FLAT_U(float, 16)
    } else if (epl == 8) {
      LMI_INT8_FLAT_U(float, 8)
    } else {
      LMI_INT8_FLAT_U(float, 4)
    }
#undef LMI_INT8_FLAT_U
#undef LMI_INT8_FLAT
  } else if (dim % 16 == 0) {
    // lanes per row: 16 or 32, several 16-element chunks per lane when the row is longer (768-d rows,
    // beside the host-link gather: 64 lanes, 48 of them busy, 39 % of HBM peak; 32 lanes x 2 steps 48 %;
    // 16 lanes x 3 steps 49 %; 8 lanes x 6 steps 46 %), or what the measurement knob asks for
    int lpr = s->gather_lpr;
    if (lpr != 8 && lpr != 16 && lpr != 32 && lpr != 64) lpr = dim / 16 <= 16 ? 16 : 32;
#define LMI_INT8_L(OUT_)                                   \
  if (lpr == 8) {                                          \
    LMI_INT8((gather_int8_kernel<OUT_, 8>));               \
  } else if (lpr == 16) {                                  \
    LMI_INT8((gather_int8_kernel<OUT_, 16>));              \
  } else if (lpr == 32) {                                  \
    LMI_INT8((gather_int8_kernel<OUT_, 32>));              \
  } else {                                                 \
    LMI_INT8((gather_int8_kernel<OUT_, 64>));              \
  }
    if (half) {
      LMI_INT8_L(__half)
    } else {
      LMI_INT8_L(float)
    }
#undef LMI_INT8_L
  } else if (half) {
    LMI_INT8((gather_int8_generic_kernel<__half>));
  } else {
    LMI_INT8((gather_int8_generic_kernel<float>));
  }
#undef LMI_INT8
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

// HBM gather of the cache hits of rows [first, last) on stream `st`, for all n pipes in one launch.
static int launch_hits(Server *s, Pipe *const *pp, int n, hipStream_t st, int seg, int seg_last) {
  LMI_TRY(lru_wait_copied(s, st));
  const int64_t n_max = s->node_cap[seg_last];
  MoveArgs m{};
  m.g.n = n;
  for (int k = 0; k < n; ++k) {
    const Pipe &p = *pp[k];
    MoveRow &r = m.g.p[k];
    r.list = nullptr;  // rows [first, n) directly; cache_index < 0 (a miss) skips the row
    r.first_ptr = seg == 0 ? nullptr : &p.st->node_counter[9 + seg - 1];
    r.n_ptr = &p.st->node_counter[9 + seg_last];
    r.src_index = p.cache_index;
    r.dst = (uint8_t *)p.features;
  }
  if (s->cache_kind == LMI_CACHE_INT8) return launch_hits_int8(s, m.g, st, seg_last);
  m.src = s->cache_data;
  m.src_row_bytes = m.dst_row_bytes = m.row_bytes = s->row_bytes;
  m.n_max = n_max;
  m.row_counter = s->prof_on ? s->d_prof_rows : nullptr;  // all rows of the segment: hits + misses
  prof_kernel_events(s, PROF_GATHER_HIT, &m.ev_start, &m.ev_stop);
  return launch_move_rows(s, st, m, s->gather_nt != 0);
}

// Gather of the rows on the segment's miss list from the feature table, on a
// small grid when the table sits behind the host link (few bytes in flight fill it).
// One launch for all n pipes; the small grid is then shared between them.
static int launch_misses(Server *s, Pipe *const *pp, int n, hipStream_t st, int seg, int seg_last, int blocks_override = 0) {
  MoveArgs m{};
  m.g.n = n;
  for (int k = 0; k < n; ++k) {
    MoveRow &r = m.g.p[k];
    r.list = pp[k]->miss_list + seg_list_base(s, seg);
    r.n_ptr = &pp[k]->st->n_miss[seg];
    r.dst = (uint8_t *)pp[k]->features;
  }
  m.src_from_list = 1;
  m.src = s->feat;
  m.src_row_bytes = m.dst_row_bytes = m.row_bytes = s->row_bytes;
  m.n_max = s->node_cap[seg_last];
  if (s->feat_loc == LMI_LOC_HOST) {
    const int blocks = blocks_override > 0 ? blocks_override : s->miss_blocks > 0 ? s->miss_blocks : s->n_cu;
    m.max_blocks = std::max(1, (blocks + n - 1) / n);  // per pipe
    m.unroll = s->miss_unroll;
    m.host_link = 1;
  }
  m.row_counter = s->prof_on ? s->d_prof_rows + 1 : nullptr;  // misses
  prof_kernel_events(s, PROF_GATHER_MISS, &m.ev_start, &m.ev_stop);
  return launch_move_rows(s, st, m, s->gather_nt != 0);
}

// Gathers the rows [first, last) of a segment into each pipe's feature buffer:
// cache hits from HBM, misses over the host link.  A wide host-link gather beside
// the HBM gather cuts its bandwidth by more than half, so the misses of one batch
// never share a stream with its hits, and run on a small grid (miss_blocks).  With
// several pipes, the hits of all are one launch and so are the misses (group_miss).
// Schedules (tuning key "split_miss"):
//   0  both on the caller's stream, one after the other;
//   1  hits on the caller's stream, misses after them on the server's side stream,
//      where they overlap the next batch's sampling;
//   2  both on the side stream (a gather stage behind the sampling stage): the
//      caller's stream is free for the next batch's sampling as soon as the lookup
//      is done.
// With 1 and 2 the caller's stream does not wait here: the next call on this pipe,
// or lmi_batch_wait, joins.  The LRU cache joins at once (its insert copies the rows).
int launch_misses_early(Server *s, Pipe *const *pp, int n, hipStream_t st, int seg, int seg_last) {
  hipEvent_t fork = pp[0]->fork_early;
  LMI_HIP(hipEventRecord(fork, st));
  LMI_HIP(hipStreamWaitEvent(s->side, fork, 0));
  if (n > 1 && s->group_miss) return launch_misses(s, pp, n, s->side, seg, seg_last, s->miss_blocks_early);
  for (int k = 0; k < n; ++k) LMI_TRY(launch_misses(s, pp + k, 1, s->side, seg, seg_last, s->miss_blocks_early));
  return LMI_OK;  // the join event that launch_gather_group records behind the batch's last misses covers these
}

int launch_gather_group(Server *s, Pipe *const *pp, int n, hipStream_t st, int seg, int seg_last, int lru_lists,
                        bool same_stream, int hit_seg_first) {
  const int hit_seg = hit_seg_first >= 0 ? hit_seg_first : seg;  // the hits of segments whose misses went ahead
  const bool have_cache = s->cache_kind != LMI_CACHE_NONE;
  int mode = (s->feat_loc == LMI_LOC_HOST && have_cache && !same_stream) ? s->split_miss : 0;
  // The gather kernels carry their own profiling events (prof_kernel_events); a bracket
  // left open by the sampling phase ends here.
  hipEvent_t closing = prof_phase(s, st, &s->prof_open, -1);
  if (mode == 0) {
    for (int k = 0; k < n; ++k) {
      pp[k]->tail_unjoined = true;  // everything is on the caller's stream
      if (have_cache) LMI_TRY(launch_hits(s, pp + k, 1, st, seg, seg_last));
      LMI_TRY(launch_misses(s, pp + k, 1, st, seg, seg_last));
      if (lru_lists > 0) LMI_TRY(launch_lru_insert(s, *pp[k], st, lru_lists));
    }
    return LMI_OK;
  }
  hipEvent_t fork = closing;  // when mode 2 forks right here, the closing event doubles as the fork
  if (mode == 2)
    for (int k = 0; k < n; ++k) pp[k]->tail_unjoined = false;  // both gathers run behind the fork
  if (mode == 1) {
    // Host-link reads in flight halve the HBM gather's bandwidth: optionally hold the hits back
    // until the side stream has drained the host-link gathers issued before (other pipes').
    if (s->protect_hits && s->side_busy) {
      if (hipEventQuery(s->side_idle) != hipSuccess) {
        (void)hipGetLastError();
        LMI_HIP(hipStreamWaitEvent(st, s->side_idle, 0));
      } else {
        s->side_busy = false;
      }
    }
    // LRU batches are host-link-bound (a fifth of their rows miss): their host-link gather starts
    // beside the HBM gather instead of behind it.  The insertion that follows it on the side stream
    // only overwrites ways this batch's lookup did not touch, so the hits never read a row it writes.
    const bool early = (lru_lists > 0 && s->lru_early_miss) ||
                       (lru_lists == 0 && (s->early_fork == 1 || (s->early_fork == 2 && n > 1)));
    // behind a late fork the join event covers the whole batch; ahead of an early one the HBM gather stays
    // on the caller's stream alone
    for (int k = 0; k < n; ++k) pp[k]->tail_unjoined = early;
    fork = nullptr;
    if (early) {
      fork = pp[0]->fork;
      LMI_HIP(hipEventRecord(fork, st));
    }
    LMI_TRY(launch_hits(s, pp, n, st, hit_seg, seg_last));  // one launch for the group
  }
  if (!fork) {  // one fork for the whole group
    fork = pp[0]->fork;
    LMI_HIP(hipEventRecord(fork, st));
  }
  LMI_HIP(hipStreamWaitEvent(s->side, fork, 0));
  // the group's host-link gathers as one launch when nothing has to come between them
  const bool misses_together = n > 1 && mode == 1 && lru_lists == 0 && s->group_miss;
  if (misses_together) LMI_TRY(launch_misses(s, pp, n, s->side, seg, seg_last));
  if (misses_together) {  // nothing else of the group goes to the side stream: one event for all its pipes
    LMI_HIP(hipEventRecord(pp[0]->join, s->side));
    for (int k = 0; k < n; ++k) pipe_side_owes(*pp[k], pp[0]->join);
  }
  for (int k = 0; k < n && !misses_together; ++k) {
    Pipe &p = *pp[k];
    if (mode == 2) LMI_TRY(launch_hits(s, pp + k, 1, s->side, seg, seg_last));
    LMI_TRY(launch_misses(s, pp + k, 1, s->side, seg, seg_last));
    if (lru_lists > 0) LMI_TRY(launch_lru_insert(s, p, s->side, lru_lists));  // reads the rows just gathered
    LMI_HIP(hipEventRecord(p.join, s->side));
    pipe_side_owes(p, p.join);
    // an LRU insertion that comes later on the caller's stream copies the gathered rows: join now
    if (s->cache_kind == LMI_CACHE_LRU && lru_lists == 0) LMI_TRY(pipe_join(p, st));
  }
  if (s->protect_hits) {
    LMI_HIP(hipEventRecord(s->side_idle, s->side));
    s->side_busy = true;
  }
  return LMI_OK;
}

int launch_gather_seg(Server *s, Pipe &p, hipStream_t st, int seg, int seg_last, int lru_lists) {
  Pipe *pp[1] = {&p};
  return launch_gather_group(s, pp, 1, st, seg, seg_last, lru_lists);
}

// --------------------------------------------------------------- LRU insert
// Batch-synchronous insertion in two launches.  lru_chain_kernel threads the misses of
// every set into a list (head[set] -> row -> next[row] ...; one atomic exchange per miss,
// on as many addresses as there are sets).  lru_place_kernel: the thread of the row at a
// list's head serves its set alone -- the set's misses in ascending row order each take
// the way with the smallest (last_use, way) among ways not touched in this batch, until
// no way is left; the rest are refused (-2).  A list is as long as the batch has misses
// in that set (one or two for any useful geometry), and the walk is serial, so a cache of
// very few sets pays for its collisions in time, not in correctness.
struct LruArgs {
  const int32_t *ids;
  const int2 *miss_list[LMI_MAX_HOPS + 1];
  const DevState *st;
  int n_lists;
  int32_t *keys, *use, *head, *next, *fill;
  int64_t sets;
  int ways;
};

static __global__ __launch_bounds__(256) void lru_chain_kernel(LruArgs a) {
  for (int l = 0; l < a.n_lists; ++l) {
    const int n = a.st->n_miss[l];
    for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < n; j += gridDim.x * blockDim.x) {
      const int2 pr = a.miss_list[l][j];  // (row, id)
      const int i = pr.x;
      if (a.fill[i] != -1) continue;  // the later row of a repeated seed
      a.next[i] = atomicExch(&a.head[(uint32_t)pr.y % (uint32_t)a.sets], i);
    }
  }
}

static __global__ __launch_bounds__(256) void lru_place_kernel(LruArgs a) {
  const int tick = a.st->lru_tick;
  for (int l = 0; l < a.n_lists; ++l) {
    const int n = a.st->n_miss[l];
    for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < n; j += gridDim.x * blockDim.x) {
      const int2 pr = a.miss_list[l][j];  // (row, id)
      const int i = pr.x;
      const int64_t set = (uint32_t)pr.y % (uint32_t)a.sets;  // sets < 2^31
      if (a.head[set] != i) continue;  // some other row's thread serves this set
      const int64_t base = set * a.ways;     // the set's first slot (row of the cache)
      const int64_t rec = set * 2 * a.ways;  // the set's record: keys, then ticks
      int last = -1;  // the row placed last; the next one is the smallest row above it
      for (int placed = 0; placed < a.ways; ++placed) {
        int row = kIntMax;
        for (int r = i; r != -1; r = a.next[r])
          if (r > last && r < row) row = r;
        if (row == kIntMax) break;  // everybody is placed
        int best = -1, best_use = kIntMax;
        if ((a.ways & 3) == 0) {  // four ways per load, same order of preference (lowest way wins a tie)
          for (int w = 0; w < a.ways; w += 4) {
            const int4 u = *reinterpret_cast<const int4 *>(a.use + rec + w);
            if (u.x < tick && u.x < best_use) best = w, best_use = u.x;
            if (u.y < tick && u.y < best_use) best = w + 1, best_use = u.y;
            if (u.z < tick && u.z < best_use) best = w + 2, best_use = u.z;
            if (u.w < tick && u.w < best_use) best = w + 3, best_use = u.w;
          }
        } else {
          for (int w = 0; w < a.ways; ++w) {
            const int u = a.use[rec + w];
            if (u < tick && u < best_use) best = w, best_use = u;
          }
        }
        if (best < 0) break;  // every way was touched in this batch
        a.keys[rec + best] = a.ids[row];
        a.use[rec + best] = tick;
        a.fill[row] = (int)(base + best);
        last = row;
      }
      for (int r = i; r != -1; r = a.next[r])
        if (a.fill[r] == -1) a.fill[r] = -2;  // no way left for these
      a.head[set] = -1;  // ready for the next batch
    }
  }
}

int launch_lru_insert(Server *s, Pipe &p, hipStream_t st, int n_lists) {
  if (s->cache_kind != LMI_CACHE_LRU) return LMI_OK;
  LruArgs a{};
  a.ids = p.ids;
  for (int l = 0; l < n_lists; ++l) a.miss_list[l] = p.miss_list + seg_list_base(s, l);
  a.st = p.st;
  a.n_lists = n_lists;
  a.keys = s->lru_keys;
  a.use = s->lru_use;
  a.fill = p.lru_fill;
  a.next = p.lru_next;
  a.head = s->lru_head;
  a.sets = s->lru_sets;
  a.ways = s->lru_ways;
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(s->max_nodes, 256), (int64_t)s->n_cu * 4));
  hipLaunchKernelGGL(lru_chain_kernel, dim3(grid), dim3(256), 0, st, a);
  hipLaunchKernelGGL(lru_place_kernel, dim3(grid), dim3(256), 0, st, a);
  LMI_HIP(hipGetLastError());
  // keys and ticks are final: the next batch's lookup may start while the rows are still copied
  LMI_HIP(hipEventRecord(s->lru_ready, st));
  s->lru_pending = true;
  // copy the granted rows from the output buffer (already gathered) into the cache
  for (int l = 0; l < n_lists; ++l) {
    MoveArgs m{};
    m.g.n = 1;
    MoveRow &r = m.g.p[0];
    r.list = p.miss_list + seg_list_base(s, l);
    r.n_ptr = &p.st->n_miss[l];
    r.src_index = nullptr;
    m.src_from_list = 0;
    r.dst_index = p.lru_fill;
    m.src = (const uint8_t *)p.features;
    r.dst = s->cache_data;
    m.src_row_bytes = m.dst_row_bytes = m.row_bytes = s->row_bytes;
    m.n_max = s->node_cap[s->cfg.hops];
    LMI_TRY(launch_move_rows(s, st, m, false));
  }
  LMI_HIP(hipEventRecord(s->lru_copied, st));
  s->lru_copy_pending = true;
  return LMI_OK;
}

// The LRU state is batch-synchronous: a lookup sees the cache after the previous batch's
// insertion.  Sampling does not touch the cache, so only the lookup has to wait.
int lru_wait_ready(Server *s, hipStream_t st) {
  if (s->cache_kind != LMI_CACHE_LRU || !s->lru_pending) return LMI_OK;
  if (hipEventQuery(s->lru_ready) == hipSuccess) {
    s->lru_pending = false;
    return LMI_OK;
  }
  (void)hipGetLastError();  // "not ready" is an answer, not a failure
  LMI_HIP(hipStreamWaitEvent(st, s->lru_ready, 0));
  return LMI_OK;
}

// The rows the previous batch's insertion granted must be in the cache before a gather reads it.
int lru_wait_copied(Server *s, hipStream_t st) {
  if (s->cache_kind != LMI_CACHE_LRU || !s->lru_copy_pending) return LMI_OK;
  if (hipEventQuery(s->lru_copied) == hipSuccess) {
    s->lru_copy_pending = false;
    return LMI_OK;
  }
  (void)hipGetLastError();
  LMI_HIP(hipStreamWaitEvent(st, s->lru_copied, 0));
  return LMI_OK;
}

// -------------------------------------------------------- static cache build
// Ranking key of a node: its out-degree, or how often presampling touched it.
__device__ __forceinline__ int64_t rank_key(const int64_t *indptr, const uint32_t *hot, int64_t v) {
  return hot ? (int64_t)hot[v] : indptr[v + 1] - indptr[v];
}

// Presampling hotness (reference: HotnessMeasure, cache/cache_impl.cuh:190-198): one
// count per appearance of a node among a batch's sampled ids.
static __global__ __launch_bounds__(256) void hotness_kernel(const int32_t *ids, const DevState *st, int64_t n_nodes,
                                                             uint32_t *hot) {
  const int n = st->node_counter[7];
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    const int32_t v = ids[i];
    if (v >= 0 && v < n_nodes) atomicAdd(&hot[v], 1u);
  }
}

int launch_hotness(Server *s, Pipe &p, hipStream_t st) {
  if (!s->hot) {
    LMI_HIP(hipMalloc(&s->hot, (size_t)s->n_nodes * 4));
    LMI_HIP(hipMemsetAsync(s->hot, 0, (size_t)s->n_nodes * 4, st));
  }
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(s->max_nodes, 256), (int64_t)s->n_cu * 4));
  hipLaunchKernelGGL(hotness_kernel, dim3(grid), dim3(256), 0, st, p.ids, p.st, s->n_nodes, s->hot);
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

static __global__ __launch_bounds__(256) void degree_stats_kernel(const int64_t *indptr, const uint32_t *hot,
                                                                  int64_t n, int64_t thr,
                                                                  unsigned long long *count_ge,
                                                                  unsigned long long *max_deg) {
  unsigned long long c = 0, m = 0;
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < n; v += (int64_t)gridDim.x * blockDim.x) {
    const unsigned long long d = (unsigned long long)rank_key(indptr, hot, v);
    c += (d >= (unsigned long long)thr) ? 1 : 0;
    m = d > m ? d : m;
  }
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) {
    c += __shfl_down(c, d, kWave);
    const unsigned long long o = __shfl_down(m, d, kWave);
    m = o > m ? o : m;
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    if (c) atomicAdd(count_ge, c);
    atomicMax(max_deg, m);
  }
}

// mode 0: cnt[v] = (deg == thr);  mode 1: cnt[v] = member flag using tie ranks.
static __global__ __launch_bounds__(kScanBlock) void member_flag_kernel(
    const int64_t *indptr, const uint32_t *hot, const int32_t *n_ptr, int64_t thr, int mode,
    const int32_t *tie_rank, int64_t ties_taken, int32_t *cnt, int32_t *tile_sums) {
  __shared__ int lds[kScanBlock / kWave];
  const int n = *n_ptr;
  const int n_tiles = (n + kScanTile - 1) / kScanTile;
  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int base = tile * kScanTile + threadIdx.x * kScanItems;
    int sum = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
      const int v = base + j;
      if (v < n) {
        const int64_t d = rank_key(indptr, hot, v);
        int f;
        if (mode == 0) f = (d == thr);
        else f = (d > thr) || (d == thr && (int64_t)tie_rank[v] < ties_taken);
        cnt[v] = f;
        sum += f;
      }
    }
    tile_reduce_store(sum, tile_sums, tile, lds);
  }
}

static __global__ __launch_bounds__(256) void publish_slots_kernel(const int32_t *member, const int32_t *slot,
                                                                   int64_t n, int table_kind, HashSlot *slots,
                                                                   int log2cap, int32_t *slot_of,
                                                                   int32_t *cached_ids) {
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < n; v += (int64_t)gridDim.x * blockDim.x) {
    const bool m = member[v] != 0;
    if (table_kind == LMI_TABLE_DIRECT) slot_of[v] = m ? slot[v] : -1;
    if (m) {
      cached_ids[slot[v]] = (int32_t)v;
      if (table_kind == LMI_TABLE_HASH) {
        const uint32_t h = table_insert_min(slots, log2cap, (int32_t)v, slot[v]);
        (void)h;
      }
    }
  }
}

// One thread per 64-id word of the bitmap + rank table.
static __global__ __launch_bounds__(256) void publish_rank_kernel(const int32_t *member, const int32_t *slot,
                                                                  int64_t n, uint4 *tab) {
  const int64_t n_words = (n + 63) / 64;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < n_words; w += (int64_t)gridDim.x * blockDim.x) {
    uint64_t bits = 0;
    const int64_t v0 = w * 64;
    for (int b = 0; b < 64 && v0 + b < n; ++b)
      if (member[v0 + b]) bits |= 1ull << b;
    tab[w] = make_uint4((uint32_t)bits, (uint32_t)(bits >> 32), (uint32_t)slot[v0], 0u);
  }
}

static __global__ void fill_i32_kernel(int32_t *p, int64_t n, int32_t v) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    p[i] = v;
}

static __global__ void fill_slots_kernel(HashSlot *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    p[i] = HashSlot{kEmptyKey, kIntMax};
}

int launch_table_clear(Table &t, hipStream_t st) {
  const int64_t n = int64_t(1) << t.log2cap;
  hipLaunchKernelGGL(fill_slots_kernel, dim3((int)std::min<int64_t>(ceil_div(n, 256), 4096)), dim3(256), 0, st,
                     t.slots, n);
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

void cache_free(Server *s) {
  (void)hipDeviceSynchronize();  // batches in flight (side stream included) still read the old cache
  s->lru_pending = s->lru_copy_pending = false;
  if (s->cache_data) (void)hipFree(s->cache_data);
  if (s->cache_scale) (void)hipFree(s->cache_scale);
  if (s->id_table.slots) (void)hipFree(s->id_table.slots);
  if (s->slot_of) (void)hipFree(s->slot_of);
  if (s->rank_tab) (void)hipFree(s->rank_tab);
  if (s->lru_keys) (void)hipFree(s->lru_keys);  // one allocation: lru_use points into it
  if (s->lru_head) (void)hipFree(s->lru_head);
  s->cache_data = nullptr;
  s->cache_scale = nullptr;
  s->id_table = Table{};
  s->slot_of = nullptr;
  s->rank_tab = nullptr;
  s->lru_keys = s->lru_use = s->lru_head = nullptr;
  s->cache_kind = LMI_CACHE_NONE;
  s->cache_rows = 0;
}

static int count_ge(const Server *s, int64_t thr, unsigned long long *d_pair, int64_t *count, int64_t *max_deg) {
  LMI_HIP(hipMemset(d_pair, 0, 16));
  hipLaunchKernelGGL(degree_stats_kernel, dim3(s->n_cu * 8), dim3(256), 0, 0, s->indptr,
                     s->policy == LMI_POLICY_PRESAMPLED ? s->hot : nullptr, s->n_nodes, thr, d_pair, d_pair + 1);
  unsigned long long h[2];
  LMI_HIP(hipMemcpy(h, d_pair, 16, hipMemcpyDeviceToHost));
  *count = (int64_t)h[0];
  if (max_deg) *max_deg = (int64_t)h[1];
  return LMI_OK;
}

// Hot set = first `capacity_rows` nodes under (out-degree desc, id asc):
// everything above the threshold degree plus the lowest-id ties at the threshold.
// slot(v) = number of cached nodes with a smaller id.
int cache_build_static(Server *s, int64_t capacity_rows, int table_kind, bool int8) {
  if (!s->indptr || !s->feat) LMI_FAIL(LMI_ERR_STATE, "load the graph and attach features before building a cache");
  if (table_kind != LMI_TABLE_HASH && table_kind != LMI_TABLE_DIRECT && table_kind != LMI_TABLE_RANK)
    LMI_FAIL(LMI_ERR_ARG, "bad table kind");
  if (s->n_nodes >= (int64_t(1) << 31) - kScanTile) LMI_FAIL(LMI_ERR_CAPACITY, "too many nodes");
  cache_free(s);
  const int64_t N = s->n_nodes;
  const int64_t cap = std::max<int64_t>(0, std::min(capacity_rows, N));
  s->table_kind = table_kind;
  s->cache_row_bytes = int8 ? s->cfg.feat_dim : s->row_bytes;
  if (cap == 0) LMI_FAIL(LMI_ERR_ARG, "cache capacity must be at least one row");
  if (s->policy == LMI_POLICY_PRESAMPLED && !s->hot)
    LMI_FAIL(LMI_ERR_STATE, "the presampled policy needs lmi_presample (or presampling operators) first");
  const uint32_t *hot_key = s->policy == LMI_POLICY_PRESAMPLED ? s->hot : nullptr;

  // build-time scratch, released on every return path
  struct Scratch {
    std::vector<void *> ptrs;
    ~Scratch() {
      for (void *q : ptrs) (void)hipFree(q);
    }
    hipError_t get(void **p, size_t bytes) {
      const hipError_t e = hipMalloc(p, bytes ? bytes : 1);
      if (e == hipSuccess) ptrs.push_back(*p);
      return e;
    }
  } scratch;
  unsigned long long *d_pair = nullptr;
  int32_t *d_cnt = nullptr, *d_tie = nullptr, *d_slot = nullptr, *d_tiles = nullptr, *d_n = nullptr,
          *d_cached = nullptr;
  LMI_HIP(scratch.get((void **)&d_pair, 16));
  LMI_HIP(scratch.get((void **)&d_cnt, (N + 1) * 4));
  LMI_HIP(scratch.get((void **)&d_tie, (N + 1) * 4));
  LMI_HIP(scratch.get((void **)&d_slot, (N + 1) * 4));
  LMI_HIP(scratch.get((void **)&d_tiles, (ceil_div(N, kScanTile) + 1) * 4));
  LMI_HIP(scratch.get((void **)&d_n, 8));
  LMI_HIP(scratch.get((void **)&d_cached, cap * 4));
  const int32_t n32[2] = {(int32_t)N, 0};
  LMI_HIP(hipMemcpy(d_n, n32, 8, hipMemcpyHostToDevice));

  // threshold degree: largest d with count(deg >= d) >= cap
  int64_t cnt = 0, max_deg = 0;
  LMI_TRY(count_ge(s, 0, d_pair, &cnt, &max_deg));
  int64_t lo = 0, hi = max_deg + 1;
  while (hi - lo > 1) {
    const int64_t mid = lo + (hi - lo) / 2;
    LMI_TRY(count_ge(s, mid, d_pair, &cnt, nullptr));
    if (cnt >= cap) lo = mid; else hi = mid;
  }
  const int64_t thr = lo;
  LMI_TRY(count_ge(s, thr + 1, d_pair, &cnt, nullptr));
  const int64_t ties_taken = cap - cnt;

  const int grid = scan_grid(N);
  hipLaunchKernelGGL(member_flag_kernel, dim3(grid), dim3(kScanBlock), 0, 0, s->indptr, hot_key, d_n, thr, 0, nullptr,
                     (int64_t)0, d_cnt, d_tiles);
  LMI_TRY(launch_scan_phases(0, d_cnt, d_tie, d_tiles, d_n, N, SCAN_EPI_NONE, nullptr, 0, d_n + 1));
  hipLaunchKernelGGL(member_flag_kernel, dim3(grid), dim3(kScanBlock), 0, 0, s->indptr, hot_key, d_n, thr, 1, d_tie,
                     ties_taken, d_cnt, d_tiles);
  LMI_TRY(launch_scan_phases(0, d_cnt, d_slot, d_tiles, d_n, N, SCAN_EPI_NONE, nullptr, 0, d_n + 1));
  int32_t total = 0;
  LMI_HIP(hipMemcpy(&total, d_n + 1, 4, hipMemcpyDeviceToHost));
  if (total != cap) LMI_FAIL(LMI_ERR_HIP, "static cache selection picked %d rows, expected %lld", total, (long long)cap);

  if (table_kind == LMI_TABLE_HASH) {
    int lg = 4;
    while ((int64_t(1) << lg) < 2 * cap) ++lg;
    if (lg > 31) LMI_FAIL(LMI_ERR_CAPACITY, "cache too large for the hash table");
    s->id_table.log2cap = lg;
    LMI_HIP(hipMalloc(&s->id_table.slots, size_t(8) << lg));
    LMI_TRY(launch_table_clear(s->id_table, 0));
  } else if (table_kind == LMI_TABLE_DIRECT) {
    LMI_HIP(hipMalloc(&s->slot_of, N * 4));
  } else {
    LMI_HIP(hipMalloc(&s->rank_tab, (size_t)ceil_div(N, 64) * 16));
    hipLaunchKernelGGL(publish_rank_kernel, dim3(s->n_cu * 8), dim3(256), 0, 0, d_cnt, d_slot, N, s->rank_tab);
  }
  hipLaunchKernelGGL(publish_slots_kernel, dim3(s->n_cu * 8), dim3(256), 0, 0, d_cnt, d_slot, N, table_kind,
                     s->id_table.slots, s->id_table.log2cap, s->slot_of, d_cached);
  LMI_HIP(hipGetLastError());

  // rows
  LMI_HIP(hipMalloc(&s->cache_data, (size_t)cap * s->cache_row_bytes));
  int32_t cap32[2] = {(int32_t)cap, 0};
  LMI_HIP(hipMemcpy(d_n, cap32, 8, hipMemcpyHostToDevice));
  if (int8) {
    LMI_HIP(hipMalloc(&s->cache_scale, (size_t)cap * 4));
    hipLaunchKernelGGL(quantize_rows_kernel, dim3(s->n_cu * 8), dim3(256), 0, 0, d_cached, cap, s->feat,
                       s->cfg.feat_dim, s->cfg.feat_dtype, s->row_bytes, (int8_t *)s->cache_data, s->cache_scale);
    LMI_HIP(hipGetLastError());
  } else {
    MoveArgs m{};
    m.g.n = 1;
    m.g.p[0].n_ptr = d_n;
    m.g.p[0].src_index = d_cached;
    m.g.p[0].dst = s->cache_data;
    m.src = s->feat;
    m.src_row_bytes = m.dst_row_bytes = m.row_bytes = s->row_bytes;
    m.n_max = cap;
    LMI_TRY(launch_move_rows(s, 0, m, false));
  }
  LMI_HIP(hipDeviceSynchronize());
  s->cache_rows = cap;
  s->cache_kind = int8 ? LMI_CACHE_INT8 : LMI_CACHE_STATIC;
  return LMI_OK;
}

// Empty LRU records: key -1 and tick 0 in every way.
static __global__ __launch_bounds__(256) void lru_init_kernel(int32_t *rec, int64_t n_words, int ways) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * blockDim.x)
    rec[i] = ((i / ways) & 1) ? 0 : -1;
}

int cache_build_lru(Server *s, int64_t n_sets, int32_t ways) {
  if (!s->feat) LMI_FAIL(LMI_ERR_STATE, "attach features before building a cache");
  if (n_sets < 1 || ways < 1 || ways > 64 || n_sets * ways >= (int64_t(1) << 31))
    LMI_FAIL(LMI_ERR_ARG, "bad LRU geometry (sets=%lld ways=%d)", (long long)n_sets, ways);
  cache_free(s);
  const int64_t rows = n_sets * ways;
  LMI_HIP(hipMalloc(&s->lru_keys, rows * 8));  // per set: `ways` keys, then `ways` ticks
  s->lru_use = s->lru_keys + ways;
  LMI_HIP(hipMalloc(&s->lru_head, n_sets * 4));
  LMI_HIP(hipMalloc(&s->cache_data, (size_t)rows * s->row_bytes));
  const int g = 2048;
  hipLaunchKernelGGL(lru_init_kernel, dim3(g), dim3(256), 0, 0, s->lru_keys, rows * 2, ways);
  hipLaunchKernelGGL(fill_i32_kernel, dim3(g), dim3(256), 0, 0, s->lru_head, n_sets, -1);
  LMI_HIP(hipDeviceSynchronize());
  s->lru_sets = n_sets;
  s->lru_ways = ways;
  s->lru_tick = 0;
  s->cache_rows = rows;
  s->cache_row_bytes = s->row_bytes;
  s->cache_kind = LMI_CACHE_LRU;
  return LMI_OK;
}

static __global__ void dump_static_kernel(int table_kind, const HashSlot *slots, int log2cap, const int32_t *slot_of,
                                          const uint4 *rank_tab, int64_t n, int32_t *out) {
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < n; v += (int64_t)gridDim.x * blockDim.x)
    out[v] = static_find(table_kind, slots, log2cap, slot_of, rank_tab, (int32_t)v);
}

int cache_dump(Server *s, int32_t *slot_of, int64_t n, int32_t *aux) {
  if (s->cache_kind == LMI_CACHE_NONE) LMI_FAIL(LMI_ERR_STATE, "no cache built");
  LMI_HIP(hipDeviceSynchronize());
  if (s->cache_kind == LMI_CACHE_LRU) {
    if (n != s->cache_rows) LMI_FAIL(LMI_ERR_ARG, "LRU dump needs n == sets*ways");
    std::vector<int32_t> rec((size_t)n * 2);
    LMI_HIP(hipMemcpy(rec.data(), s->lru_keys, (size_t)n * 8, hipMemcpyDeviceToHost));
    const int64_t ways = s->lru_ways;
    for (int64_t slot = 0; slot < n; ++slot) {  // slot = set * ways + way
      const int64_t at = slot / ways * 2 * ways + slot % ways;
      slot_of[slot] = rec[at];
      if (aux) aux[slot] = rec[at + ways];
    }
    return LMI_OK;
  }
  if (n != s->n_nodes) LMI_FAIL(LMI_ERR_ARG, "dump needs n == n_nodes");
  int32_t *d = nullptr;
  LMI_HIP(hipMalloc(&d, n * 4));
  hipLaunchKernelGGL(dump_static_kernel, dim3(s->n_cu * 4), dim3(256), 0, 0, s->table_kind, s->id_table.slots,
                     s->id_table.log2cap, s->slot_of, s->rank_tab, n, d);
  LMI_HIP(hipMemcpy(slot_of, d, n * 4, hipMemcpyDeviceToHost));
  (void)hipFree(d);
  return LMI_OK;
}

}  // namespace lmi

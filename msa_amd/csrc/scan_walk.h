// Tile order of the persistent routing scan, as plain functions shared by the kernel and by a host-side simulation
// (msa_diag_scan_walk) that checks that every tile is visited exactly once.
//
// Workgroup b of the launch sits on XCD b % 8 (workgroups are dealt to the XCDs round-robin) and is the (b / 8)-th of
// that XCD.  With a gather job attached the last workgroup of the launch copies instead of scoring.  The last `pool_n`
// N tiles belong to no XCD: they are a pool that workgroups draw from, one tile at a time, once their own share is
// done.  The other N tiles are split over the XCDs in proportion to their scoring workgroups; inside an XCD's range
// the tiles form a dense order (groups of `m_group` M tiles, a group's M tiles of one N tile adjacent, so that the
// workgroups that share a K_r tile run side by side on one L2), and workgroup w of the XCD takes positions w,
// w + (scoring workgroups of the XCD), ...
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MSA_WALK_FN __host__ __device__ inline
#else
#define MSA_WALK_FN inline
#endif

struct ScanWalk {
  int tiles_m, tiles_n, m_group, pool_n;
  int n_begin, n_in_xcd;      // the XCD's own N range
  int wg_in_xcd, wgs_in_xcd;  // this workgroup among the XCD's scoring workgroups
  int dense_total;            // tiles of the XCD's own range
  int pool_total;             // tiles of the pool
  int own_count;              // own tiles of this workgroup
};

// position p of the dense order over n_in N tiles from nb on -> (M tile, N tile)
MSA_WALK_FN void scan_walk_decode(int tiles_m, int m_group, int p, int nb, int n_in, int& tm, int& tn) {
  const int full_groups = tiles_m / m_group, full = full_groups * n_in * m_group;
  int g, rem, mg;
  if (p < full) { g = p / (n_in * m_group); rem = p - g * n_in * m_group; mg = m_group; }
  else { g = full_groups; rem = p - full; mg = tiles_m - full_groups * m_group; }
  tn = nb + rem / mg;
  tm = g * m_group + rem % mg;
}

MSA_WALK_FN ScanWalk scan_walk_init(int block, int grid, int has_copy_wg, int tiles_m, int tiles_n, int m_group, int pool_n) {
  ScanWalk w;
  w.tiles_m = tiles_m; w.tiles_n = tiles_n; w.m_group = m_group; w.pool_n = pool_n;
  const int xcd = block % 8;
  const int scoring_wgs = grid - (has_copy_wg ? 1 : 0);
  int before = 0;                                   // scoring workgroups on XCDs 0 .. xcd - 1
  for (int y = 0; y < xcd; ++y) before += (scoring_wgs - y + 7) / 8;
  w.wg_in_xcd = block / 8;
  w.wgs_in_xcd = (scoring_wgs - xcd + 7) / 8;
  const int tiles_n_own = tiles_n - pool_n;
  const int denom = scoring_wgs > 0 ? scoring_wgs : 1;
  w.n_begin = (int)((int64_t)tiles_n_own * before / denom);
  const int n_stop = (int)((int64_t)tiles_n_own * (before + w.wgs_in_xcd) / denom);
  w.n_in_xcd = n_stop - w.n_begin;
  w.dense_total = w.n_in_xcd * tiles_m;
  w.pool_total = pool_n * tiles_m;
  w.own_count = w.wg_in_xcd < w.dense_total && w.wgs_in_xcd > 0
                    ? (w.dense_total - w.wg_in_xcd + w.wgs_in_xcd - 1) / w.wgs_in_xcd : 0;
  return w;
}

// the workgroup's idx-th own tile
MSA_WALK_FN void scan_walk_own(const ScanWalk& w, int idx, int& tm, int& tn) {
  scan_walk_decode(w.tiles_m, w.m_group, w.wg_in_xcd + idx * w.wgs_in_xcd, w.n_begin, w.n_in_xcd, tm, tn);
}

// pool position p (a value drawn from the pool's counter; valid while p < pool_total)
MSA_WALK_FN void scan_walk_pool(const ScanWalk& w, int p, int& tm, int& tn) {
  scan_walk_decode(w.tiles_m, w.m_group, p, w.tiles_n - w.pool_n, w.pool_n, tm, tn);
}

// The workgroup's own tiles in order, without a division per tile: the cursor steps by the XCD's workgroup count
// through the dense order, keeping (group of M tiles, N offset, M offset) and the step split into whole N tiles and a
// remainder of M tiles; only a step that crosses into the next group of M tiles divides.
struct ScanWalkCursor {
  int g, mg, tn_off, tm_off, dq, dr;
};

MSA_WALK_FN int scan_walk_group_size(const ScanWalk& w, int g) {
  const int full_groups = w.tiles_m / w.m_group;
  return g < full_groups ? w.m_group : w.tiles_m - full_groups * w.m_group;
}

MSA_WALK_FN void scan_walk_cursor_place(const ScanWalk& w, ScanWalkCursor& c, int g, int rem) {
  int mg = scan_walk_group_size(w, g);
  while (mg > 0 && rem >= w.n_in_xcd * mg) {      // (past the last group the cursor is never read)
    rem -= w.n_in_xcd * mg;
    mg = scan_walk_group_size(w, ++g);
  }
  if (mg <= 0) mg = 1;
  c.g = g; c.mg = mg;
  c.tn_off = rem / mg; c.tm_off = rem % mg;
  c.dq = w.wgs_in_xcd / mg; c.dr = w.wgs_in_xcd % mg;
}

// cursor on the workgroup's first own tile
MSA_WALK_FN ScanWalkCursor scan_walk_cursor(const ScanWalk& w) {
  ScanWalkCursor c;
  scan_walk_cursor_place(w, c, 0, w.wg_in_xcd);
  return c;
}

MSA_WALK_FN void scan_walk_cursor_tile(const ScanWalk& w, const ScanWalkCursor& c, int& tm, int& tn) {
  tm = c.g * w.m_group + c.tm_off;
  tn = w.n_begin + c.tn_off;
}

// on to the workgroup's next own tile (the caller counts them: own_count)
MSA_WALK_FN void scan_walk_cursor_next(const ScanWalk& w, ScanWalkCursor& c) {
  c.tm_off += c.dr;
  c.tn_off += c.dq;
  if (c.tm_off >= c.mg) { c.tm_off -= c.mg; ++c.tn_off; }
  if (c.tn_off >= w.n_in_xcd) scan_walk_cursor_place(w, c, c.g + 1, (c.tn_off - w.n_in_xcd) * c.mg + c.tm_off);
}

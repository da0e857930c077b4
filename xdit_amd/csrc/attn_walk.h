// Which work a workgroup of an attention launch does, and which threads of the merge kernel hold
// which row: index arithmetic only, written as plain C++ so that the same code is compiled into
// the kernels (hipcc) and into a host program that walks every workgroup of a planned launch and
// checks that each query tile and KV iteration is covered exactly once (g++, no GPU).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define XDIT_HD __host__ __device__ __forceinline__
#else
#define XDIT_HD inline
#endif

namespace xdit {

// Workgroup index -> work tile, XCD-aware.  Workgroups are handed to the 8 XCDs round-robin
// (workgroup i runs on XCD i % 8).  Giving XCD x the contiguous tile range
// [x * tiles_per_xcd, (x+1) * tiles_per_xcd) keeps the query tiles of one (batch, head) — which
// all stream the same K/V — on one XCD, so that K/V is fetched into that XCD's L2 once.
// A bijection onto [0, 8 * tiles_per_xcd) only.
XDIT_HD int xcd_tile_index(int block, int tiles_per_xcd) {
  return (block & 7) * tiles_per_xcd + (block >> 3);
}

// One piece of work of a workgroup: KV iterations [it0, it1) of query tile `tile`.  slot < 0: the
// workgroup owns the whole tile and writes the final result; otherwise the piece is one part of a
// query tile whose KV iterations are shared, and its partial result goes to that workspace slot.
// dyn >= 0: after [it0, it1) the workgroup goes on with KV iterations pool0 + ticket of the same
// query tile, one at a time, tickets drawn from counter `dyn` of the launch until they run past
// the tile's last iteration; everything it processes goes into the one partial result of `slot`.
struct Segment {
  int tile, it0, it1;
  int64_t slot;
  int dyn, pool0;
};

// The sequence of segments of workgroup `w`.  P is any struct with the launch-geometry members of
// AttnParams (total_tiles, tiles_per_xcd, split_full, split_units, split_len, split_pmax,
// split_fuse0, split_claimers, split_dyn, split_s0, split_order); `nt` is the number of KV iterations of a
// whole tile.
// Plain launch (split_units == 0): workgroup = one query tile over all KV iterations.  Balanced
// launch: the first split_full workgroups each take a whole query tile; the KV iterations of the
// remaining query tiles, laid end to end, are cut into split_units ranges of split_len
// iterations.  A range may cover the end of one query tile and the start of the next.  The ranges
// are processed by split_claimers workgroups: the workgroups split_fuse0 .. split_full-1 (the
// last to be dispatched) after their own query tile, so that no compute unit waits for a new
// workgroup to be dispatched in between, or, with fewer whole tiles than that
// (split_fuse0 > split_full), workgroups of their own, split_full .. split_full+claimers-1.
// Claimer c starts with range c; when there are more ranges than claimers the caller hands out
// every further range through a counter (wants_claim / claimed), so that compute units that run
// faster (the clocks of the eight XCDs differ by several per cent) take more of them.
// Streamed sharing (split_dyn != 0; few shared tiles, short shares): the claimers are dealt out
// over the shared tiles in contiguous groups (consecutive workgroups sit on different XCDs);
// member g of a tile's group owns KV iterations [g s0, (g+1) s0) of the tile and then draws the
// remaining iterations one at a time from the tile's counter, so that a group ends together
// however its members' speeds differ.  Which iterations land in which partial result then
// depends on timing: results are reproducible only to rounding.
// Parts first (split_order != 0; only when every claimer has exactly one range, i.e. without a
// counter, and runs a whole tile too): a claimer processes its range BEFORE its whole query tile,
// so that the partial results of the shared tiles are long complete when the workgroups reach
// their ends and fold them there, a slice each (see fold duties in attn_split.h).
struct WorkgroupWalk {
  int whole_tile;  // a whole query tile still to do (< 0: none)
  int u_next;      // the range to take next (< 0: none)
  int u, lin, lin_end, rem_iters;
  bool claimer;

  template <typename P>
  XDIT_HD bool start(const P& p, int nt, int w) {
    whole_tile = -1;
    u_next = -1;
    u = lin = lin_end = 0;
    claimer = false;
    rem_iters = (p.total_tiles - p.split_full) * nt;
    if (p.split_units == 0) {
      whole_tile = xcd_tile_index(w, p.tiles_per_xcd);
      return whole_tile < p.total_tiles;
    }
    if (w < p.split_full) {
      // the XCD-aware order needs a multiple of 8 whole tiles (it is one for every compute-unit
      // count that is a multiple of 8); any other count keeps the dispatch order
      whole_tile = (p.split_full & 7) == 0 ? xcd_tile_index(w, p.split_full >> 3) : w;
      u_next = w - p.split_fuse0;
    } else {
      u_next = w - p.split_full;
    }
    claimer = w >= p.split_fuse0 || w >= p.split_full;
    return true;
  }

  // The next segment; false when the workgroup is done.
  template <typename P>
  XDIT_HD bool next(const P& p, int nt, Segment& s) {
    const bool range_left = lin < lin_end || (u_next >= 0 && u_next < p.split_units);
    if (whole_tile >= 0 && !(p.split_order != 0 && range_left)) {
      s.tile = whole_tile; s.it0 = 0; s.it1 = nt; s.slot = -1; s.dyn = -1; s.pool0 = 0;
      whole_tile = -1;
      return true;
    }
    if (lin >= lin_end) {  // the next range
      if (u_next < 0 || u_next >= p.split_units) return false;
      u = u_next;
      u_next = -1;
      lin = u * p.split_len;
      lin_end = lin + p.split_len < rem_iters ? lin + p.split_len : rem_iters;
      if (p.split_dyn != 0) lin = lin_end = 0;
    }
    s.dyn = -1;
    s.pool0 = 0;
    if (p.split_dyn != 0) {  // one segment: this claimer's place in its tile's group
      const int rem = p.total_tiles - p.split_full;
      const int r = (int)(((int64_t)u * rem) / p.split_claimers);
      const int c0 = (int)(((int64_t)r * p.split_claimers + rem - 1) / rem);
      const int c1 = (int)(((int64_t)(r + 1) * p.split_claimers + rem - 1) / rem);
      const int g = u - c0;
      s.tile = p.split_full + r;
      s.it0 = g * p.split_s0;
      s.it1 = s.it0 + p.split_s0;
      s.slot = (int64_t)r * p.split_pmax + g;
      s.dyn = r;
      s.pool0 = (c1 - c0) * p.split_s0;
      lin = lin_end = 0;
      return true;
    }
    const int r = lin / nt;  // which of the remaining query tiles
    s.it0 = lin - r * nt;
    s.it1 = (lin_end - r * nt) < nt ? (lin_end - r * nt) : nt;
    const int part = u - (r * nt) / p.split_len;  // ranges are consecutive: index within the tile
    s.slot = (int64_t)r * p.split_pmax + part;
    s.tile = p.split_full + r;
    lin += s.it1 - s.it0;
    return true;
  }

  // After a segment: true when the workgroup has to draw its next range from the counter
  // (`counter`: the launch hands ranges out that way); claimed(ticket) records the draw.
  XDIT_HD bool wants_claim(bool counter) const {
    return counter && claimer && whole_tile < 0 && lin >= lin_end && u_next < 0;
  }
  template <typename P>
  XDIT_HD void claimed(const P& p, unsigned ticket) { u_next = p.split_claimers + (int)ticket; }
};

// Parts of shared query tile r (0-based among the remaining tiles) as the fold reads them:
// workspace slots r * split_pmax + [0, parts).
template <typename P>
XDIT_HD int shared_tile_parts(const P& p, int nt, int r) {
  if (p.split_dyn != 0) {
    const int rem = p.total_tiles - p.split_full;
    return (int)(((int64_t)(r + 1) * p.split_claimers + rem - 1) / rem) - (int)(((int64_t)r * p.split_claimers + rem - 1) / rem);
  }
  const int first_unit = (r * nt) / p.split_len;
  const int last_unit = ((r + 1) * nt - 1) / p.split_len;
  return last_unit - first_unit + 1;
}

// Folding the parts of a shared query tile inside the attention kernel, without anybody waiting
// for anybody.  The tile's parts (at most kFoldMaxParts) are folded in slices of rows: slice j,
// rows [j R / n, (j+1) R / n) of the tile's R rows, is the fold duty of the workgroup that wrote
// part j of its n parts.  One 32-bit word per shared tile records, through atomic adds only,
//   bits 0..7    parts that have arrived (partial result written and released),
//   bits 8..23   slices whose duty was presented before the last part had arrived (deferred),
//   bits 24..31  events so far: every part contributes two (its arrival and its duty).
// A workgroup presents its duty either together with its arrival (one add) or later, at its very
// end (parts-first launches, where the parts are long complete by then).  Whoever makes the tile
// complete (the last arrival) folds every slice deferred so far (plus its own if it presented its
// duty with the arrival); a duty presented after completion is folded by its own workgroup.  The
// atomic adds on one word are totally ordered, so each slice is folded exactly once, after all
// parts are there; the workgroup that makes the last event puts the word back to zero.
constexpr int kFoldMaxParts = 16;
constexpr unsigned kFoldSliceShift = 8, kFoldEventShift = 24;
XDIT_HD unsigned fold_arrive_word(int j, bool with_duty) {
  return with_duty ? 1u + (1u << (kFoldSliceShift + j)) + (2u << kFoldEventShift) : 1u + (1u << kFoldEventShift);
}
XDIT_HD unsigned fold_duty_word(int j) { return (1u << (kFoldSliceShift + j)) + (1u << kFoldEventShift); }
// `old` is what the atomic add returned.  The slices (bit j = slice j) to fold now:
XDIT_HD unsigned fold_after_arrival(unsigned old, int j, bool with_duty, int n) {
  if ((int)(old & 0xffu) + 1 != n) return 0u;
  const unsigned deferred = (old >> kFoldSliceShift) & 0xffffu;
  return with_duty ? deferred | (1u << j) : deferred;
}
XDIT_HD unsigned fold_after_duty(unsigned old, int j, int n) { return (int)(old & 0xffu) == n ? 1u << j : 0u; }
XDIT_HD bool fold_last_event(unsigned old, unsigned word, int n) {
  return (int)((old >> kFoldEventShift) + (word >> kFoldEventShift)) == 2 * n;
}
XDIT_HD void fold_slice_rows(int j, int n, int rows, int& r0, int& r1) {
  r0 = j * rows / n;
  r1 = (j + 1) * rows / n;
}

// Thread -> (row, first 8-element chunk) map of the merge kernel.  A row of `cpr` chunks is held
// by cpr adjacent lanes of ONE wavefront (cpr <= 64, i.e. head_dim <= 512), a wavefront holds
// rows_per_wave = 64 / cpr whole rows and its remaining lanes idle.  A row never spans two wavefronts: every lane of a row reads the
// row's log-sum-exp before the row's first lane overwrites it, which only program order inside
// one wavefront guarantees.
struct MergeMap {
  int cpr, lanes_per_row, rows_per_wave;
  unsigned inv;  // ceil(2^16 / lanes_per_row): lane / lanes_per_row == (lane * inv) >> 16 for lane < 64
};
XDIT_HD MergeMap merge_map(int D) {
  MergeMap m;
  m.cpr = D >> 3;
  m.lanes_per_row = m.cpr < 64 ? m.cpr : 64;
  m.rows_per_wave = 64 / m.lanes_per_row;
  m.inv = (65536u + m.lanes_per_row - 1) / m.lanes_per_row;
  return m;
}
// False for an idle lane.  `wave` is the global wavefront index, `lane` 0..63.
XDIT_HD bool merge_thread_row(const MergeMap& m, int64_t wave, int lane, int64_t& row, int& chunk0) {
  const int r = (int)(((unsigned)lane * m.inv) >> 16);
  row = wave * m.rows_per_wave + r;
  chunk0 = lane - r * m.lanes_per_row;
  return r < m.rows_per_wave;
}

}  // namespace xdit

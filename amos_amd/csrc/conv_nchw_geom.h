// Geometry of the convolution kernel that reads NCDHW activations and KCTRS weights as they are
// (conv_nchw_kernel.h): which input positions a tile of output positions touches, where each of
// them sits in the LDS patch, which thread fetches it, and where a lane finds the operand of an
// output position at a window tap.  Plain integer functions shared by the kernel, the host-side
// planner (LDS and task budgets) and a CPU check that every reader address meets the element a
// writer put there.
//
// A tile is BJ consecutive output positions j = ((n * OD + od) * OP + op) * OQ + oq and may touch
// up to kNchwMaxSeg (image, output depth) slices.  Per slice the patch is a zero-padded window
// [rows][Wp] of input positions, 64 bytes of channels each (32 halves / 64 int8: one matrix-core
// K sub-step).  A window tap (r, s) only shifts the position a lane reads: by r * dil_h rows and
// s * dil_w columns.
//
// Bank conflicts (measured on gfx950 with a microbenchmark: 16-byte accesses of one wave, lane l on
// a chosen 16-byte slot of the 256-byte bank space).  A 16-byte read of a wave is served in four
// cycles, two per half of the wave, when no slot is used by more than two lanes of a half (248
// bytes per clock and CU); sixteen consecutive lanes on sixteen slots, or any other split of a
// half's 32 lanes into two conflict-free sixteens, all run at that rate, four lanes per slot at
// half of it.  16-byte writes reach a third of the read rate whatever the slots.
// Layout: eight consecutive positions form a 512-byte block of two 256-byte lines -- chunks 0 and
// 1 in the first, 2 and 3 in the second -- chunk c of position P in slot
// ((P & 7) * 2 + (c & 1)) ^ ((c >> 1) * 4) of its line.
//   * A fragment read: the lower half of a wave holds sixteen consecutive positions x chunks 0 and
//     1, the upper half chunks 2 and 3 (lane group q = lane / 16 reads chunk q): every slot twice
//     per half, whatever position the sixteen start at, so also at every window tap.
//   * Consecutive outputs are consecutive positions except where they wrap into the next patch
//     row; with a row pitch that differs from the outputs per row by a multiple of 8 the slots
//     continue across the wrap.
//   * The weight tiles use the same formula with the row in the place of the position.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define AMOS_HD __host__ __device__ __forceinline__
#else
#define AMOS_HD inline
#endif

namespace amos {

constexpr int kNchwMaxSeg = 4;
constexpr int kNchwPosBytes = 64;   // bytes of channels per patch position and macro step

// Loader waves of a workgroup (beside its matrix-core waves): they fetch and transpose the patch,
// 16 load groups (x four chunks of channels) per wave and round.
constexpr int nchw_loader_waves(bool packed, int groups) { return (void)packed, (void)groups, 4; }

// n / d for 0 <= n < 2^31 by a multiplication with a host-built constant (the extents are known
// when the kernel is launched; a hardware-less integer division costs dozens of instructions)
struct NchwDiv {
  uint32_t magic, shift, one, d;
};
inline NchwDiv nchw_make_div(uint32_t d) {
  NchwDiv f = {0, 0, 0, d};
  if (d <= 1) { f.one = 1; return f; }
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;
  const uint64_t sft = 31 + l;
  f.magic = (uint32_t)(((1ull << sft) + d - 1) / d);
  f.shift = (uint32_t)(sft - 32);
  return f;
}
AMOS_HD int nchw_div(int n, const NchwDiv& f) {
  const uint32_t hi = (uint32_t)(((uint64_t)(uint32_t)n * f.magic) >> 32);
  return (int)((hi + (uint32_t)n * f.one) >> f.shift);
}

struct NchwShape {
  int N, C, D, H, W, K, T, R, S;
  int sd, sh, sw, pd, ph, pw, dd, dh, dw;
  int OD, OP, OQ;
  int J;           // N * OD * OP * OQ
  int Wp;          // patch row pitch in positions
  int pg_shift;    // log2 of the input positions per 8-byte load: 2 (16-bit types) or 3 (int8)
  NchwDiv div_opq, div_oq, div_w, div_od;
};

// patch row pitch: the columns a row of outputs touches, rounded up so that the pitch differs from
// the outputs per row by a multiple of `align` (16: conflict-free across row wraps; 1: smallest)
AMOS_HD int nchw_patch_pitch(int OQ, int S, int sw, int dw, int sh, int align) {
  int wp = (OQ - 1) * sw + (S - 1) * dw + 1;
  if (sw == 1 && sh == 1 && align > 1) wp += (align - ((wp - OQ) % align)) % align;
  return wp;
}

struct NchwSeg {
  int pos0;      // first LDS position of the slice's window (multiple of 8)
  int pa;        // first output row of the tile in this slice
  int h_first;   // input row of window row 0 (may be negative: padding)
  int n, d0;     // image, input depth of depth tap 0 (may be out of range: padding)
  int flo, fhi;  // flat in-plane range [flo, fhi) of the input positions that exist (h * W + w)
  int glo;       // first load group: flo / pg
  int grp0;      // groups of the slices before this one
  int rows;      // window rows
};

// per-slice fields as 4-element vectors: a lane-dependent slice index then becomes a chain of
// selects (an array inside the struct would put the whole tile into scratch memory on the GPU)
typedef int nchw_i4 __attribute__((vector_size(16)));
struct NchwTile {
  int bj0, j_last, sl_a, nseg;
  int npos;      // LDS positions used
  int ngroups;   // load groups of all slices
  nchw_i4 pos0, pa, h_first, n, d0, flo, fhi, glo, grp0, rows;   // NchwSeg's fields, one element per slice
};
static_assert(kNchwMaxSeg == 4, "NchwTile holds four slices");

// nseg > kNchwMaxSeg is reported as it is; only the first kNchwMaxSeg slices are filled
AMOS_HD NchwTile nchw_tile(const NchwShape& s, int bj0, int BJ) {
  NchwTile t;
  const int OPQ = s.OP * s.OQ;
  const int pg = 1 << s.pg_shift;
  t.bj0 = bj0;
  t.j_last = bj0 + BJ - 1 < s.J ? bj0 + BJ - 1 : s.J - 1;
  t.sl_a = nchw_div(bj0, s.div_opq);
  const int sl_b = nchw_div(t.j_last, s.div_opq);
  t.nseg = sl_b - t.sl_a + 1;
  int pos = 0, grp = 0;
#pragma unroll
  for (int g = 0; g < kNchwMaxSeg; ++g) {
    const bool live = g < t.nseg;
    const int sl = t.sl_a + (live ? g : t.nseg - 1);
    const int lo = bj0 > sl * OPQ ? bj0 : sl * OPQ;
    const int hi = t.j_last < (sl + 1) * OPQ - 1 ? t.j_last : (sl + 1) * OPQ - 1;
    const int pa = nchw_div(lo - sl * OPQ, s.div_oq), pb = nchw_div(hi - sl * OPQ, s.div_oq);
    const int rows = (pb - pa) * s.sh + (s.R - 1) * s.dh + 1;
    const int h_first = pa * s.sh - s.ph;
    const int hlo = h_first > 0 ? h_first : 0;
    const int hhi = h_first + rows - 1 < s.H - 1 ? h_first + rows - 1 : s.H - 1;
    const int flo = hlo * s.W;
    const int fhi = hhi >= hlo ? (hhi + 1) * s.W : flo;
    const int glo = flo >> s.pg_shift;
    const int ghi = (fhi + pg - 1) >> s.pg_shift;
    const int n = nchw_div(sl, s.div_od);
    t.pa[g] = pa;
    t.rows[g] = rows;
    t.h_first[g] = h_first;
    t.flo[g] = flo;
    t.fhi[g] = fhi;
    t.glo[g] = glo;
    t.n[g] = n;
    t.d0[g] = (sl - n * s.OD) * s.sd - s.pd;
    t.pos0[g] = pos;
    t.grp0[g] = grp;
    if (live) {
      pos += (rows * s.Wp + 7) & ~7;   // whole 8-position blocks
      grp += fhi > flo ? ghi - glo : 0;
    }
  }
  t.npos = pos;
  t.ngroups = grp;
  return t;
}

// LDS byte offset (inside a patch buffer / a weight tile) of 16-byte chunk `chunk` of position
// (row) P
AMOS_HD int nchw_position_offset(int P, int chunk) {
  return ((P >> 3) << 9) + ((chunk >> 1) << 8) + (((((P & 7) << 1) | (chunk & 1)) ^ ((chunk >> 1) << 2)) << 4);
}
// the chunk lane group q (lane / 16) of a fragment read takes
AMOS_HD int nchw_frag_chunk(int q) { return q; }
// the row (of sixteen) that the lanes 4x .. 4x+3 of a wave fill when a wave writes sixteen rows
// of a weight tile with one store
AMOS_HD int nchw_row_of_slot(int x) { return (x & 3) | ((x & 4) << 1) | ((x & 8) >> 1); }
// the inverse of nchw_position_offset inside a 1 KB block of 16 rows: which (row, chunk) lives in
// 16-byte slot x = 0..63 (a direct global -> LDS copy puts lane x's bytes there)
AMOS_HD void nchw_unit_of_slot(int x, int* row, int* chunk) {
  const int hi = (x >> 4) & 1;
  const int y = (x & 15) ^ (hi << 2);
  *row = (x >> 5) * 8 + (y >> 1);
  *chunk = hi * 2 + (y & 1);
}
// ... of the position in window row hr, window column wc of slice `q`
AMOS_HD int nchw_lds_offset(const NchwShape& s, const NchwSeg& q, int hr, int wc, int chunk) {
  return nchw_position_offset(q.pos0 + hr * s.Wp + wc, chunk);
}

// slice `idx` (0 .. kNchwMaxSeg - 1) of a tile, picked by selects on constant element numbers
#define AMOS_NCHW_PICK(field) (idx == 1 ? t.field[1] : idx == 2 ? t.field[2] : idx == 3 ? t.field[3] : t.field[0])
AMOS_HD NchwSeg nchw_pick_seg(const NchwTile& t, int idx) {
  NchwSeg q;
  q.pos0 = AMOS_NCHW_PICK(pos0); q.pa = AMOS_NCHW_PICK(pa); q.h_first = AMOS_NCHW_PICK(h_first);
  q.n = AMOS_NCHW_PICK(n); q.d0 = AMOS_NCHW_PICK(d0); q.flo = AMOS_NCHW_PICK(flo); q.fhi = AMOS_NCHW_PICK(fhi);
  q.glo = AMOS_NCHW_PICK(glo); q.grp0 = AMOS_NCHW_PICK(grp0); q.rows = AMOS_NCHW_PICK(rows);
  return q;
}
#undef AMOS_NCHW_PICK

// A load group: `pg` consecutive in-plane input positions of one slice, fetched (for one chunk of
// channels) by one thread with one 8-byte load per channel.  Returns the slice and sets f, the
// group's first in-plane position (a multiple of the group size).
AMOS_HD NchwSeg nchw_group(const NchwShape& s, const NchwTile& t, int grp, int* f) {
  int idx = 0;
#pragma unroll
  for (int g = 1; g < kNchwMaxSeg; ++g)
    if (g < t.nseg && grp >= t.grp0[g]) idx = g;
  const NchwSeg q = nchw_pick_seg(t, idx);
  *f = (q.glo + grp - q.grp0) << s.pg_shift;
  return q;
}
// LDS byte offset where chunk `chunk` of in-plane position f of slice q goes, or -1 when the
// position is not part of the slice's window (outside [flo, fhi), or a column no output reads)
AMOS_HD int nchw_writer_offset(const NchwShape& s, const NchwSeg& q, int f, int chunk) {
  if (f < q.flo || f >= q.fhi) return -1;
  const int h = nchw_div(f, s.div_w), w = f - h * s.W;
  if (w + s.pw >= s.Wp) return -1;   // image columns right of what the last output column reads
  return nchw_lds_offset(s, q, h - q.h_first, w + s.pw, chunk);
}

// where the lanes of a fragment read find output position j (clamped into the tile by the caller)
// at tap (0, 0): its LDS position; a tap adds (tr * dh * Wp + ts * dw)
AMOS_HD int nchw_column(const NchwShape& s, const NchwTile& t, int j) {
  const int OPQ = s.OP * s.OQ;
  const int sl = nchw_div(j, s.div_opq), rem = j - sl * OPQ;
  const int op = nchw_div(rem, s.div_oq), oq = rem - op * s.OQ;
  const NchwSeg q = nchw_pick_seg(t, (sl - t.sl_a) & (kNchwMaxSeg - 1));
  return q.pos0 + (op - q.pa) * s.sh * s.Wp + oq * s.sw;
}
AMOS_HD int nchw_reader_offset(const NchwShape& s, int column, int tr, int ts, int chunk) {
  return nchw_position_offset(column + tr * s.dh * s.Wp + ts * s.dw, chunk);
}

}  // namespace amos

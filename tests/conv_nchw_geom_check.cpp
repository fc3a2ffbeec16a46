// CPU check of amos_amd/csrc/conv_nchw_geom.h: for every tile of a list of convolution shapes, play
// the writers (one thread per load group and channel chunk) into a model of the LDS patch, then ask
// the readers' address function for every (output position, window tap, chunk) and require that it
// meets exactly the input element the convolution wants there, or a slot nobody wrote (zero padding);
// all addresses inside the buffer, no slot written twice, and, with unit strides, no 16-byte bank
// slot used by more than two lanes of a half wave in a fragment read.
//   g++ -O1 -I amos_amd/csrc -o geom_check tests/conv_nchw_geom_check.cpp && ./geom_check
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "conv_nchw_geom.h"

using namespace amos;

struct Case {
  int N, C, D, H, W, K, T, R, S, sd, sh, sw, pd, ph, pw, dd, dh, dw, pg_shift, BJ, align;
};

static int fails = 0;
#define REQUIRE(cond, ...)                                   \
  do {                                                       \
    if (!(cond)) {                                           \
      if (fails < 20) { printf("FAIL %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); } \
      ++fails;                                               \
    }                                                        \
  } while (0)

static int out_extent(int in, int pad, int dil, int k, int stride) {
  const int eff = (k - 1) * dil + 1;
  return in + 2 * pad < eff ? 0 : (in + 2 * pad - eff) / stride + 1;
}

static void run(const Case& c, bool quiet = false) {
  NchwShape s;
  s.N = c.N; s.C = c.C; s.D = c.D; s.H = c.H; s.W = c.W; s.K = c.K; s.T = c.T; s.R = c.R; s.S = c.S;
  s.sd = c.sd; s.sh = c.sh; s.sw = c.sw; s.pd = c.pd; s.ph = c.ph; s.pw = c.pw; s.dd = c.dd; s.dh = c.dh; s.dw = c.dw;
  s.OD = out_extent(c.D, c.pd, c.dd, c.T, c.sd);
  s.OP = out_extent(c.H, c.ph, c.dh, c.R, c.sh);
  s.OQ = out_extent(c.W, c.pw, c.dw, c.S, c.sw);
  s.J = s.N * s.OD * s.OP * s.OQ;
  s.Wp = nchw_patch_pitch(s.OQ, s.S, s.sw, s.dw, s.sh, c.align);
  s.pg_shift = c.pg_shift;
  s.div_opq = nchw_make_div(s.OP * s.OQ);
  s.div_oq = nchw_make_div(s.OQ);
  s.div_w = nchw_make_div(s.W);
  s.div_od = nchw_make_div(s.OD);
  REQUIRE((s.H * s.W) % (1 << s.pg_shift) == 0, "plane size must be a multiple of the load group");
  // the left padding must fit the window: column w + pw >= 0 always; the right end inside Wp
  REQUIRE(s.W - 1 + s.pw < s.Wp + (s.S - 1) * s.dw + s.sw * s.OQ, "sanity");
  const int OPQ = s.OP * s.OQ;
  const int pg = 1 << s.pg_shift;
  int max_pos = 0, max_groups = 0, max_seg = 0;
  long conflicts = 0, reads = 0, wconflicts = 0, writes = 0;
  for (int bj0 = 0; bj0 < s.J; bj0 += c.BJ) {
    const NchwTile t = nchw_tile(s, bj0, c.BJ);
    if (t.nseg > max_seg) max_seg = t.nseg;
    if (t.nseg > kNchwMaxSeg) continue;   // the planner refuses such a tile size
    if (t.npos > max_pos) max_pos = t.npos;
    if (t.ngroups > max_groups) max_groups = t.ngroups;
    // content of every 16-byte slot: -1 = zero, else ((n * H + h) * W + w) * 4 + chunk
    std::vector<long> lds((size_t)t.npos * 4, -1);
    for (int grp = 0; grp < t.ngroups; ++grp)
      for (int cg = 0; cg < 4; ++cg) {
        int f = 0;
        const NchwSeg q = nchw_group(s, t, grp, &f);
        REQUIRE(f >= 0 && f + pg <= s.H * s.W, "group [%d, %d) leaves the plane", f, f + pg);
        for (int i = 0; i < pg; ++i) {
          const int off = nchw_writer_offset(s, q, f + i, cg);
          if (off < 0) continue;
          REQUIRE(off % 16 == 0 && off + 16 <= t.npos * 64, "writer offset %d outside %d", off, t.npos * 64);
          if (off % 16 || off + 16 > t.npos * 64) continue;
          REQUIRE(lds[off / 16] == -1, "slot %d written twice", off / 16);
          const int h = (f + i) / s.W, w = (f + i) % s.W;
          lds[off / 16] = (((long)q.n * s.H + h) * s.W + w) * 4 + cg;
        }
      }
    // bank slots of a staging store: lanes l .. l+7 (two consecutive load groups x four chunks) are
    // served with lanes l+32 .. l+39 (the groups eight further on), whose threads store position i ^ 1
    for (int g0 = 0; g0 + 9 < t.ngroups; g0 += 16)
      for (int pair = 0; pair < 8 && g0 + pair + 9 < t.ngroups; pair += 2)
        for (int i = 0; i < pg; ++i) {
          unsigned seen = 0;
          bool counted = true;
          for (int l = 0; l < 16 && counted; ++l) {
            const int upper = l >> 3;
            int f = 0;
            const NchwSeg q = nchw_group(s, t, g0 + pair + ((l >> 2) & 1) + 8 * upper, &f);
            const int off = nchw_writer_offset(s, q, f + (upper ? i ^ 1 : i), l & 3);
            if (off < 0) { counted = false; break; }
            const unsigned bit = 1u << ((off & 255) >> 4);
            if (seen & bit) ++wconflicts;
            seen |= bit;
          }
          if (counted) ++writes;
        }
    // every input position a slice needs must have been written exactly where readers look
    for (int j = bj0; j <= t.j_last; ++j) {
      const int sl = j / OPQ, rem = j % OPQ, op = rem / s.OQ, oq = rem % s.OQ;
      const int n = sl / s.OD;
      const int col = nchw_column(s, t, j);
      for (int tr = 0; tr < s.R; ++tr)
        for (int ts = 0; ts < s.S; ++ts)
          for (int ch = 0; ch < 4; ++ch) {
            const int off = nchw_reader_offset(s, col, tr, ts, ch);
            REQUIRE(off >= 0 && off % 16 == 0 && off + 16 <= t.npos * 64, "reader offset %d outside %d (j %d tap %d,%d)",
                    off, t.npos * 64, j, tr, ts);
            if (off < 0 || off % 16 || off + 16 > t.npos * 64) continue;
            const int h = op * s.sh - s.ph + tr * s.dh, w = oq * s.sw - s.pw + ts * s.dw;
            const bool inside = h >= 0 && h < s.H && w >= 0 && w < s.W;
            const long want = inside ? (((long)n * s.H + h) * s.W + w) * 4 + ch : -1;
            REQUIRE(lds[off / 16] == want, "j %d tap (%d,%d) chunk %d reads slot %d = %ld, wants %ld", j, tr, ts, ch,
                    off / 16, lds[off / 16], want);
          }
    }
    // bank slots of a fragment read: half a wave = sixteen consecutive outputs of one slice x the chunks
    // of two lane groups; no slot may be used by more than two of the 32 lanes
    if (s.sh == 1 && s.sw == 1)
      for (int j0 = bj0; j0 + 15 <= t.j_last; j0 += 16) {
        if (j0 / OPQ != (j0 + 15) / OPQ) continue;
        for (int tr = 0; tr < s.R; ++tr)
          for (int ts = 0; ts < s.S; ++ts)
            for (int half = 0; half < 2; ++half) {
              int uses[16] = {0};
              for (int l = 0; l < 32; ++l) {
                const int off = nchw_reader_offset(s, nchw_column(s, t, j0 + (l & 15)), tr, ts, nchw_frag_chunk(2 * half + (l >> 4)));
                if (++uses[(off & 255) >> 4] > 2) ++conflicts;
              }
              ++reads;
            }
      }
  }
  if (quiet) return;   // (seeded random shapes: addresses and contents only)
  if (c.align >= 8) REQUIRE(conflicts == 0, "%ld bank-group collisions in %ld fragment reads", conflicts, reads);
  printf("%5.1f %% of fragment reads and %5.1f %% of staging stores with a bank-group collision; ",
         reads ? 100.0 * conflicts / reads : 0.0, writes ? 100.0 * wconflicts / writes : 0.0);
  printf("N%d C%d D%d %dx%d K%d %dx%dx%d s%d%d%d p%d%d%d d%d%d%d BJ%d pg%d: Wp %d, max positions %d, groups %d, slices %d%s\n",
         c.N, c.C, c.D, c.H, c.W, c.K, c.T, c.R, c.S, c.sd, c.sh, c.sw, c.pd, c.ph, c.pw, c.dd, c.dh, c.dw, c.BJ, pg,
         s.Wp, max_pos, max_groups, max_seg, max_seg > kNchwMaxSeg ? " (too many: refused by the planner)" : "");
}

int main() {
  const Case cases[] = {
      // N  C   D  H   W   K   T  R  S  strides  pads     dils     pg BJ  pitch alignment
      {32, 256, 1, 14, 14, 256, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 2, 128, 8},   // fp16 conv2d of the benchmark
      {32, 256, 1, 14, 14, 256, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 2, 256, 8},
      {4, 128, 1, 28, 28, 128, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 3, 256, 8},    // int8 conv2d (one 8-byte load = 8 positions)
      {4, 128, 1, 28, 28, 128, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 3, 128, 8},
      {2, 64, 5, 56, 56, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 256, 8},      // conv3d of the benchmark (fewer slices)
      {2, 64, 5, 56, 56, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 128, 8},
      {3, 32, 1, 7, 8, 40, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 2, 128, 8},        // small images: several per tile
      {2, 32, 1, 9, 12, 40, 1, 3, 3, 1, 1, 1, 0, 0, 0, 1, 1, 1, 2, 128, 8},       // no padding
      {2, 32, 1, 10, 12, 40, 1, 3, 3, 1, 2, 2, 0, 1, 1, 1, 1, 1, 2, 128, 8},      // strides
      {2, 32, 1, 12, 12, 40, 1, 3, 3, 1, 1, 1, 0, 2, 2, 1, 2, 2, 2, 128, 8},      // dilation
      {2, 32, 3, 6, 8, 40, 3, 3, 3, 2, 1, 2, 1, 1, 0, 1, 1, 1, 2, 128, 8},        // mixed strides, 3-d
      {1, 32, 1, 20, 18, 8, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 2, 256, 8},       // a ragged last tile (360 outputs)
      {2, 64, 1, 16, 16, 8, 1, 3, 3, 1, 1, 2, 0, 1, 2, 1, 1, 1, 3, 128, 8},       // int8, column stride
      {1, 32, 1, 224, 224, 8, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 2, 128, 8},     // wide rows
      {70, 32, 1, 2, 2, 8, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 2, 128, 8},        // 4 outputs per image: too many slices
      {32, 256, 1, 14, 14, 256, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 2, 128, 1},    // the smallest pitch: collisions at row wraps only
      {2, 64, 5, 56, 56, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 256, 4},
      {2, 64, 5, 56, 56, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 256, 16},
      {2, 64, 5, 56, 56, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 3, 256, 8},      // 16-bit types with 16-byte loads: 8 positions
      {2, 64, 5, 56, 56, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 3, 128, 8},
      {3, 32, 1, 6, 12, 40, 1, 3, 3, 1, 1, 1, 0, 1, 1, 1, 1, 1, 3, 128, 8},       // ... groups that straddle image rows
      {2, 32, 1, 10, 12, 40, 1, 3, 3, 1, 2, 2, 0, 1, 1, 1, 1, 1, 3, 128, 8},      // ... strides
      {2, 32, 3, 6, 8, 40, 3, 3, 3, 2, 1, 2, 1, 1, 0, 1, 1, 1, 3, 128, 8},        // ... mixed strides, 3-d
  };
  for (const Case& c : cases) run(c);
  // seeded random shapes (window 3x3, any stride / padding / dilation the planner accepts): every
  // writer inside its channel plane and its buffer, every reader on the element it wants
  {
    unsigned long long state = 0x9e3779b97f4a7c15ull;
    auto rnd = [&](int lo, int hi) {   // uniform in [lo, hi]
      state = state * 6364136223846793005ull + 1442695040888963407ull;
      return lo + (int)((state >> 33) % (unsigned long long)(hi - lo + 1));
    };
    int ran = 0;
    for (int it = 0; it < 40000 && ran < 3000; ++it) {
      Case c;
      c.N = rnd(1, 5); c.C = 32; c.K = 8; c.R = 3; c.S = 3;
      const bool three_d = rnd(0, 2) == 0;
      c.D = three_d ? rnd(1, 5) : 1; c.T = three_d ? 3 : 1;
      c.H = rnd(2, 40); c.W = rnd(2, 40);
      c.sd = three_d ? rnd(1, 2) : 1; c.sh = rnd(1, 2); c.sw = rnd(1, 2);
      c.pd = three_d ? rnd(0, 1) : 0; c.ph = rnd(0, 2); c.pw = rnd(0, 2);
      c.dd = 1; c.dh = rnd(1, 2); c.dw = rnd(1, 2);
      c.pg_shift = rnd(2, 3); c.BJ = rnd(0, 1) ? 128 : 256; c.align = rnd(0, 1) ? 8 : 1;
      if ((c.H * c.W) % (1 << c.pg_shift)) continue;
      if (out_extent(c.D, c.pd, c.dd, c.T, c.sd) <= 0 || out_extent(c.H, c.ph, c.dh, 3, c.sh) <= 0 ||
          out_extent(c.W, c.pw, c.dw, 3, c.sw) <= 0)
        continue;
      const int before = fails;
      run(c, true);
      if (fails != before)
        printf("  ... in random case N%d D%d %dx%d s%d%d%d p%d%d%d d%d%d%d pg%d BJ%d align %d\n", c.N, c.D, c.H, c.W, c.sd, c.sh,
               c.sw, c.pd, c.ph, c.pw, c.dd, c.dh, c.dw, 1 << c.pg_shift, c.BJ, c.align);
      ++ran;
    }
    printf("%d seeded random shapes\n", ran);
  }
  // weight tiles: a bijection; a fragment read (rows r .. r+7, chunks of lane groups q and q + 2) and
  // a store (lanes 4x .. 4x+3 fill row nchw_row_of_slot(x); lanes l .. l+7 with l+32 .. l+39) on
  // sixteen different slots
  {
    std::vector<int> used(64 * 4, 0);
    for (int row = 0; row < 64; ++row)
      for (int ch = 0; ch < 4; ++ch) {
        const int off = nchw_position_offset(row, ch);
        REQUIRE(off % 16 == 0 && off >= 0 && off < 64 * 64 && !used[off / 16], "weight tile offset %d", off);
        if (off >= 0 && off < 64 * 64) used[off / 16] = 1;
      }
    for (int r0 = 0; r0 < 64; r0 += 16)
      for (int half = 0; half < 2; ++half) {
        int uses[16] = {0};
        for (int l = 0; l < 32; ++l)
          REQUIRE(++uses[(nchw_position_offset(r0 + (l & 15), nchw_frag_chunk(2 * half + (l >> 4))) & 255) >> 4] <= 2,
                  "weight fragment read: a slot used by more than two lanes of a half (rows %d..)", r0);
      }
    for (int x0 = 0; x0 < 8; x0 += 2) {
      unsigned seen = 0;
      for (int l = 0; l < 16; ++l) {
        const int x = x0 + ((l >> 2) & 1) + 8 * (l >> 3);
        const unsigned bit = 1u << ((nchw_position_offset(nchw_row_of_slot(x), l & 3) & 255) >> 4);
        REQUIRE(!(seen & bit), "weight store collides (lanes of slots %d..)", x0);
        seen |= bit;
      }
    }
    // a direct copy of a block of 16 rows: slot x holds the unit nchw_unit_of_slot names
    for (int x = 0; x < 64; ++x) {
      int row = -1, ch = -1;
      nchw_unit_of_slot(x, &row, &ch);
      REQUIRE(row >= 0 && row < 16 && ch >= 0 && ch < 4 && nchw_position_offset(row, ch) == x * 16,
              "slot %d is not where unit (%d, %d) lives", x, row, ch);
      REQUIRE(nchw_position_offset(32 + row, ch) == 2048 + x * 16, "blocks of 16 rows are not 1 KB apart (slot %d)", x);
    }
    unsigned rows = 0;
    for (int x = 0; x < 16; ++x) rows |= 1u << nchw_row_of_slot(x);
    REQUIRE(rows == 0xffffu, "nchw_row_of_slot is not a permutation");
  }
  if (fails) { printf("%d checks failed\n", fails); return 1; }
  printf("ok\n");
  return 0;
}

// Host-side helper of the block-sparse entry points (no GPU work): the order in which the workgroups of the forward and of
// the dQ kernel take the 16-row blocks of a layout (fa_fwd_args.row_order).  A workgroup owns eight consecutive entries of
// the order and stages every key block that any of the eight lists; each of its four waves owns two consecutive entries
// and computes on every key block that either of the two lists.  The cost of an order is therefore
//     sum over groups of eight of |union of the eight lists|  +  sum over pairs of |union of the two lists|,
// and this file looks for an order that makes it small: a greedy grouping (a group starts with the fullest row block left
// and takes, seven times, the row block that adds the fewest key blocks to the group's set), then a fixed number of
// pairwise exchanges between random positions, each kept if the cost does not rise (2000 attempts per row block, four million at most).  Deterministic (own generator, fixed seed).
#include <cstdint>
#include <cstring>
#include <vector>

#include "../../include/flash_attn_gfx950.h"

namespace {

struct Layout {
  int nr, W;
  std::vector<uint64_t> bits;  // [nr][W]
  const uint64_t* row(int r) const { return bits.data() + (size_t)r * W; }
};

inline int popcount_or(const uint64_t* a, const uint64_t* b, int W) {
  int n = 0;
  for (int w = 0; w < W; w++) n += __builtin_popcountll(a[w] | b[w]);
  return n;
}

// staged key blocks of the group that starts at position g0, and the sum of its pairs' unions
void group_cost(const Layout& L, const int32_t* order, int g0, int* staged, int* pairs) {
  uint64_t un[64];  // (W <= 64: checked by the caller)
  std::memset(un, 0, sizeof(uint64_t) * L.W);
  const int g1 = g0 + 8 < L.nr ? g0 + 8 : L.nr;
  int pu = 0;
  for (int i = g0; i < g1; i += 2) {
    const uint64_t* a = L.row(order[i]);
    const uint64_t* b = i + 1 < g1 ? L.row(order[i + 1]) : a;
    for (int w = 0; w < L.W; w++) {
      const uint64_t u = a[w] | b[w];
      pu += __builtin_popcountll(u);
      un[w] |= u;
    }
  }
  int st = 0;
  for (int w = 0; w < L.W; w++) st += __builtin_popcountll(un[w]);
  *staged = st;
  *pairs = pu;
}

}  // namespace

extern "C" int fa_blocksparse_row_order(const uint8_t* layout, int32_t n_row_blocks, int32_t n_col_blocks, int32_t* order) {
  if (!layout || !order || n_row_blocks <= 0 || n_col_blocks <= 0 || n_col_blocks > 64 * 64) return FA_ERR_INVALID_ARGUMENT;
  Layout L;
  L.nr = n_row_blocks;
  L.W = (n_col_blocks + 63) / 64;
  L.bits.assign((size_t)L.nr * L.W, 0);
  for (int r = 0; r < L.nr; r++)
    for (int c = 0; c < n_col_blocks; c++)
      if (layout[(size_t)r * n_col_blocks + c]) L.bits[(size_t)r * L.W + (c >> 6)] |= uint64_t(1) << (c & 63);
  const int nr = L.nr, W = L.W;

  // ---- greedy grouping
  std::vector<int> count(nr);
  std::vector<char> left(nr, 1);
  for (int r = 0; r < nr; r++) {
    int n = 0;
    for (int w = 0; w < W; w++) n += __builtin_popcountll(L.row(r)[w]);
    count[r] = n;
  }
  std::vector<uint64_t> un(W);
  int pos = 0;
  while (pos < nr) {
    int seed = -1;
    for (int r = 0; r < nr; r++)
      if (left[r] && (seed < 0 || count[r] > count[seed])) seed = r;
    left[seed] = 0;
    order[pos++] = seed;
    for (int w = 0; w < W; w++) un[w] = L.row(seed)[w];
    for (int k = 1; k < 8 && pos < nr; k++) {
      int best = -1;
      int64_t best_score = 0;
      for (int r = 0; r < nr; r++) {
        if (!left[r]) continue;
        int added = 0, shared = 0;
        for (int w = 0; w < W; w++) {
          added += __builtin_popcountll(L.row(r)[w] & ~un[w]);
          shared += __builtin_popcountll(L.row(r)[w] & un[w]);
        }
        const int64_t score = (int64_t)added * (n_col_blocks + 1) - shared;
        if (best < 0 || score < best_score) { best = r; best_score = score; }
      }
      left[best] = 0;
      order[pos++] = best;
      for (int w = 0; w < W; w++) un[w] |= L.row(best)[w];
    }
  }

  // ---- exchanges
  const int ng = (nr + 7) / 8;
  std::vector<int> gst(ng), gpu(ng);
  for (int g = 0; g < ng; g++) group_cost(L, order, g * 8, &gst[g], &gpu[g]);
  uint64_t s = 0x9E3779B97F4A7C15ull;  // xorshift64*
  auto next = [&]() {
    s ^= s >> 12; s ^= s << 25; s ^= s >> 27;
    return (uint32_t)((s * 0x2545F4914F6CDD1Dull) >> 32);
  };
  const int64_t rounds = (int64_t)2000 * nr < 4000000 ? (int64_t)2000 * nr : 4000000;  // (a second or so at most)
  for (int64_t it = 0; it < rounds; it++) {
    const int i = (int)(((uint64_t)next() * (uint64_t)nr) >> 32), j = (int)(((uint64_t)next() * (uint64_t)nr) >> 32);
    if (i == j) continue;
    const int gi = i >> 3, gj = j >> 3;
    int32_t t = order[i]; order[i] = order[j]; order[j] = t;
    int si, pi, sj = 0, pj = 0;
    group_cost(L, order, gi * 8, &si, &pi);
    if (gj != gi) group_cost(L, order, gj * 8, &sj, &pj);
    const int before = gst[gi] + gpu[gi] + (gj != gi ? gst[gj] + gpu[gj] : 0);
    if (si + pi + sj + pj <= before) {
      gst[gi] = si; gpu[gi] = pi;
      if (gj != gi) { gst[gj] = sj; gpu[gj] = pj; }
    } else {
      t = order[i]; order[i] = order[j]; order[j] = t;
    }
  }

  // ---- layouts made of whole 128-row tiles gain nothing: keep their rows where they are
  int64_t staged = 0, plain = 0;
  for (int g = 0; g < ng; g++) staged += gst[g];
  std::vector<int32_t> ident(nr);
  for (int r = 0; r < nr; r++) ident[r] = r;
  for (int g = 0; g < ng; g++) {
    int st, pu;
    group_cost(L, ident.data(), g * 8, &st, &pu);
    plain += st;
  }
  if (staged * 100 > plain * 95) std::memcpy(order, ident.data(), sizeof(int32_t) * nr);
  return FA_OK;
}

// Host-side check of the index arithmetic that the per-volume kernels of so3_fused4r.h rely on (compiled with
// hipcc --cuda-host-only and run on the CPU by tests/test_fused_geometry.py): every item (c, a, n) of a grid sits in exactly
// one place, the rounds that a truncated spectrum keeps hold every item below its bandwidth, the slot permutation of a line
// is a permutation and index_of inverts it, and the sizes follow from the threads and rounds.
#include <cstdio>
#include <set>
#include <tuple>
#include "so3_fused4r.h"

template <class G>
int check(const char* name) {
  int bad = 0;
  std::set<std::tuple<int, int, int>> seen;
  for (int p = 0; p < G::NIT * G::THREADS; ++p) {
    int c, a, n;
    if (!G::decode(p, c, a, n)) continue;
    if (c < 0 || c >= G::NCG || a < 0 || n < 0 || a >= G::width(c) || n >= G::width(c)) { std::printf("%s: place %d holds (%d,%d,%d)\n", name, p, c, a, n); ++bad; }
    if (!seen.insert({c, a, n}).second) { std::printf("%s: item (%d,%d,%d) twice\n", name, c, a, n); ++bad; }
    if (p != G::offset(c) + a * G::width(c) + n) { std::printf("%s: place %d is not the number of its item\n", name, p); ++bad; }
  }
  int want = 0;
  for (int c = 0; c < G::NCG; ++c) want += G::width(c) * G::width(c);
  if ((int)seen.size() != want || want != G::NITEMS) { std::printf("%s: %d items, want %d\n", name, (int)seen.size(), want); ++bad; }
  // every column (a, n) < bandwidth has the degree groups c >= max(a, n) / 4 and no others
  for (int a = 0; a < G::NR; ++a)
    for (int n = 0; n < G::NR; ++n)
      for (int c = 0; c < G::NCG; ++c) {
        const bool has = seen.count({c, a, n}) != 0, should = 4 * c + 3 >= (a > n ? a : n);
        if (has != should) { std::printf("%s: column (%d,%d) group %d: %d, want %d\n", name, a, n, c, (int)has, (int)should); ++bad; }
      }
  // truncated spectra: the active rounds hold every item with a degree below nl
  for (int nl = 1; nl <= G::NR + 5; ++nl) {
    const int rounds = G::active_rounds(nl);
    if (rounds < 1 || rounds > G::NIT) { std::printf("%s: %d rounds for %d degrees\n", name, rounds, nl); ++bad; }
    for (int p = rounds * G::THREADS; p < G::NIT * G::THREADS; ++p) {
      int c, a, n;
      if (G::decode(p, c, a, n) && 4 * c < nl && 4 * c < G::NR) { std::printf("%s: nl %d drops item (%d,%d,%d)\n", name, nl, c, a, n); ++bad; }
    }
  }
  std::set<int> slots;
  for (int k = 0; k < G::N; ++k) {
    const int s = G::slot_of(k);
    if (s < 0 || s >= G::N || !slots.insert(s).second || G::index_of(s) != k) { std::printf("%s: slot of %d\n", name, k); ++bad; }
  }
  if (G::A_THREADS != G::N * G::N / 4 || G::B_THREADS != 4 * G::N || G::B_COLS_FIRST % 64 || G::B_COLS_FIRST + G::B_THREADS > G::THREADS) ++bad;
  if (G::REC_BYTES != (size_t)G::NIT * 4 * G::THREADS * 16 || G::PACKED_FLOATS != (size_t)G::NJ * G::NIT * 2 * G::THREADS * 4) ++bad;
  for (int a = 0; a <= G::NR; ++a)       // quad rows do not overlap and stay 16-byte aligned
    if (G::quad_row(a) % 2 || (a < G::NR && G::quad_row(a) + 4 * (G::NR + 1) > G::quad_row(a + 1)) || G::quad_row(a) + 4 * (G::NR + 1) > G::QUAD_ELEMS) ++bad;
  std::printf("%s: N %d threads %d rounds %d items %d record %zu B table %zu B: %s\n", name, G::N, G::THREADS, G::NIT, G::NITEMS, G::REC_BYTES,
              G::PACKED_FLOATS * 4, bad ? "FAILED" : "ok");
  return bad;
}

int main() {
  int bad = check<fused4r::Grid20>("20^3") + check<fused4r::Grid32>("32^3") + check<fused4r::Grid44>("44^3");
  // the generated item table of the 64^3 kernels: every item once
  std::set<std::tuple<int, int, int>> seen;
  for (int i = 0; i < fused64::NIT * fused64::THREADS; ++i) {
    const unsigned e = fused64::ITEM_TABLE_HOST[i];
    if (!((e >> 13) & 1u)) continue;
    const int n = e & 31, a = (e >> 5) & 31, c = (e >> 10) & 7;
    if (4 * c + 3 < (a > n ? a : n) || !seen.insert({c, a, n}).second) ++bad;
  }
  if ((int)seen.size() != fused64::NITEMS) ++bad;
  std::printf("64^3: %d items: %s\n", (int)seen.size(), (int)seen.size() == fused64::NITEMS ? "ok" : "FAILED");
  return bad ? 1 : 0;
}

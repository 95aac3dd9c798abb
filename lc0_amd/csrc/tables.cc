#include "tables.h"

#include <cstdlib>
#include <map>
#include <utility>

namespace lc0mi {
namespace {

struct MoveIndex {
  int16_t plain[64][64];
  int16_t promo[8][8][3];  // from-file, to-file, piece (q, r, b)
  MoveIndex() {
    int idx = 0;
    for (int f = 0; f < 64; f++)
      for (int t = 0; t < 64; t++) {
        plain[f][t] = -1;
        if (f == t) continue;
        int dr = std::abs(t / 8 - f / 8), df = std::abs(t % 8 - f % 8);
        bool queen = dr == 0 || df == 0 || dr == df;
        bool knight = (dr == 1 && df == 2) || (dr == 2 && df == 1);
        if (queen || knight) plain[f][t] = static_cast<int16_t>(idx++);
      }
    for (int ff = 0; ff < 8; ff++)
      for (int tf = 0; tf < 8; tf++)
        for (int p = 0; p < 3; p++) promo[ff][tf][p] = -1;
    for (int ff = 0; ff < 8; ff++)
      for (int tf = ff - 1; tf <= ff + 1; tf++) {
        if (tf < 0 || tf > 7) continue;
        for (int p = 0; p < 3; p++) promo[ff][tf][p] = static_cast<int16_t>(idx++);
      }
  }
};

const MoveIndex& Moves() {
  static const MoveIndex m;
  return m;
}

std::vector<int16_t> Invert(const std::vector<int16_t>& map) {
  std::vector<int16_t> inv(1858, -1);
  for (size_t i = 0; i < map.size(); i++)
    if (map[i] >= 0) inv[map[i]] = static_cast<int16_t>(i);
  return inv;
}

}  // namespace

const std::vector<int16_t>& AttnPolicyMap() {
  static const std::vector<int16_t> map = [] {
    std::vector<int16_t> m(64 * 64 + 8 * 24, -1);
    const MoveIndex& mi = Moves();
    for (int f = 0; f < 64; f++)
      for (int t = 0; t < 64; t++) m[f * 64 + t] = mi.plain[f][t];
    for (int ff = 0; ff < 8; ff++)
      for (int tf = 0; tf < 8; tf++)
        for (int p = 0; p < 3; p++) m[4096 + 24 * ff + 3 * tf + p] = mi.promo[ff][tf][p];
    return m;
  }();
  return map;
}

const std::vector<int16_t>& ConvPolicyMap() {
  static const std::vector<int16_t> map = [] {
    std::vector<int16_t> m(73 * 64, -1);
    const MoveIndex& mi = Moves();
    // (rank step, file step): N, NE, E, SE, S, SW, W, NW.
    static const int dirs[8][2] = {{1, 0}, {1, 1}, {0, 1}, {-1, 1}, {-1, 0}, {-1, -1}, {0, -1}, {1, -1}};
    static const int knight[8][2] = {{2, 1}, {1, 2}, {-1, 2}, {-2, 1}, {-2, -1}, {-1, -2}, {1, -2}, {2, -1}};
    static const int promo_piece[3] = {1, 2, 0};  // planes hold r, b, q; table order is q, r, b
    for (int sq = 0; sq < 64; sq++) {
      int r = sq / 8, f = sq % 8;
      for (int d = 0; d < 8; d++)
        for (int dist = 1; dist < 8; dist++) {
          int rr = r + dirs[d][0] * dist, ff = f + dirs[d][1] * dist;
          if (rr < 0 || rr > 7 || ff < 0 || ff > 7) continue;
          m[(d * 7 + dist - 1) * 64 + sq] = mi.plain[sq][rr * 8 + ff];
        }
      for (int k = 0; k < 8; k++) {
        int rr = r + knight[k][0], ff = f + knight[k][1];
        if (rr < 0 || rr > 7 || ff < 0 || ff > 7) continue;
        m[(56 + k) * 64 + sq] = mi.plain[sq][rr * 8 + ff];
      }
      if (r == 6) {
        for (int di = 0; di < 3; di++) {  // NW, N, NE
          int ff = f + di - 1;
          if (ff < 0 || ff > 7) continue;
          for (int pi = 0; pi < 3; pi++) m[(64 + di * 3 + pi) * 64 + sq] = mi.promo[f][ff][promo_piece[pi]];
        }
      }
    }
    return m;
  }();
  return map;
}

const std::vector<float>& PosEncoding() {
  static const std::vector<float> pe = [] {
    std::vector<float> v(64 * 64, 0.0f);
    const MoveIndex& mi = Moves();
    for (int f = 0; f < 64; f++)
      for (int t = 0; t < 64; t++) v[f * 64 + t] = f == t ? -1.0f : (mi.plain[f][t] >= 0 ? 1.0f : 0.0f);
    return v;
  }();
  return pe;
}

const std::vector<int16_t>& AttnPolicyInverseMap() {
  static const std::vector<int16_t> inv = Invert(AttnPolicyMap());
  return inv;
}

const std::vector<int16_t>& ConvPolicyInverseMap() {
  static const std::vector<int16_t> inv = Invert(ConvPolicyMap());
  return inv;
}

}  // namespace lc0mi

/*
 * TEST INFRASTRUCTURE -- CPU restatement of lc0's chess board, position
 * history, input-plane encoder and move->policy-index mapping, in plain C.
 * It exists to (a) generate seeded random-playout input positions and (b)
 * serve as the bit-exact checker for input planes and move indices.  It is
 * never linked into the shipped library.
 *
 * Follows (reference file:line):
 *   board model / Mirror            src/chess/board.cc:57-69, board.h:237-254
 *   GeneratePseudolegalMoves        src/chess/board.cc:430-575
 *   ApplyMove                       src/chess/board.cc:596-726
 *   IsUnderAttack                   src/chess/board.cc:728-760
 *   GenerateLegalMoves (semantics)  src/chess/board.cc:762-967
 *   SetFromFen                      src/chess/board.cc:977-1119
 *   ParseMove                       src/chess/board.cc:1154-1200
 *   Position / repetitions          src/chess/position.cc:40-46,105-130
 *   EncodePositionForNN             src/neural/encoder.cc:134-328
 *   ChooseTransform                 src/neural/encoder.cc:36-102
 *   bit transforms                  src/utils/bititer.h:64-89
 *   MoveToNNIndex                   src/neural/encoder.cc:574-619
 *
 * Pinned by: perft known answers (board_test.cc:127-183 and the Chess960
 * table), the repetition cases of position_test.cc and all ten cases of
 * encoder_test.cc; see tests/test_oracle_chess.py.
 */
#include <ctype.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef uint64_t u64;

typedef struct {
  u64 ours, theirs, rooks, bishops, pawns;
  uint8_t our_king, their_king;
  uint8_t castle; /* bit0 we 00, bit1 we 000, bit2 they 00, bit3 they 000 */
  uint8_t our_qrook, their_qrook, our_krook, their_krook; /* files */
  uint8_t flipped;
} Board;

typedef struct {
  Board b;
  int rule50, repetitions, cycle, ply;
} Position;

enum {
  MV_TO = 0x003f, MV_FROM = 0x0fc0, MV_SPECIAL = 0x7000, MV_CASTLING = 0x1000,
  MV_ENPASSANT = 0x2000, MV_PROMOTION = 0x4000, MV_PIECE = 0x3000
};
/* promotion piece ids: knight 0, queen 1, rook 2, bishop 3 (types.h:52-57) */
enum { P_KNIGHT = 0, P_QUEEN = 1, P_ROOK = 2, P_BISHOP = 3 };

#define BIT(sq) (1ULL << (sq))
#define SQ(file, rank) ((rank) * 8 + (file))
static const u64 kPawnMask = 0x00FFFFFFFFFFFF00ULL;

static u64 bswap64(u64 v) { return __builtin_bswap64(v); }

/* ---- bit transforms (bititer.h:64-89) ---- */
u64 orc_reverse_bits_in_bytes(u64 v) {
  v = ((v >> 1) & 0x5555555555555555ULL) | ((v & 0x5555555555555555ULL) << 1);
  v = ((v >> 2) & 0x3333333333333333ULL) | ((v & 0x3333333333333333ULL) << 2);
  v = ((v >> 4) & 0x0F0F0F0F0F0F0F0FULL) | ((v & 0x0F0F0F0F0F0F0F0FULL) << 4);
  return v;
}
u64 orc_reverse_bytes_in_bytes(u64 v) { return bswap64(v); }
/* Transpose across the diagonal that joins bit 7 and bit 56. */
u64 orc_transpose_bits_in_bytes(u64 v) {
  v = (v & 0xAA00AA00AA00AA00ULL) >> 9 | (v & 0x0055005500550055ULL) << 9 |
      (v & 0x55AA55AA55AA55AAULL);
  v = (v & 0xCCCC0000CCCC0000ULL) >> 18 | (v & 0x0000333300003333ULL) << 18 |
      (v & 0x3333CCCC3333CCCCULL);
  v = (v & 0xF0F0F0F000000000ULL) >> 36 | (v & 0x000000000F0F0F0FULL) << 36 |
      (v & 0x0F0F0F0FF0F0F0F0ULL);
  return v;
}

/* ---- attack tables built at first use ---- */
static u64 g_knight[64], g_pawn_att[64]; /* pawn_att: squares from which THEIR pawn attacks sq */
static int g_init = 0;
static void init_tables(void) {
  if (g_init) return;
  static const int kd[8][2] = {{1, 2}, {2, 1}, {2, -1}, {1, -2},
                               {-1, -2}, {-2, -1}, {-2, 1}, {-1, 2}};
  for (int s = 0; s < 64; s++) {
    int r = s / 8, f = s % 8;
    u64 k = 0;
    for (int i = 0; i < 8; i++) {
      int rr = r + kd[i][0], ff = f + kd[i][1];
      if (rr >= 0 && rr < 8 && ff >= 0 && ff < 8) k |= BIT(SQ(ff, rr));
    }
    g_knight[s] = k;
    /* Their pawns move down the board, so they attack sq from rank+1. */
    u64 p = 0;
    if (r + 1 < 8) {
      if (f > 0) p |= BIT(SQ(f - 1, r + 1));
      if (f < 7) p |= BIT(SQ(f + 1, r + 1));
    }
    g_pawn_att[s] = p;
  }
  g_init = 1;
}

static u64 ray_attacks(int sq, u64 occ, const int dirs[4][2]) {
  u64 a = 0;
  int r0 = sq / 8, f0 = sq % 8;
  for (int d = 0; d < 4; d++) {
    int r = r0 + dirs[d][0], f = f0 + dirs[d][1];
    while (r >= 0 && r < 8 && f >= 0 && f < 8) {
      u64 b = BIT(SQ(f, r));
      a |= b;
      if (occ & b) break;
      r += dirs[d][0];
      f += dirs[d][1];
    }
  }
  return a;
}
static const int kRookDirs[4][2] = {{1, 0}, {-1, 0}, {0, 1}, {0, -1}};
static const int kBishopDirs[4][2] = {{1, 1}, {-1, 1}, {1, -1}, {-1, -1}};
static u64 rook_attacks(int sq, u64 occ) { return ray_attacks(sq, occ, kRookDirs); }
static u64 bishop_attacks(int sq, u64 occ) { return ray_attacks(sq, occ, kBishopDirs); }

/* ---- board ---- */
void orc_board_mirror(Board* b) {
  u64 o = bswap64(b->ours), t = bswap64(b->theirs);
  b->ours = t;
  b->theirs = o;
  b->rooks = bswap64(b->rooks);
  b->bishops = bswap64(b->bishops);
  b->pawns = bswap64(b->pawns);
  uint8_t ok = b->our_king ^ 0x38, tk = b->their_king ^ 0x38;
  b->our_king = tk;
  b->their_king = ok;
  uint8_t t8;
  t8 = b->our_qrook; b->our_qrook = b->their_qrook; b->their_qrook = t8;
  t8 = b->our_krook; b->our_krook = b->their_krook; b->their_krook = t8;
  b->castle = (uint8_t)(((b->castle & 3) << 2) + ((b->castle & 12) >> 2));
  b->flipped = !b->flipped;
}

static void board_clear(Board* b) {
  memset(b, 0, sizeof(*b));
  b->our_qrook = 0; b->their_qrook = 0; b->our_krook = 7; b->their_krook = 7;
}

static int board_eq(const Board* a, const Board* b) {
  return a->ours == b->ours && a->theirs == b->theirs && a->rooks == b->rooks &&
         a->bishops == b->bishops && a->pawns == b->pawns &&
         a->our_king == b->our_king && a->their_king == b->their_king &&
         a->castle == b->castle && a->our_qrook == b->our_qrook &&
         a->their_qrook == b->their_qrook && a->our_krook == b->our_krook &&
         a->their_krook == b->their_krook && a->flipped == b->flipped;
}

int orc_is_under_attack(const Board* b, int sq) {
  init_tables();
  int r = sq / 8, f = sq % 8;
  int kr = b->their_king / 8, kf = b->their_king % 8;
  if (abs(kr - r) <= 1 && abs(kf - f) <= 1) return 1;
  u64 occ = b->ours | b->theirs;
  if (rook_attacks(sq, occ) & b->theirs & b->rooks) return 1;
  if (bishop_attacks(sq, occ) & b->theirs & b->bishops) return 1;
  if (g_pawn_att[sq] & b->theirs & b->pawns) return 1;
  u64 their_knights = b->theirs & ~BIT(b->their_king) & ~b->rooks & ~b->bishops &
                      ~(b->pawns & kPawnMask);
  if (g_knight[sq] & their_knights) return 1;
  return 0;
}

static int pop_lsb(u64* v) {
  int i = __builtin_ctzll(*v);
  *v &= *v - 1;
  return i;
}

static uint16_t mv(int from, int to) { return (uint16_t)((from << 6) | to); }

static int walk_free(const Board* b, int from, int to, int rook, int king) {
  for (int i = from; i <= to; i++) {
    if (i == rook || i == king) continue;
    if ((b->ours | b->theirs) & BIT(SQ(i, 0))) return 0;
  }
  return 1;
}
static int range_attacked(const Board* b, int from, int to) {
  if (from == to) return orc_is_under_attack(b, SQ(from, 0));
  int inc = from < to ? 1 : -1;
  while (from != to) {
    if (orc_is_under_attack(b, SQ(from, 0))) return 1;
    from += inc;
  }
  return 0;
}

/* Pseudolegal moves in the reference's emission order. Returns count. */
int orc_gen_pseudolegal(const Board* b, uint16_t* out) {
  init_tables();
  static const int kKing[8][2] = {{-1, -1}, {-1, 0}, {-1, 1}, {0, -1},
                                  {0, 1}, {1, -1}, {1, 0}, {1, 1}};
  static const int kPromo[4] = {P_QUEEN, P_ROOK, P_BISHOP, P_KNIGHT};
  int n = 0;
  u64 occ = b->ours | b->theirs;
  u64 it = b->ours;
  while (it) {
    int src = pop_lsb(&it);
    int r = src / 8, f = src % 8;
    if (src == b->our_king) {
      for (int i = 0; i < 8; i++) {
        int rr = r + kKing[i][0], ff = f + kKing[i][1];
        if (rr < 0 || rr > 7 || ff < 0 || ff > 7) continue;
        int dst = SQ(ff, rr);
        if (b->ours & BIT(dst)) continue;
        if (orc_is_under_attack(b, dst)) continue;
        out[n++] = mv(src, dst);
      }
      int king = f;
      if (b->castle & 2) {
        int q = b->our_qrook;
        int lo = q < 2 ? q : 2, hi = king > 3 ? king : 3;
        if (walk_free(b, lo, hi, q, king) && !range_attacked(b, king, 2))
          out[n++] = (uint16_t)((king << 6) | q | MV_CASTLING);
      }
      if (b->castle & 1) {
        int k = b->our_krook;
        int lo = king < 5 ? king : 5, hi = k > 6 ? k : 6;
        if (walk_free(b, lo, hi, k, king) && !range_attacked(b, king, 6))
          out[n++] = (uint16_t)((king << 6) | k | MV_CASTLING);
      }
      continue;
    }
    int processed = 0;
    if (b->rooks & BIT(src)) {
      processed = 1;
      u64 a = rook_attacks(src, occ) & ~b->ours;
      while (a) out[n++] = mv(src, pop_lsb(&a));
    }
    if (b->bishops & BIT(src)) {
      processed = 1;
      u64 a = bishop_attacks(src, occ) & ~b->ours;
      while (a) out[n++] = mv(src, pop_lsb(&a));
    }
    if (processed) continue;
    if ((b->pawns & kPawnMask) & BIT(src)) {
      int dr = r + 1;
      int dst = SQ(f, dr);
      if (!(occ & BIT(dst))) {
        if (dr != 7) {
          out[n++] = mv(src, dst);
          if (dr == 2) {
            int jump = SQ(f, 3);
            if (!(occ & BIT(jump))) out[n++] = mv(src, jump);
          }
        } else {
          for (int p = 0; p < 4; p++)
            out[n++] = (uint16_t)(mv(src, dst) | MV_PROMOTION | (kPromo[p] << 12));
        }
      }
      for (int dir = -1; dir <= 1; dir += 2) {
        int df = f + dir;
        if (df < 0 || df > 7) continue;
        int d2 = SQ(df, dr);
        if (b->theirs & BIT(d2)) {
          if (dr == 7) {
            for (int p = 0; p < 4; p++)
              out[n++] = (uint16_t)(mv(src, d2) | MV_PROMOTION | (kPromo[p] << 12));
          } else {
            out[n++] = mv(src, d2);
          }
        } else if (dr == 5 && (b->pawns & BIT(SQ(df, 7)))) {
          out[n++] = (uint16_t)(mv(src, d2) | MV_ENPASSANT);
        }
      }
      continue;
    }
    u64 a = g_knight[src] & ~b->ours;
    while (a) out[n++] = mv(src, pop_lsb(&a));
  }
  return n;
}

/* Applies a move for "ours"; returns 1 if the rule-50 counter resets. */
int orc_apply_move(Board* b, uint16_t m) {
  init_tables();
  int from = (m & MV_FROM) >> 6, to = m & MV_TO;
  int from_rank = from / 8, from_file = from % 8, to_rank = to / 8, to_file = to % 8;
  if (from == b->our_king) {
    b->castle &= (uint8_t)~3;
    if ((m & MV_SPECIAL) == MV_CASTLING) {
      int king_dst, rook_dst;
      if (to_file > from_file) { king_dst = 6; rook_dst = 5; }
      else { king_dst = 2; rook_dst = 3; }
      b->pawns &= kPawnMask;
      b->ours &= ~BIT(b->our_king);
      b->ours &= ~BIT(to);
      b->rooks &= ~BIT(to);
      b->our_king = (uint8_t)SQ(king_dst, 0);
      b->ours |= BIT(b->our_king);
      b->ours |= BIT(SQ(rook_dst, 0));
      b->rooks |= BIT(SQ(rook_dst, 0));
      return 0;
    }
  }
  b->ours &= ~BIT(from);
  b->ours |= BIT(to);
  int reset50 = (b->theirs & BIT(to)) != 0;
  if (reset50) {
    b->theirs &= ~BIT(to);
    b->rooks &= ~BIT(to);
    b->bishops &= ~BIT(to);
    b->pawns &= ~BIT(to);
    if (to == SQ(b->their_krook, 7)) b->castle &= (uint8_t)~4;
    if (to == SQ(b->their_qrook, 7)) b->castle &= (uint8_t)~8;
  }
  if ((m & MV_SPECIAL) == MV_ENPASSANT && !(m & MV_PROMOTION)) {
    int ep = SQ(to_file, 4);
    b->pawns &= ~BIT(ep);
    b->theirs &= ~BIT(ep);
  }
  b->pawns &= kPawnMask;
  reset50 |= (b->pawns & BIT(from)) != 0;
  if (from == b->our_king) {
    b->our_king = (uint8_t)to;
    return reset50;
  }
  if (m & MV_PROMOTION) {
    int p = (m & MV_PIECE) >> 12;
    if (p == P_ROOK) b->rooks |= BIT(to);
    else if (p == P_BISHOP) b->bishops |= BIT(to);
    else if (p == P_QUEEN) { b->rooks |= BIT(to); b->bishops |= BIT(to); }
    b->pawns &= ~BIT(from);
    return 1;
  }
  if (from_rank == 0 && (b->rooks & BIT(from))) {
    if (from_file == b->our_qrook) b->castle &= (uint8_t)~2;
    if (from_file == b->our_krook) b->castle &= (uint8_t)~1;
  }
  if (b->rooks & BIT(from)) b->rooks |= BIT(to);
  if (b->bishops & BIT(from)) b->bishops |= BIT(to);
  if (b->pawns & BIT(from)) b->pawns |= BIT(to);
  b->rooks &= ~BIT(from);
  b->bishops &= ~BIT(from);
  b->pawns &= ~BIT(from);
  if (to_rank - from_rank == 2 && (b->pawns & BIT(to))) {
    int ep_sq = SQ(to_file, to_rank - 1);
    if (g_pawn_att[ep_sq] & b->theirs & b->pawns) b->pawns |= BIT(SQ(to_file, 0));
  }
  return reset50;
}

/* Legal moves = pseudolegal moves that do not leave our king attacked
 * (same set and order as GenerateLegalMoves, board.cc:959-967). */
int orc_gen_legal(const Board* b, uint16_t* out) {
  uint16_t tmp[256];
  int n = orc_gen_pseudolegal(b, tmp), k = 0;
  for (int i = 0; i < n; i++) {
    Board c = *b;
    orc_apply_move(&c, tmp[i]);
    if (!orc_is_under_attack(&c, c.our_king)) out[k++] = tmp[i];
  }
  return k;
}

static void put_piece(Board* b, int sq, char piece, int theirs) {
  if (theirs) b->theirs |= BIT(sq); else b->ours |= BIT(sq);
  if (piece == 'k') { if (theirs) b->their_king = (uint8_t)sq; else b->our_king = (uint8_t)sq; }
  if (piece == 'p') b->pawns |= BIT(sq);
  if (piece == 'r' || piece == 'q') b->rooks |= BIT(sq);
  if (piece == 'b' || piece == 'q') b->bishops |= BIT(sq);
}

static int skip_ws(const char* fen, size_t len, size_t* pos) {
  while (*pos < len && fen[*pos] == ' ') ++*pos;
  return *pos == len;
}

/* Returns 0 on success, negative on a malformed FEN. */
int orc_board_from_fen(Board* b, const char* fen, int* rule50, int* moves) {
  board_clear(b);
  if (rule50) *rule50 = 0;
  if (moves) *moves = 1;
  size_t len = strlen(fen), pos = 0;
  int rank = 7, file = 0;
  skip_ws(fen, len, &pos);
  for (; pos < len; ++pos) {
    char c = fen[pos];
    if (c == ' ') break;
    if (c == '/') { if (rank == 0) return -1; --rank; file = 0; continue; }
    if (c >= '1' && c <= '8') { file += c - '0'; if (file > 8) return -2; continue; }
    char lc = (char)tolower(c);
    if (!strchr("nqrbpk", lc)) return -3;
    if (file > 7 || rank < 0) return -4;
    if (lc == 'p' && (rank == 0 || rank == 7)) return -5;
    put_piece(b, SQ(file, rank), lc, islower(c) != 0);
    ++file;
  }
  if (skip_ws(fen, len, &pos)) return 0;
  char stm = (char)tolower(fen[pos++]);
  if (stm == 'b') orc_board_mirror(b);
  else if (stm != 'w') return -6;
  if (skip_ws(fen, len, &pos)) return 0;
  if (fen[pos] == '-') {
    ++pos;
  } else {
    for (; pos < len; ++pos) {
      char c = fen[pos];
      if (c == ' ') break;
      int theirs = (isupper(c) != 0) == (b->flipped != 0);
      int kingside = 0, f = -1;
      int kfile = (theirs ? b->their_king : b->our_king) % 8;
      if (c == 'K' || c == 'Q' || c == 'k' || c == 'q') {
        kingside = tolower(c) == 'k';
        int rk = theirs ? 7 : 0;
        u64 pure_rooks = b->rooks & ~b->bishops;
        for (int ff = kingside ? 7 : 0; ff != kfile; kingside ? --ff : ++ff) {
          int sq = SQ(ff, rk);
          if (!(pure_rooks & BIT(sq))) continue;
          if ((theirs ? b->theirs : b->ours) & BIT(sq)) { f = ff; break; }
        }
        if (f < 0) return -7;
      } else {
        f = tolower(c) - 'a';
        if (f < 0 || f > 7) return -8;
        kingside = f > kfile;
      }
      if (kingside && theirs) { b->castle |= 4; b->their_krook = (uint8_t)f; }
      else if (kingside && !theirs) { b->castle |= 1; b->our_krook = (uint8_t)f; }
      else if (!kingside && theirs) { b->castle |= 8; b->their_qrook = (uint8_t)f; }
      else { b->castle |= 2; b->our_qrook = (uint8_t)f; }
    }
  }
  if (skip_ws(fen, len, &pos)) return 0;
  if (fen[pos] == '-') {
    ++pos;
  } else {
    if (pos + 2 >= len) return -9;
    int f = tolower(fen[pos]) - 'a', r = fen[pos + 1] - '1';
    if (f < 0 || f > 7 || r < 0 || r > 7) return -10;
    if (r != (b->flipped ? 2 : 5)) return -11;
    if ((b->ours | b->theirs) & BIT(SQ(f, 5))) return -12;
    if (!(b->theirs & b->pawns & kPawnMask & BIT(SQ(f, 4)))) return -13;
    b->pawns |= BIT(SQ(f, 7));
    pos += 2;
  }
  if (skip_ws(fen, len, &pos)) return 0;
  char* end;
  long v = strtol(fen + pos, &end, 10);
  if (end == fen + pos) return -14;
  if (rule50) *rule50 = (int)v;
  pos = (size_t)(end - fen);
  if (skip_ws(fen, len, &pos)) return 0;
  v = strtol(fen + pos, &end, 10);
  if (end == fen + pos) return -15;
  if (moves) *moves = (int)v;
  pos = (size_t)(end - fen);
  if (!skip_ws(fen, len, &pos)) return -16;
  return 0;
}

/* Move text in normal (white-at-bottom) notation -> move from the mover's
 * point of view. Returns 0xffff on error. */
uint16_t orc_parse_move(const Board* b, const char* s) {
  size_t n = strlen(s);
  if (n < 4 || n > 5) return 0xffff;
  int ff = tolower(s[0]) - 'a', fr = s[1] - '1', tf = tolower(s[2]) - 'a', tr = s[3] - '1';
  if (ff < 0 || ff > 7 || fr < 0 || fr > 7 || tf < 0 || tf > 7 || tr < 0 || tr > 7) return 0xffff;
  if (b->flipped) { fr ^= 7; tr ^= 7; }
  int from = SQ(ff, fr), to = SQ(tf, tr);
  if (!(b->ours & BIT(from))) return 0xffff;
  if ((b->pawns & BIT(from)) && (fr != 0 && fr != 7) && (tr == 0 || tr == 7)) {
    int p = P_KNIGHT;
    if (n > 4) {
      switch (tolower(s[4])) {
        case 'n': p = P_KNIGHT; break;
        case 'q': p = P_QUEEN; break;
        case 'r': p = P_ROOK; break;
        case 'b': p = P_BISHOP; break;
        default: return 0xffff;
      }
    }
    return (uint16_t)(mv(from, to) | MV_PROMOTION | (p << 12));
  }
  if (from == b->our_king && (b->ours & BIT(to)))
    return (uint16_t)((ff << 6) | tf | MV_CASTLING);
  if (from == b->our_king && from == 4 && to == 6) return (uint16_t)((ff << 6) | 7 | MV_CASTLING);
  if (from == b->our_king && from == 4 && to == 2) return (uint16_t)((ff << 6) | 0 | MV_CASTLING);
  if (ff != tf && (b->pawns & kPawnMask & BIT(from)) && !(b->theirs & BIT(to)))
    return (uint16_t)(mv(from, to) | MV_ENPASSANT);
  return mv(from, to);
}

/* Move (mover's view) -> UCI text in normal notation; castling printed as the
 * classical e1g1/e1c1 when the king stands on the e-file (types.h:231-243). */
void orc_move_to_uci(uint16_t m, int black_to_move, char out[6]) {
  int from = (m & MV_FROM) >> 6, to = m & MV_TO;
  if (black_to_move) { from ^= 0x38; to ^= 0x38; }
  int tf = to % 8;
  if ((m & MV_SPECIAL) == MV_CASTLING && !(m & MV_PROMOTION) && from % 8 == 4) {
    if (tf == 0) tf = 2; else if (tf == 7) tf = 6;
  }
  out[0] = (char)('a' + from % 8); out[1] = (char)('1' + from / 8);
  out[2] = (char)('a' + tf); out[3] = (char)('1' + to / 8);
  out[4] = 0; out[5] = 0;
  if (m & MV_PROMOTION) out[4] = "nqrb"[(m & MV_PIECE) >> 12];
}

uint64_t orc_perft(const Board* b, int depth) {
  if (depth == 0) return 1;
  uint16_t moves[256];
  int n = orc_gen_legal(b, moves);
  if (depth == 1) return (uint64_t)n;
  uint64_t total = 0;
  for (int i = 0; i < n; i++) {
    Board c = *b;
    orc_apply_move(&c, moves[i]);
    orc_board_mirror(&c);
    total += orc_perft(&c, depth - 1);
  }
  return total;
}

/* ---- position history ---- */
typedef struct {
  Position* pos;
  int n, cap;
} History;

History* orc_history_new(void) {
  History* h = (History*)calloc(1, sizeof(History));
  h->cap = 64;
  h->pos = (Position*)calloc((size_t)h->cap, sizeof(Position));
  return h;
}
void orc_history_free(History* h) { if (h) { free(h->pos); free(h); } }
int orc_history_len(const History* h) { return h->n; }
const Position* orc_history_at(const History* h, int i) { return &h->pos[i]; }
const Board* orc_history_last_board(const History* h) { return &h->pos[h->n - 1].b; }

void orc_history_reset(History* h, const Board* b, int rule50, int ply) {
  h->n = 1;
  memset(&h->pos[0], 0, sizeof(Position));
  h->pos[0].b = *b;
  h->pos[0].rule50 = rule50;
  h->pos[0].ply = ply;
}

int orc_history_reset_fen(History* h, const char* fen) {
  Board b;
  int r50, mvs;
  int rc = orc_board_from_fen(&b, fen, &r50, &mvs);
  if (rc) return rc;
  orc_history_reset(h, &b, r50, 2 * mvs - (b.flipped ? 1 : 2));
  return 0;
}

/* position.cc:40-46 (child position) and :105-130 (repetitions). */
void orc_history_append(History* h, uint16_t m) {
  if (h->n == h->cap) {
    h->cap *= 2;
    h->pos = (Position*)realloc(h->pos, (size_t)h->cap * sizeof(Position));
  }
  const Position* parent = &h->pos[h->n - 1];
  Position p;
  memset(&p, 0, sizeof(p));
  p.b = parent->b;
  p.rule50 = parent->rule50 + 1;
  p.ply = parent->ply + 1;
  int zeroing = orc_apply_move(&p.b, m);
  orc_board_mirror(&p.b);
  if (zeroing) p.rule50 = 0;
  h->pos[h->n++] = p;
  Position* last = &h->pos[h->n - 1];
  last->repetitions = 0;
  last->cycle = 0;
  if (last->rule50 < 4) return;
  for (int idx = h->n - 5; idx >= 0; idx -= 2) {
    const Position* q = &h->pos[idx];
    if (board_eq(&q->b, &last->b)) {
      last->cycle = h->n - 1 - idx;
      last->repetitions = 1 + q->repetitions;
      return;
    }
    if (q->rule50 < 2) return;
  }
}

int orc_history_did_repeat_since_zeroing(const History* h) {
  for (int i = h->n - 1; i >= 0; i--) {
    if (h->pos[i].repetitions > 0) return 1;
    if (h->pos[i].rule50 == 0) return 0;
  }
  return 0;
}

/* ---- encoder ---- */
enum { T_NONE = 0, T_FLIP = 1, T_MIRROR = 2, T_TRANSPOSE = 4 };
enum {
  IN_CLASSICAL = 1, IN_CASTLING_PLANE = 2, IN_CANON = 3, IN_CANON_HECTO = 4,
  IN_CANON_HECTO_ARMA = 132, IN_CANON_V2 = 5, IN_CANON_V2_ARMA = 133
};
enum { FILL_NO = 0, FILL_FEN_ONLY = 1, FILL_ALWAYS = 2 };

static u64 bd_pawns(const Board* b) { return b->pawns & kPawnMask; }
static u64 bd_enpassant(const Board* b) { return b->pawns & ~kPawnMask; }
static u64 bd_bishops(const Board* b) { return b->bishops & ~b->rooks; }
static u64 bd_rooks(const Board* b) { return b->rooks & ~b->bishops; }
static u64 bd_queens(const Board* b) { return b->rooks & b->bishops; }
static u64 bd_kings(const Board* b) { return BIT(b->our_king) | BIT(b->their_king); }
static u64 bd_knights(const Board* b) {
  return (b->ours | b->theirs) & ~bd_pawns(b) & ~BIT(b->our_king) & ~BIT(b->their_king) &
         ~b->rooks & ~b->bishops;
}

static int compare_transposing(u64 value, int initial) {
  if (initial & T_FLIP) value = orc_reverse_bits_in_bytes(value);
  if (initial & T_MIRROR) value = orc_reverse_bytes_in_bytes(value);
  u64 alt = orc_transpose_bits_in_bytes(value);
  if (value < alt) return -1;
  if (value > alt) return 1;
  return 0;
}

int orc_choose_transform(const Board* b) {
  if (b->castle != 0) return 0;
  u64 our_king = BIT(b->our_king);
  int t = T_NONE;
  if (our_king & 0x0F0F0F0F0F0F0F0FULL) { t |= T_FLIP; our_king = orc_reverse_bits_in_bytes(our_king); }
  if (bd_pawns(b) != 0) return t;
  if (our_king & 0xFFFFFFFF00000000ULL) { t |= T_MIRROR; our_king = orc_reverse_bytes_in_bytes(our_king); }
  if (our_king & 0xE0C08000ULL) {
    t |= T_TRANSPOSE;
  } else if (our_king & 0x10204080ULL) {
    u64 seq[7] = {b->ours | b->theirs, b->ours, bd_kings(b), bd_queens(b),
                  bd_rooks(b), bd_knights(b), bd_bishops(b)};
    for (int i = 0; i < 7; i++) {
      int o = compare_transposing(seq[i], t);
      if (o == -1) return t;
      if (o == 1) return t | T_TRANSPOSE;
    }
  }
  return t;
}

static int is_canonical(int fmt) { return fmt >= IN_CANON; }
static int is_canonical_armageddon(int fmt) { return fmt == IN_CANON_HECTO_ARMA || fmt == IN_CANON_V2_ARMA; }
static int is_hectoplies(int fmt) { return fmt >= IN_CANON_HECTO; }

static Board g_startpos;
static int g_startpos_init = 0;

/* Writes 112 masks and 112 values. Returns 0, or -1 for an unknown format. */
int orc_encode_position(const History* h, int input_format, int history_planes,
                        int fill_empty, u64 masks[112], float values[112],
                        int* transform_out) {
  if (!g_startpos_init) {
    orc_board_from_fen(&g_startpos, "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1", 0, 0);
    g_startpos_init = 1;
  }
  const int kAux = 104;
  for (int i = 0; i < 112; i++) { masks[i] = 0; values[i] = 1.0f; }
  int transform = 0;
  int stop_early = is_canonical(input_format);
  uint8_t castle0 = 0;
  {
    const Position* lastp = &h->pos[h->n - 1];
    const Board* b = &lastp->b;
    int we_are_black = b->flipped;
    if (is_canonical(input_format)) transform = orc_choose_transform(b);
    switch (input_format) {
      case IN_CLASSICAL:
        if (b->castle & 2) masks[kAux + 0] = ~0ULL;
        if (b->castle & 1) masks[kAux + 1] = ~0ULL;
        if (b->castle & 8) masks[kAux + 2] = ~0ULL;
        if (b->castle & 4) masks[kAux + 3] = ~0ULL;
        break;
      case IN_CASTLING_PLANE: case IN_CANON: case IN_CANON_HECTO:
      case IN_CANON_HECTO_ARMA: case IN_CANON_V2: case IN_CANON_V2_ARMA:
        masks[kAux + 0] = ((b->castle & 2) ? BIT(SQ(b->our_qrook, 0)) : 0) |
                          ((b->castle & 8) ? BIT(SQ(b->their_qrook, 7)) : 0);
        masks[kAux + 1] = ((b->castle & 1) ? BIT(SQ(b->our_krook, 0)) : 0) |
                          ((b->castle & 4) ? BIT(SQ(b->their_krook, 7)) : 0);
        break;
      default:
        return -1;
    }
    if (is_canonical(input_format)) masks[kAux + 4] = bd_enpassant(b);
    else if (we_are_black) masks[kAux + 4] = ~0ULL;
    masks[kAux + 5] = ~0ULL;
    values[kAux + 5] = is_hectoplies(input_format) ? lastp->rule50 / 100.0f : (float)lastp->rule50;
    if (is_canonical_armageddon(input_format) && we_are_black) masks[kAux + 6] = ~0ULL;
    masks[kAux + 7] = ~0ULL;
    if (stop_early) castle0 = b->castle;
  }
  int skip_non_repeats = input_format == IN_CANON_V2 || input_format == IN_CANON_V2_ARMA;
  int flip = 0;
  int hidx = h->n - 1;
  int nplanes = history_planes < 8 ? history_planes : 8;
  for (int i = 0; i < nplanes; ++i, --hidx) {
    const Position* position = &h->pos[hidx < 0 ? 0 : hidx];
    Board board = position->b;
    if (flip) orc_board_mirror(&board);
    if (stop_early && board.castle != castle0) break;
    if (stop_early && hidx != h->n - 1 && bd_enpassant(&board) != 0) break;
    if (fill_empty == FILL_NO && (hidx < -1 || (hidx == -1 && bd_enpassant(&board) == 0))) break;
    if (hidx < 0 && fill_empty == FILL_FEN_ONLY && board_eq(&position->b, &g_startpos)) break;
    int reps = position->repetitions;
    if (skip_non_repeats && reps == 0 && i > 0) {
      if (hidx > 0) flip = !flip;
      if (position->rule50 == 0) break;
      --i;
      continue;
    }
    int base = i * 13;
    masks[base + 0] = board.ours & bd_pawns(&board);
    masks[base + 1] = board.ours & bd_knights(&board);
    masks[base + 2] = board.ours & bd_bishops(&board);
    masks[base + 3] = board.ours & bd_rooks(&board);
    masks[base + 4] = board.ours & bd_queens(&board);
    masks[base + 5] = board.ours & bd_kings(&board);
    masks[base + 6] = board.theirs & bd_pawns(&board);
    masks[base + 7] = board.theirs & bd_knights(&board);
    masks[base + 8] = board.theirs & bd_bishops(&board);
    masks[base + 9] = board.theirs & bd_rooks(&board);
    masks[base + 10] = board.theirs & bd_queens(&board);
    masks[base + 11] = board.theirs & bd_kings(&board);
    if (reps >= 1) masks[base + 12] = ~0ULL;
    if (hidx < 0 && bd_enpassant(&board) != 0) {
      int idx = __builtin_ctzll(bd_enpassant(&board));
      if (idx < 8) masks[base + 0] += ((0x0000000000000100ULL - 0x0000000001000000ULL) << idx);
      else masks[base + 6] += ((0x0001000000000000ULL - 0x0000000100000000ULL) << (idx - 56));
    }
    if (hidx > 0) flip = !flip;
    if (stop_early && position->rule50 == 0) break;
  }
  if (transform != T_NONE) {
    for (int i = 0; i <= kAux + 4; i++) {
      u64 v = masks[i];
      if (v == 0 || v == ~0ULL) continue;
      if (transform & T_FLIP) v = orc_reverse_bits_in_bytes(v);
      if (transform & T_MIRROR) v = orc_reverse_bytes_in_bytes(v);
      if (transform & T_TRANSPOSE) v = orc_transpose_bits_in_bytes(v);
      masks[i] = v;
    }
  }
  if (transform_out) *transform_out = transform;
  return 0;
}

/* ---- move -> NN index (encoder.cc:339-619) ----
 * The 1858-entry move list in closed form: every (from,to) pair that is a
 * queen-line or knight move, ascending by (from,to); then, for each from-file
 * on rank 7 and each to-file within one step on rank 8, promotions q, r, b.
 * Knight promotion shares the index of the plain move. */
static int16_t g_packed_to_nn[4 * 4096];
static char g_move_strs[1858][6];
static int g_nn_init = 0;
static void init_nn_index(void) {
  if (g_nn_init) return;
  for (int i = 0; i < 4 * 4096; i++) g_packed_to_nn[i] = -1;
  int idx = 0;
  for (int from = 0; from < 64; from++)
    for (int to = 0; to < 64; to++) {
      if (from == to) continue;
      int dr = abs(to / 8 - from / 8), df = abs(to % 8 - from % 8);
      int queen = (dr == 0 || df == 0 || dr == df);
      int knight = (dr == 1 && df == 2) || (dr == 2 && df == 1);
      if (!queen && !knight) continue;
      g_packed_to_nn[from * 64 + to] = (int16_t)idx;
      char* s = g_move_strs[idx];
      s[0] = (char)('a' + from % 8); s[1] = (char)('1' + from / 8);
      s[2] = (char)('a' + to % 8); s[3] = (char)('1' + to / 8); s[4] = 0;
      idx++;
    }
  static const int promo_piece[3] = {P_QUEEN, P_ROOK, P_BISHOP};
  static const char promo_char[3] = {'q', 'r', 'b'};
  for (int ff = 0; ff < 8; ff++)
    for (int tf = ff - 1; tf <= ff + 1; tf++) {
      if (tf < 0 || tf > 7) continue;
      for (int p = 0; p < 3; p++) {
        int from = SQ(ff, 6), to = SQ(tf, 7);
        g_packed_to_nn[promo_piece[p] * 4096 + from * 64 + to] = (int16_t)idx;
        char* s = g_move_strs[idx];
        s[0] = (char)('a' + ff); s[1] = '7'; s[2] = (char)('a' + tf); s[3] = '8';
        s[4] = promo_char[p]; s[5] = 0;
        idx++;
      }
    }
  g_nn_init = 1;
}

const char* orc_move_str(int idx) { init_nn_index(); return g_move_strs[idx]; }

static int transform_square(int sq, int t) {
  int f = sq % 8, r = sq / 8;
  if (t & (T_MIRROR | T_TRANSPOSE)) r ^= 7;
  if (t & (T_FLIP | T_TRANSPOSE)) f ^= 7;
  return SQ(f, r);
}

static int packed_int(uint16_t m) {
  return (m & MV_PROMOTION) ? (m & (0x0fff | MV_PIECE)) : (m & 0x0fff);
}

int orc_move_to_nn_index(uint16_t m, int transform) {
  init_nn_index();
  if (transform == 0) return g_packed_to_nn[packed_int(m)];
  int from = transform_square((m & MV_FROM) >> 6, transform);
  int to = transform_square(m & MV_TO, transform);
  uint16_t t = (m & MV_PROMOTION) ? (uint16_t)(mv(from, to) | MV_PROMOTION | (m & MV_PIECE))
                                  : mv(from, to);
  return g_packed_to_nn[packed_int(t)];
}

/* ---- seeded random playouts ---- */
static u64 splitmix64(u64* s) {
  u64 z = (*s += 0x9E3779B97F4A7C15ULL);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

/* Plays `plies` uniformly random legal moves from the start position (plies
 * drawn from U{10..80} by the same generator); if the game ends early the
 * whole game is redrawn, also when the final position is mate or stalemate.
 * UCI moves are appended to `uci` separated by spaces.
 * Returns the number of plies played. */
int orc_random_playout(History* h, u64* rng_state, char* uci, int uci_cap) {
  Board start;
  orc_board_from_fen(&start, "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1", 0, 0);
  for (;;) {
    int plies = 10 + (int)(splitmix64(rng_state) % 71);
    orc_history_reset(h, &start, 0, 0);
    int len = 0, ok = 1;
    if (uci_cap > 0) uci[0] = 0;
    for (int p = 0; p < plies; p++) {
      uint16_t moves[256];
      const Board* b = orc_history_last_board(h);
      int n = orc_gen_legal(b, moves);
      if (n == 0) { ok = 0; break; }
      uint16_t m = moves[splitmix64(rng_state) % (u64)n];
      char s[6];
      orc_move_to_uci(m, b->flipped, s);
      int sl = (int)strlen(s);
      if (len + sl + 2 < uci_cap) {
        if (len) uci[len++] = ' ';
        memcpy(uci + len, s, (size_t)sl + 1);
        len += sl;
      }
      orc_history_append(h, m);
    }
    if (ok) {
      /* A finished game is never sent to the network: redraw it too. */
      uint16_t moves[256];
      if (orc_gen_legal(orc_history_last_board(h), moves) > 0) return plies;
    }
  }
}

int orc_sizeof_board(void) { return (int)sizeof(Board); }
int orc_sizeof_position(void) { return (int)sizeof(Position); }

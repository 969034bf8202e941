#include "chess.hpp"

#include <cstdlib>
#include <cstring>
#include <mutex>

namespace crl {

static inline bool is_white(uint8_t p) { return p >= WP && p <= WK; }
static inline bool is_black(uint8_t p) { return p >= BP; }
static inline int file_of(int s) { return s & 7; }
static inline int rank_of(int s) { return s >> 3; }
static inline bool on_board(int f, int r) { return f >= 0 && f < 8 && r >= 0 && r < 8; }

static const int KNIGHT_D[8][2] = {{1, 2}, {2, 1}, {2, -1}, {1, -2}, {-1, -2}, {-2, -1}, {-2, 1}, {-1, 2}};
static const int KING_D[8][2] = {{1, 0}, {1, 1}, {0, 1}, {-1, 1}, {-1, 0}, {-1, -1}, {0, -1}, {1, -1}};
static const int ROOK_D[4][2] = {{1, 0}, {-1, 0}, {0, 1}, {0, -1}};
static const int BISHOP_D[4][2] = {{1, 1}, {1, -1}, {-1, 1}, {-1, -1}};

void Board::set_start() {
  set_fen("rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1");
}

static int piece_from_char(char c) {
  switch (c) {
    case 'P': return WP; case 'N': return WN; case 'B': return WB;
    case 'R': return WR; case 'Q': return WQ; case 'K': return WK;
    case 'p': return BP; case 'n': return BN; case 'b': return BB;
    case 'r': return BR; case 'q': return BQ; case 'k': return BK;
  }
  return -1;
}
static const char PIECE_CHARS[] = ".PNBRQKpnbrqk";

static int fail(std::string* err, const char* msg) {
  if (err) *err = msg;
  return -1;
}

int Board::set_fen(const char* fen, std::string* err) {
  if (!fen) return fail(err, "null FEN");
  std::vector<std::string> parts;
  {
    std::string cur;
    for (const char* p = fen;; ++p) {
      if (*p == ' ' || *p == '\t' || *p == '\n' || *p == 0) {
        if (!cur.empty()) parts.push_back(cur);
        cur.clear();
        if (*p == 0) break;
      } else {
        cur.push_back(*p);
      }
    }
  }
  if (parts.empty() || parts.size() > 6) return fail(err, "FEN needs 1 to 6 fields");
  std::memset(sq, 0, sizeof(sq));
  int r = 7, f = 0;
  for (char c : parts[0]) {
    if (c == '/') {
      if (f != 8) return fail(err, "FEN rank does not have 8 files");
      --r; f = 0;
      if (r < 0) return fail(err, "FEN has more than 8 ranks");
    } else if (c >= '1' && c <= '8') {
      f += c - '0';
      if (f > 8) return fail(err, "FEN rank overflows");
    } else {
      int pc = piece_from_char(c);
      if (pc < 0) return fail(err, "FEN has an unknown piece letter");
      if (f >= 8) return fail(err, "FEN rank overflows");
      sq[r * 8 + f] = (uint8_t)pc;
      ++f;
    }
  }
  if (r != 0 || f != 8) return fail(err, "FEN board field is incomplete");
  white_to_move = 1; castling = 0; ep = -1; halfmove = 0; fullmove = 1;
  if (parts.size() > 1) {
    if (parts[1] == "w") white_to_move = 1;
    else if (parts[1] == "b") white_to_move = 0;
    else return fail(err, "FEN side-to-move field must be w or b");
  }
  if (parts.size() > 2 && parts[2] != "-") {
    for (char c : parts[2]) {
      switch (c) {
        case 'K': castling |= CR_WK; break;
        case 'Q': castling |= CR_WQ; break;
        case 'k': castling |= CR_BK; break;
        case 'q': castling |= CR_BQ; break;
        default: return fail(err, "FEN castling field must use KQkq or -");
      }
    }
  }
  if (parts.size() > 3 && parts[3] != "-") {
    const std::string& e = parts[3];
    if (e.size() != 2 || e[0] < 'a' || e[0] > 'h' || (e[1] != '3' && e[1] != '6'))
      return fail(err, "FEN en-passant field is not a square on rank 3 or 6");
    ep = (int8_t)((e[1] - '1') * 8 + (e[0] - 'a'));
  }
  if (parts.size() > 4) {
    char* end = nullptr;
    long v = std::strtol(parts[4].c_str(), &end, 10);
    if (*end || v < 0) return fail(err, "FEN halfmove clock is not a non-negative integer");
    halfmove = (int32_t)v;
  }
  if (parts.size() > 5) {
    char* end = nullptr;
    long v = std::strtol(parts[5].c_str(), &end, 10);
    if (*end || v < 0) return fail(err, "FEN fullmove number is not a non-negative integer");
    fullmove = (int32_t)(v < 1 ? 1 : v);
  }
  return 0;
}

uint8_t Board::clean_castling() const {
  uint8_t c = castling;
  if (sq[4] != WK) c &= ~(CR_WK | CR_WQ);
  if (sq[60] != BK) c &= ~(CR_BK | CR_BQ);
  if (sq[7] != WR) c &= ~CR_WK;
  if (sq[0] != WR) c &= ~CR_WQ;
  if (sq[63] != BR) c &= ~CR_BK;
  if (sq[56] != BR) c &= ~CR_BQ;
  return c;
}

bool Board::attacked(int s, bool by_white) const {
  const int f = file_of(s), r = rank_of(s);
  // Pawns: a white pawn on (f±1, r-1) attacks s.
  const int pr = by_white ? r - 1 : r + 1;
  const uint8_t pawn = by_white ? WP : BP;
  if (pr >= 0 && pr < 8) {
    if (f > 0 && sq[pr * 8 + f - 1] == pawn) return true;
    if (f < 7 && sq[pr * 8 + f + 1] == pawn) return true;
  }
  const uint8_t kn = by_white ? WN : BN, kg = by_white ? WK : BK;
  for (auto& d : KNIGHT_D) {
    int nf = f + d[0], nr = r + d[1];
    if (on_board(nf, nr) && sq[nr * 8 + nf] == kn) return true;
  }
  for (auto& d : KING_D) {
    int nf = f + d[0], nr = r + d[1];
    if (on_board(nf, nr) && sq[nr * 8 + nf] == kg) return true;
  }
  const uint8_t rk = by_white ? WR : BR, bs = by_white ? WB : BB, qn = by_white ? WQ : BQ;
  for (auto& d : ROOK_D) {
    int nf = f + d[0], nr = r + d[1];
    while (on_board(nf, nr)) {
      uint8_t p = sq[nr * 8 + nf];
      if (p) { if (p == rk || p == qn) return true; break; }
      nf += d[0]; nr += d[1];
    }
  }
  for (auto& d : BISHOP_D) {
    int nf = f + d[0], nr = r + d[1];
    while (on_board(nf, nr)) {
      uint8_t p = sq[nr * 8 + nf];
      if (p) { if (p == bs || p == qn) return true; break; }
      nf += d[0]; nr += d[1];
    }
  }
  return false;
}

bool Board::in_check() const {
  const uint8_t kg = white_to_move ? WK : BK;
  for (int s = 0; s < 64; ++s)
    if (sq[s] == kg) return attacked(s, !white_to_move);
  return false;
}

static inline void push_move(std::vector<Move>& out, int from, int to, int promo, int flag) {
  out.push_back(Move{(uint8_t)from, (uint8_t)to, (uint8_t)promo, (uint8_t)flag});
}

void Board::pseudo_legal(std::vector<Move>& out) const {
  const bool w = white_to_move;
  for (int s = 0; s < 64; ++s) {
    const uint8_t p = sq[s];
    if (!p || (w ? !is_white(p) : !is_black(p))) continue;
    const int f = file_of(s), r = rank_of(s);
    const int kind = w ? p : p - 6;  // 1..6
    switch (kind) {
      case 1: {  // pawn
        const int dir = w ? 1 : -1, start = w ? 1 : 6, last = w ? 7 : 0;
        const int nr = r + dir;
        if (nr < 0 || nr > 7) break;
        if (!sq[nr * 8 + f]) {
          if (nr == last) { for (int pr = 4; pr >= 1; --pr) push_move(out, s, nr * 8 + f, pr, 0); }
          else {
            push_move(out, s, nr * 8 + f, 0, 0);
            if (r == start && !sq[(nr + dir) * 8 + f]) push_move(out, s, (nr + dir) * 8 + f, 0, 1);
          }
        }
        for (int df = -1; df <= 1; df += 2) {
          const int nf = f + df;
          if (nf < 0 || nf > 7) continue;
          const int t = nr * 8 + nf;
          const uint8_t q = sq[t];
          if (q && (w ? is_black(q) : is_white(q))) {
            if (nr == last) { for (int pr = 4; pr >= 1; --pr) push_move(out, s, t, pr, 0); }
            else push_move(out, s, t, 0, 0);
          } else if (!q && t == ep && r == (w ? 4 : 3) && sq[r * 8 + nf] == (w ? BP : WP)) {
            push_move(out, s, t, 0, 2);
          }
        }
        break;
      }
      case 2:
        for (auto& d : KNIGHT_D) {
          int nf = f + d[0], nr = r + d[1];
          if (!on_board(nf, nr)) continue;
          uint8_t q = sq[nr * 8 + nf];
          if (!q || (w ? is_black(q) : is_white(q))) push_move(out, s, nr * 8 + nf, 0, 0);
        }
        break;
      case 6:
        for (auto& d : KING_D) {
          int nf = f + d[0], nr = r + d[1];
          if (!on_board(nf, nr)) continue;
          uint8_t q = sq[nr * 8 + nf];
          if (!q || (w ? is_black(q) : is_white(q))) push_move(out, s, nr * 8 + nf, 0, 0);
        }
        break;
      default: {
        if (kind == 4 || kind == 5)
          for (auto& d : ROOK_D) {
            int nf = f + d[0], nr = r + d[1];
            while (on_board(nf, nr)) {
              uint8_t q = sq[nr * 8 + nf];
              if (!q) push_move(out, s, nr * 8 + nf, 0, 0);
              else { if (w ? is_black(q) : is_white(q)) push_move(out, s, nr * 8 + nf, 0, 0); break; }
              nf += d[0]; nr += d[1];
            }
          }
        if (kind == 3 || kind == 5)
          for (auto& d : BISHOP_D) {
            int nf = f + d[0], nr = r + d[1];
            while (on_board(nf, nr)) {
              uint8_t q = sq[nr * 8 + nf];
              if (!q) push_move(out, s, nr * 8 + nf, 0, 0);
              else { if (w ? is_black(q) : is_white(q)) push_move(out, s, nr * 8 + nf, 0, 0); break; }
              nf += d[0]; nr += d[1];
            }
          }
      }
    }
  }
  // Castling: rights must survive the king/rook home-square filter, the squares
  // between must be empty, and the king may not start on, cross or land on an
  // attacked square.
  const uint8_t cr = clean_castling();
  if (w) {
    if ((cr & CR_WK) && !sq[5] && !sq[6] && !attacked(4, false) && !attacked(5, false) && !attacked(6, false))
      push_move(out, 4, 6, 0, 3);
    if ((cr & CR_WQ) && !sq[3] && !sq[2] && !sq[1] && !attacked(4, false) && !attacked(3, false) && !attacked(2, false))
      push_move(out, 4, 2, 0, 3);
  } else {
    if ((cr & CR_BK) && !sq[61] && !sq[62] && !attacked(60, true) && !attacked(61, true) && !attacked(62, true))
      push_move(out, 60, 62, 0, 3);
    if ((cr & CR_BQ) && !sq[59] && !sq[58] && !sq[57] && !attacked(60, true) && !attacked(59, true) && !attacked(58, true))
      push_move(out, 60, 58, 0, 3);
  }
}

void Board::make(const Move& m) {
  const uint8_t p = sq[m.from];
  const uint8_t captured = sq[m.to];
  const bool w = white_to_move;
  const bool pawn = (p == WP || p == BP);
  sq[m.from] = EMPTY;
  if (m.flag == 2) sq[(w ? m.to - 8 : m.to + 8)] = EMPTY;
  if (m.promo) {
    static const uint8_t WPROMO[5] = {0, WN, WB, WR, WQ};
    static const uint8_t BPROMO[5] = {0, BN, BB, BR, BQ};
    sq[m.to] = w ? WPROMO[m.promo] : BPROMO[m.promo];
  } else {
    sq[m.to] = p;
  }
  if (m.flag == 3) {
    if (m.to == 6) { sq[7] = EMPTY; sq[5] = WR; }
    else if (m.to == 2) { sq[0] = EMPTY; sq[3] = WR; }
    else if (m.to == 62) { sq[63] = EMPTY; sq[61] = BR; }
    else if (m.to == 58) { sq[56] = EMPTY; sq[59] = BR; }
  }
  // Rights disappear when the king or a corner rook moves or a corner is captured on.
  auto touch = [&](int s) {
    if (s == 4) castling &= ~(CR_WK | CR_WQ);
    else if (s == 60) castling &= ~(CR_BK | CR_BQ);
    else if (s == 7) castling &= ~CR_WK;
    else if (s == 0) castling &= ~CR_WQ;
    else if (s == 63) castling &= ~CR_BK;
    else if (s == 56) castling &= ~CR_BQ;
  };
  touch(m.from);
  touch(m.to);
  ep = (m.flag == 1) ? (int8_t)(w ? m.from + 8 : m.from - 8) : (int8_t)-1;
  halfmove = (pawn || captured || m.flag == 2) ? 0 : halfmove + 1;
  if (!w) ++fullmove;
  white_to_move = !w;
}

void Board::legal(std::vector<Move>& out) const {
  std::vector<Move> pl;
  pl.reserve(64);
  pseudo_legal(pl);
  const uint8_t kg = white_to_move ? WK : BK;
  for (const Move& m : pl) {
    Board c = *this;
    c.make(m);
    int ks = -1;
    for (int s = 0; s < 64; ++s) if (c.sq[s] == kg) { ks = s; break; }
    if (ks < 0 || !c.attacked(ks, !white_to_move)) out.push_back(m);
  }
}

int Board::piece_count() const {
  int n = 0;
  for (int s = 0; s < 64; ++s) n += sq[s] != 0;
  return n;
}

uint64_t Board::perft(int depth) const {
  if (depth == 0) return 1;
  std::vector<Move> mv;
  mv.reserve(64);
  legal(mv);
  if (depth == 1) return mv.size();
  uint64_t n = 0;
  for (const Move& m : mv) {
    Board c = *this;
    c.make(m);
    n += c.perft(depth - 1);
  }
  return n;
}

std::string Board::fen(bool ep_legal_only) const {
  std::string s;
  for (int r = 7; r >= 0; --r) {
    int run = 0;
    for (int f = 0; f < 8; ++f) {
      uint8_t p = sq[r * 8 + f];
      if (!p) { ++run; continue; }
      if (run) { s.push_back((char)('0' + run)); run = 0; }
      s.push_back(PIECE_CHARS[p]);
    }
    if (run) s.push_back((char)('0' + run));
    if (r) s.push_back('/');
  }
  s += white_to_move ? " w " : " b ";
  const uint8_t cr = clean_castling();
  if (!cr) s += "-";
  else {
    if (cr & CR_WK) s += "K";
    if (cr & CR_WQ) s += "Q";
    if (cr & CR_BK) s += "k";
    if (cr & CR_BQ) s += "q";
  }
  s += " ";
  bool write_ep = ep >= 0;
  if (write_ep && ep_legal_only) {
    write_ep = false;
    std::vector<Move> mv;
    legal(mv);
    for (const Move& m : mv) if (m.flag == 2) { write_ep = true; break; }
  }
  if (write_ep) { s.push_back((char)('a' + file_of(ep))); s.push_back((char)('1' + rank_of(ep))); }
  else s += "-";
  s += " " + std::to_string(halfmove) + " " + std::to_string(fullmove);
  return s;
}

void Board::planes(float* out) const {
  std::memset(out, 0, sizeof(float) * 64 * NUM_PLANES);
  const uint8_t cr = clean_castling();
  float hm = halfmove / 100.0f;
  if (hm > 1.0f) hm = 1.0f;
  for (int t = 0; t < 64; ++t) {
    const int r = 7 - (t >> 3), f = t & 7;
    float* o = out + t * NUM_PLANES;
    const uint8_t p = sq[r * 8 + f];
    if (p) o[p - 1] = 1.0f;
    o[12] = white_to_move ? 1.0f : 0.0f;
    o[14] = (cr & CR_WK) ? 1.0f : 0.0f;
    o[15] = (cr & CR_WQ) ? 1.0f : 0.0f;
    o[16] = (cr & CR_BK) ? 1.0f : 0.0f;
    o[17] = (cr & CR_BQ) ? 1.0f : 0.0f;
    o[18] = hm;
  }
  if (ep >= 0) out[((7 - rank_of(ep)) * 8 + file_of(ep)) * NUM_PLANES + 13] = 1.0f;
}

void Board::compact(uint8_t* ids64, uint8_t* flags4) const {
  for (int t = 0; t < 64; ++t) ids64[t] = sq[(7 - (t >> 3)) * 8 + (t & 7)];
  flags4[0] = white_to_move;
  flags4[1] = clean_castling();
  flags4[2] = ep >= 0 ? (uint8_t)((7 - rank_of(ep)) * 8 + file_of(ep)) : (uint8_t)255;
  flags4[3] = (uint8_t)(halfmove > 100 ? 100 : halfmove);
}

static std::string sq_name(int s) {
  std::string n;
  n.push_back((char)('a' + file_of(s)));
  n.push_back((char)('1' + rank_of(s)));
  return n;
}

std::string move_uci(const Move& m) {
  std::string s = sq_name(m.from) + sq_name(m.to);
  static const char PR[] = " nbrq";
  if (m.promo) s.push_back(PR[m.promo]);
  return s;
}

// ---------------------------------------------------------------- vocabulary
namespace {
struct Vocab {
  std::vector<std::string> rl, leela;
  int16_t idx[64][64][5];  // [from][to][promo] -> policy_index slot
  int32_t to_rl_white[VOCAB_LEELA], to_rl_black[VOCAB_LEELA];
  Vocab() {
    // The 1792 four-character moves: for every origin square in a1..h8 order, every
    // destination in a1..h8 order that a queen or a knight could reach.
    for (int from = 0; from < 64; ++from)
      for (int to = 0; to < 64; ++to) {
        if (to == from) continue;
        const int df = std::abs(file_of(to) - file_of(from)), dr = std::abs(rank_of(to) - rank_of(from));
        const bool queen = df == 0 || dr == 0 || df == dr;
        const bool knight = (df == 1 && dr == 2) || (df == 2 && dr == 1);
        if (queen || knight) leela.push_back(sq_name(from) + sq_name(to));
      }
    // 66 white under/queen promotions, origin file a..h, destination file left/same/right, q r b.
    auto promos = [](std::vector<std::string>& v, char from_rank, char to_rank) {
      for (int f = 0; f < 8; ++f)
        for (int t = f - 1; t <= f + 1; ++t) {
          if (t < 0 || t > 7) continue;
          for (char p : {'q', 'r', 'b'}) {
            std::string s;
            s.push_back((char)('a' + f)); s.push_back(from_rank);
            s.push_back((char)('a' + t)); s.push_back(to_rank);
            s.push_back(p);
            v.push_back(s);
          }
        }
    };
    promos(leela, '7', '8');
    rl = leela;
    promos(rl, '2', '1');
    for (const char* t : {"<thinking>", "</thinking>", "end_variation", "end", "padding_token"}) rl.push_back(t);

    std::memset(idx, 0xff, sizeof(idx));
    for (int i = 0; i < (int)rl.size() - 5; ++i) {
      const std::string& s = rl[i];
      const int from = (s[1] - '1') * 8 + (s[0] - 'a'), to = (s[3] - '1') * 8 + (s[2] - 'a');
      int pr = 0;
      if (s.size() == 5) pr = s[4] == 'q' ? 4 : s[4] == 'r' ? 3 : 2;
      idx[from][to][pr] = (int16_t)i;
      if (pr == 0) idx[from][to][1] = (int16_t)i;  // knight promotion shares the plain move's slot
    }
    for (int i = 0; i < VOCAB_LEELA; ++i) {
      const std::string& s = leela[i];
      const int from = (s[1] - '1') * 8 + (s[0] - 'a'), to = (s[3] - '1') * 8 + (s[2] - 'a');
      int pr = 0;
      if (s.size() == 5) pr = s[4] == 'q' ? 4 : s[4] == 'r' ? 3 : 2;
      to_rl_white[i] = i;
      to_rl_black[i] = idx[from ^ 56][to ^ 56][pr];
    }
  }
};
const Vocab& vocab() {
  static Vocab v;
  return v;
}
}  // namespace

const std::vector<std::string>& policy_index() { return vocab().rl; }
const std::vector<std::string>& policy_leela() { return vocab().leela; }
int rl_index(int from, int to, int promo) { return vocab().idx[from][to][promo]; }
int leela_index(int from, int to, int promo, bool white_to_move) {
  if (!white_to_move) { from ^= 56; to ^= 56; }
  int i = vocab().idx[from][to][promo];
  return i < VOCAB_LEELA ? i : -1;
}
const int32_t* leela_to_rl_white() { return vocab().to_rl_white; }
const int32_t* leela_to_rl_black() { return vocab().to_rl_black; }

int legal_mask_rl(const Board& b, uint8_t* mask) {
  std::memset(mask, 0, VOCAB_RL);
  std::vector<Move> mv;
  mv.reserve(64);
  b.legal(mv);
  for (const Move& m : mv) {
    int i = rl_index(m.from, m.to, m.promo);
    if (i >= 0) mask[i] = 1;
  }
  return (int)mv.size();
}

int legal_mask_leela(const Board& b, uint8_t* mask) {
  std::memset(mask, 0, VOCAB_LEELA);
  std::vector<Move> mv;
  mv.reserve(64);
  b.legal(mv);
  for (const Move& m : mv) {
    int i = leela_index(m.from, m.to, m.promo, b.white_to_move);
    if (i >= 0) mask[i] = 1;
  }
  return (int)mv.size();
}

Board random_playout(SplitMix64& rng, int max_plies, int max_pieces) {
  std::vector<Move> mv;
  for (;;) {
    Board b;
    b.set_start();
    const int target = max_pieces > 0 ? 100000 : (int)(rng.next() % (uint64_t)(max_plies + 1));
    bool ok = true;
    int ply = 0;
    for (;;) {
      mv.clear();
      b.legal(mv);
      if (mv.empty()) { ok = false; break; }
      if (max_pieces > 0) {
        if (b.piece_count() <= max_pieces) break;
        if (ply >= 2000) { ok = false; break; }
      } else if (ply >= target) {
        break;
      }
      b.make(mv[rng.next() % mv.size()]);
      ++ply;
    }
    if (ok) return b;
  }
}

}  // namespace crl

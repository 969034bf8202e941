// Host-side chess substrate for the policy/value forward path: FEN parsing, the
// 19-plane board encoding, legal move generation, the 1929/1858-entry move
// vocabularies and seeded random-playout position generation.
//
// Square numbering is a1=0, b1=1 ... h8=63 (rank*8+file). The token order the
// models consume is t=(7-rank)*8+file (a8 first, h1 last), which is the layout of
// the reference's fen_to_tensor (utils/fen_encoder.py:5-38).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace crl {

enum Piece : uint8_t {
  EMPTY = 0,
  WP = 1, WN, WB, WR, WQ, WK,
  BP = 7, BN, BB, BR, BQ, BK
};

constexpr int VOCAB_RL = 1929;     // utils/vocab.py:9-227
constexpr int VOCAB_LEELA = 1858;  // utils/vocab.py:229-438
constexpr int NUM_PLANES = 19;

// Castling-right bits.
constexpr uint8_t CR_WK = 1, CR_WQ = 2, CR_BK = 4, CR_BQ = 8;

struct Move {
  uint8_t from, to;
  uint8_t promo;  // 0 none, 1 knight, 2 bishop, 3 rook, 4 queen
  uint8_t flag;   // 0 normal, 1 double push, 2 en passant, 3 castle
};

struct Board {
  uint8_t sq[64];
  uint8_t white_to_move;
  uint8_t castling;   // rights exactly as the FEN field states them
  int8_t ep;          // en-passant target square as the FEN field states it, or -1
  int32_t halfmove;
  int32_t fullmove;

  void set_start();
  // Returns 0 on success, negative on a malformed FEN (message in *err if given).
  int set_fen(const char* fen, std::string* err = nullptr);
  // ep_legal_only: write the en-passant square only when an en-passant capture is
  // legal (what python-chess board.fen() does for the child positions built in
  // new_paradigm/value.py:337-339).
  std::string fen(bool ep_legal_only = true) const;

  // Rights filtered the way python-chess cleans them: the right counts only if the
  // king stands on e1/e8 and the rook on its corner.
  uint8_t clean_castling() const;

  bool attacked(int square, bool by_white) const;
  bool in_check() const;
  void pseudo_legal(std::vector<Move>& out) const;
  void legal(std::vector<Move>& out) const;
  void make(const Move& m);
  int piece_count() const;
  uint64_t perft(int depth) const;

  // float32[64*19] in token order (utils/fen_encoder.py:5-38).
  void planes(float* out) const;
  // Compact form: 64 piece codes (0..12) in token order + 4 flag bytes
  // {white_to_move, clean castling bits, ep token or 255, min(halfmove,100)}.
  void compact(uint8_t* ids64, uint8_t* flags4) const;
};

std::string move_uci(const Move& m);

// Vocabulary. policy_index (1929) = policy_leela (1858) + 66 black promotions +
// 5 special tokens. Built from the generation rule, never read from a file.
const std::vector<std::string>& policy_index();
const std::vector<std::string>& policy_leela();
// (from,to,promo) -> index in policy_index, or -1. A knight promotion maps to the
// plain four-character move (model_bis.py:376-377).
int rl_index(int from, int to, int promo);
// Index in the 1858-entry list for a move seen from the side to move: ranks are
// mirrored for black (Leela/compare_policy.py:437-463). -1 if absent.
int leela_index(int from, int to, int promo, bool white_to_move);
// For each Leela index i: its policy_index slot for a white row (identity) and a
// black row (rank-mirrored move), Leela/compare_policy.py:470-491.
const int32_t* leela_to_rl_white();
const int32_t* leela_to_rl_black();

// uint8 mask[1929] / mask[1858] of the legal moves; returns the number of legal moves.
int legal_mask_rl(const Board& b, uint8_t* mask);
int legal_mask_leela(const Board& b, uint8_t* mask);

struct SplitMix64 {
  uint64_t s;
  explicit SplitMix64(uint64_t seed) : s(seed) {}
  uint64_t next() {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
};

// Uniform-random legal playout from the start position. plies ~ U{0..max_plies};
// if max_pieces > 0 the playout instead continues until at most max_pieces pieces
// remain. A playout that runs into a finished game is restarted. The result always
// has at least one legal move.
Board random_playout(SplitMix64& rng, int max_plies, int max_pieces);

}  // namespace crl

"""Pure-Python chess rules used to check the C++ host code. TEST INFRASTRUCTURE ONLY.

Restates, without python-chess (not installable here), what the reference gets from it:
  fen_to_planes      utils/fen_encoder.py:5-38 (board.piece_map, board.turn, board.ep_square,
                     has_*_castling_rights, halfmove_clock)
  legal_moves_uci    list(board.legal_moves) -> move.uci()   (model_bis.py:375-379)
  legal_mask         the mask loop of model_bis.py:373-380 (trailing 'n' stripped)

Semantics taken from python-chess as documented: ep_square is the FEN field as written;
castling rights count only with the king on e1/e8 and the rook on its corner; castling is
written king-from king-to (e1g1).

Pins: perft known answers (tests/test_host.py: start position, Kiwipete, positions 3-5 of
the chessprogramming perft suite) and hand-written expectations for the planes. The
implementation is deliberately different from the C++ one (0x88 board, ray tables) so a
shared mistake is unlikely.
"""

KNIGHT = (0x21, 0x1F, 0x12, 0x0E, -0x21, -0x1F, -0x12, -0x0E)
KING = (0x01, 0x11, 0x10, 0x0F, -0x01, -0x11, -0x10, -0x0F)
ROOK = (0x01, -0x01, 0x10, -0x10)
BISHOP = (0x11, 0x0F, -0x11, -0x0F)
PLANE = {c: i for i, c in enumerate("PNBRQKpnbrqk")}


def sq88(file, rank):
    return rank * 16 + file


def name88(s):
    return "abcdefgh"[s & 7] + str((s >> 4) + 1)


class Position:
    def __init__(self, fen):
        parts = fen.split()
        self.board = {}
        rank, file = 7, 0
        for ch in parts[0]:
            if ch == "/":
                rank, file = rank - 1, 0
            elif ch.isdigit():
                file += int(ch)
            else:
                self.board[sq88(file, rank)] = ch
                file += 1
        self.white = (parts[1] == "w") if len(parts) > 1 else True
        self.castling = parts[2] if len(parts) > 2 and parts[2] != "-" else ""
        ep = parts[3] if len(parts) > 3 else "-"
        self.ep = None if ep == "-" else sq88(ord(ep[0]) - 97, int(ep[1]) - 1)
        self.halfmove = int(parts[4]) if len(parts) > 4 else 0

    def copy(self):
        p = Position.__new__(Position)
        p.board = dict(self.board)
        p.white, p.castling, p.ep, p.halfmove = self.white, self.castling, self.ep, self.halfmove
        return p

    def clean_castling(self):
        ok = ""
        b = self.board
        if b.get(sq88(4, 0)) == "K":
            if "K" in self.castling and b.get(sq88(7, 0)) == "R":
                ok += "K"
            if "Q" in self.castling and b.get(sq88(0, 0)) == "R":
                ok += "Q"
        if b.get(sq88(4, 7)) == "k":
            if "k" in self.castling and b.get(sq88(7, 7)) == "r":
                ok += "k"
            if "q" in self.castling and b.get(sq88(0, 7)) == "r":
                ok += "q"
        return ok

    def attacked(self, s, by_white):
        b = self.board
        pawn, knight, king = ("P", "N", "K") if by_white else ("p", "n", "k")
        rook, bishop, queen = ("R", "B", "Q") if by_white else ("r", "b", "q")
        for d in ((-0x0F, -0x11) if by_white else (0x0F, 0x11)):
            if b.get(s + d) == pawn and not (s + d) & 0x88:
                return True
        for d in KNIGHT:
            if not (s + d) & 0x88 and b.get(s + d) == knight:
                return True
        for d in KING:
            if not (s + d) & 0x88 and b.get(s + d) == king:
                return True
        for dirs, slider in ((ROOK, rook), (BISHOP, bishop)):
            for d in dirs:
                t = s + d
                while not t & 0x88:
                    p = b.get(t)
                    if p:
                        if p == slider or p == queen:
                            return True
                        break
                    t += d
        return False

    def pseudo(self):
        b, w = self.board, self.white
        mine = str.isupper if w else str.islower
        out = []
        for s, p in list(b.items()):
            if not mine(p):
                continue
            k = p.upper()
            if k == "P":
                d = 0x10 if w else -0x10
                start, last = (1, 7) if w else (6, 0)
                t = s + d
                if not t & 0x88 and t not in b:
                    if (t >> 4) == last:
                        out += [(s, t, pr) for pr in "qrbn"]
                    else:
                        out.append((s, t, ""))
                        if (s >> 4) == start and (t + d) not in b:
                            out.append((s, t + d, ""))
                for dc in (d - 1, d + 1):
                    t = s + dc
                    if t & 0x88:
                        continue
                    q = b.get(t)
                    if q and not mine(q):
                        if (t >> 4) == last:
                            out += [(s, t, pr) for pr in "qrbn"]
                        else:
                            out.append((s, t, ""))
                    elif q is None and t == self.ep and (s >> 4) == (4 if w else 3) and b.get(t - d) == ("p" if w else "P"):
                        out.append((s, t, "ep"))
            elif k in "NK":
                for d in (KNIGHT if k == "N" else KING):
                    t = s + d
                    if t & 0x88:
                        continue
                    q = b.get(t)
                    if q is None or not mine(q):
                        out.append((s, t, ""))
            else:
                dirs = ROOK if k == "R" else BISHOP if k == "B" else ROOK + BISHOP
                for d in dirs:
                    t = s + d
                    while not t & 0x88:
                        q = b.get(t)
                        if q is None:
                            out.append((s, t, ""))
                        else:
                            if not mine(q):
                                out.append((s, t, ""))
                            break
                        t += d
        rights = self.clean_castling()
        r = 0 if w else 7
        e = sq88(4, r)
        if ("K" if w else "k") in rights and all(sq88(f, r) not in b for f in (5, 6)) \
                and not any(self.attacked(sq88(f, r), not w) for f in (4, 5, 6)):
            out.append((e, sq88(6, r), "castle"))
        if ("Q" if w else "q") in rights and all(sq88(f, r) not in b for f in (1, 2, 3)) \
                and not any(self.attacked(sq88(f, r), not w) for f in (4, 3, 2)):
            out.append((e, sq88(2, r), "castle"))
        return out

    def make(self, mv):
        s, t, kind = mv
        b, w = self.board, self.white
        p = b.pop(s)
        captured = b.get(t)
        if kind == "ep":
            del b[t - (0x10 if w else -0x10)]
        if kind in ("q", "r", "b", "n"):
            p = kind.upper() if w else kind
        b[t] = p
        if kind == "castle":
            r = t >> 4
            if (t & 7) == 6:
                b[sq88(5, r)] = b.pop(sq88(7, r))
            else:
                b[sq88(3, r)] = b.pop(sq88(0, r))
        lost = {sq88(4, 0): "KQ", sq88(7, 0): "K", sq88(0, 0): "Q", sq88(4, 7): "kq", sq88(7, 7): "k", sq88(0, 7): "q"}
        for x in (s, t):
            for c in lost.get(x, ""):
                self.castling = self.castling.replace(c, "")
        self.ep = (s + t) // 2 if p.upper() == "P" and abs(t - s) == 0x20 else None
        self.halfmove = 0 if (p.upper() == "P" or captured or kind == "ep") else self.halfmove + 1
        self.white = not w

    def legal(self):
        out = []
        king = "K" if self.white else "k"
        for mv in self.pseudo():
            c = self.copy()
            c.make(mv)
            ks = next(s for s, p in c.board.items() if p == king)
            if not c.attacked(ks, c.white):
                out.append(mv)
        return out

    def perft(self, depth):
        if depth == 0:
            return 1
        moves = self.legal()
        if depth == 1:
            return len(moves)
        n = 0
        for mv in moves:
            c = self.copy()
            c.make(mv)
            n += c.perft(depth - 1)
        return n


def uci(mv):
    s, t, kind = mv
    return name88(s) + name88(t) + (kind if kind in ("q", "r", "b", "n") else "")


def legal_moves_uci(fen):
    return [uci(m) for m in Position(fen).legal()]


def legal_mask(fen, vocab):
    """0/1 list over `vocab` (the 1929-entry list) with the reference's knight-promotion strip."""
    index = {m: i for i, m in enumerate(vocab)}
    mask = [0] * len(vocab)
    for m in legal_moves_uci(fen):
        if m.endswith("n"):
            m = m[:-1]
        mask[index[m]] = 1
    return mask


def mirror_uci(m):
    """Rank mirror of Leela/compare_policy.py:437-463."""
    return m[0] + str(9 - int(m[1])) + m[2] + str(9 - int(m[3])) + m[4:]


def legal_mask_leela(fen, vocab_leela):
    """Mask over the 1858-entry side-to-move frame: black moves are rank-mirrored."""
    index = {m: i for i, m in enumerate(vocab_leela)}
    pos = Position(fen)
    mask = [0] * len(vocab_leela)
    for m in legal_moves_uci(fen):
        if m.endswith("n"):
            m = m[:-1]
        if not pos.white:
            m = mirror_uci(m)
        mask[index[m]] = 1
    return mask


def fen_to_planes(fen):
    """8x8x19 nested lists indexed [7-rank][file][plane] (utils/fen_encoder.py:5-38)."""
    pos = Position(fen)
    t = [[[0.0] * 19 for _ in range(8)] for _ in range(8)]
    for s, p in pos.board.items():
        t[7 - (s >> 4)][s & 7][PLANE[p]] = 1.0
    rights = pos.clean_castling()
    hm = min(pos.halfmove / 100.0, 1.0)
    for r in range(8):
        for f in range(8):
            c = t[r][f]
            c[12] = 1.0 if pos.white else 0.0
            c[14] = 1.0 if "K" in rights else 0.0
            c[15] = 1.0 if "Q" in rights else 0.0
            c[16] = 1.0 if "k" in rights else 0.0
            c[17] = 1.0 if "q" in rights else 0.0
            c[18] = hm
    if pos.ep is not None:
        t[7 - (pos.ep >> 4)][pos.ep & 7][13] = 1.0
    return t

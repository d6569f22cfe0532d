/* CPU rules engine for the 32-slot piece-list position format.
 *
 * Purpose: produce synthetic inputs for the network evaluator -- seeded uniformly
 * random legal playouts, the packed position words and the [32] x u64 legal-move
 * words that go with them.  It is not on the evaluator's hot path.
 *
 * Position format (reference docs/reference/spec.md:38-88):
 *   word  bit 11 captured, bit 10 colour (1 = black), bit 9 special, bits 8:6 type
 *         (0 P, 1 N, 2 B, 3 R, 4 Q, 5 K), bits 5:0 square (row * 8 + col, 0 = a1)
 *   slots 0-7 white pawns, 8-9 N, 10-11 B, 12-13 R, 14 Q, 15 K, 16-31 the same for black
 *   special = "has moved" on K/R, "just double-pushed" on a pawn
 *   control = sign: side to move (+ white), magnitude: halfmove clock + 1
 *   mask    bit s of word p set iff slot p may legally move to square s
 *           (reference docs/reference/spec.md:141-143)
 *
 * Rule behaviour follows the reference environment brokefish/env/torch_impl.py:
 * pawn and en-passant generation :77-126, castling :161-181, full legality by
 * replaying every pseudo-legal move :251-289, move application :412-540 (the castled
 * rook does NOT get its special bit set; the clock restarts at 1 on a capture or a
 * pawn move), FEN import :781-837.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define CAPTURED 0x800u
#define COLOR 0x400u
#define SPECIAL 0x200u
#define SQMASK 0x3Fu

enum { PAWN, KNIGHT, BISHOP, ROOK, QUEEN, KING };

typedef struct {
    uint16_t w[32];
    int16_t control;
} Pos;

static inline int w_type(uint16_t w) { return (w >> 6) & 7; }
static inline int w_sq(uint16_t w) { return w & SQMASK; }
static inline int w_black(uint16_t w) { return (w >> 10) & 1; }
static inline int w_alive(uint16_t w) { return !(w & CAPTURED); }

static const int KN_D[8][2] = {{1, 2}, {2, 1}, {2, -1}, {1, -2}, {-1, -2}, {-2, -1}, {-2, 1}, {-1, 2}};
static const int KG_D[8][2] = {{1, 0}, {1, 1}, {0, 1}, {-1, 1}, {-1, 0}, {-1, -1}, {0, -1}, {1, -1}};
static const int RAY_D[8][2] = {{1, 0}, {-1, 0}, {0, 1}, {0, -1}, {1, 1}, {1, -1}, {-1, 1}, {-1, -1}};

/* square -> slot (or -1) */
static void mailbox(const Pos* p, int8_t at[64]) {
    memset(at, -1, 64);
    for (int s = 0; s < 32; s++)
        if (w_alive(p->w[s])) at[w_sq(p->w[s])] = (int8_t)s;
}

/* Is `sq` attacked by a piece of colour `by_black`? */
static int attacked(const Pos* p, const int8_t at[64], int sq, int by_black) {
    const int r = sq >> 3, c = sq & 7;
    /* pawns: a white pawn on (r-1, c+-1) attacks (r, c) */
    const int pr = by_black ? r + 1 : r - 1;
    if (pr >= 0 && pr < 8) {
        for (int dc = -1; dc <= 1; dc += 2) {
            const int pc = c + dc;
            if (pc < 0 || pc > 7) continue;
            const int s = at[pr * 8 + pc];
            if (s >= 0 && w_type(p->w[s]) == PAWN && w_black(p->w[s]) == by_black) return 1;
        }
    }
    for (int i = 0; i < 8; i++) {
        int rr = r + KN_D[i][0], cc = c + KN_D[i][1];
        if (rr >= 0 && rr < 8 && cc >= 0 && cc < 8) {
            const int s = at[rr * 8 + cc];
            if (s >= 0 && w_type(p->w[s]) == KNIGHT && w_black(p->w[s]) == by_black) return 1;
        }
        rr = r + KG_D[i][0]; cc = c + KG_D[i][1];
        if (rr >= 0 && rr < 8 && cc >= 0 && cc < 8) {
            const int s = at[rr * 8 + cc];
            if (s >= 0 && w_type(p->w[s]) == KING && w_black(p->w[s]) == by_black) return 1;
        }
    }
    for (int d = 0; d < 8; d++) {
        int rr = r + RAY_D[d][0], cc = c + RAY_D[d][1];
        while (rr >= 0 && rr < 8 && cc >= 0 && cc < 8) {
            const int s = at[rr * 8 + cc];
            if (s >= 0) {
                if (w_black(p->w[s]) == by_black) {
                    const int t = w_type(p->w[s]);
                    if (t == QUEEN || (d < 4 && t == ROOK) || (d >= 4 && t == BISHOP)) return 1;
                }
                break;
            }
            rr += RAY_D[d][0]; cc += RAY_D[d][1];
        }
    }
    return 0;
}

/* Pseudo-legal destinations of every slot of the side to move (king safety not applied). */
static void pseudo_moves(const Pos* p, const int8_t at[64], uint64_t out[32]) {
    const int black = p->control < 0;
    for (int s = 0; s < 32; s++) {
        out[s] = 0;
        const uint16_t w = p->w[s];
        if (!w_alive(w) || w_black(w) != black) continue;
        const int sq = w_sq(w), r = sq >> 3, c = sq & 7, t = w_type(w);
        uint64_t m = 0;
        if (t == PAWN) {
            const int dir = black ? -1 : 1;
            const int r1 = r + dir;
            if (r1 >= 0 && r1 < 8) {
                if (at[r1 * 8 + c] < 0) {
                    m |= 1ull << (r1 * 8 + c);
                    const int start = black ? 6 : 1;
                    const int r2 = r + 2 * dir;
                    if (r == start && at[r2 * 8 + c] < 0) m |= 1ull << (r2 * 8 + c);
                }
                for (int dc = -1; dc <= 1; dc += 2) {
                    const int cc = c + dc;
                    if (cc < 0 || cc > 7) continue;
                    const int o = at[r1 * 8 + cc];
                    if (o >= 0 && w_black(p->w[o]) != black) m |= 1ull << (r1 * 8 + cc);
                    /* en passant: an enemy pawn flagged `special` stands beside us on
                     * our fifth rank */
                    if (r == (black ? 3 : 4)) {
                        const int v = at[r * 8 + cc];
                        if (v >= 0 && w_type(p->w[v]) == PAWN && w_black(p->w[v]) != black &&
                            (p->w[v] & SPECIAL))
                            m |= 1ull << (r1 * 8 + cc);
                    }
                }
            }
        } else if (t == KNIGHT || t == KING) {
            const int (*D)[2] = (t == KNIGHT) ? KN_D : KG_D;
            for (int i = 0; i < 8; i++) {
                const int rr = r + D[i][0], cc = c + D[i][1];
                if (rr < 0 || rr > 7 || cc < 0 || cc > 7) continue;
                const int o = at[rr * 8 + cc];
                if (o < 0 || w_black(p->w[o]) != black) m |= 1ull << (rr * 8 + cc);
            }
            if (t == KING && !(w & SPECIAL)) {
                const int row = black ? 56 : 0;
                const uint16_t rook = (uint16_t)((black ? COLOR : 0) | (ROOK << 6));
                int short_ok = 0, long_ok = 0;
                for (int q = 0; q < 32; q++) {
                    if (p->w[q] == (uint16_t)(rook | (row + 7))) short_ok = 1;
                    if (p->w[q] == (uint16_t)(rook | row)) long_ok = 1;
                }
                if (short_ok && at[row + 5] < 0 && at[row + 6] < 0) m |= 1ull << (row + 6);
                if (long_ok && at[row + 1] < 0 && at[row + 2] < 0 && at[row + 3] < 0)
                    m |= 1ull << (row + 2);
            }
        } else {
            const int d0 = (t == BISHOP) ? 4 : 0, d1 = (t == ROOK) ? 4 : 8;
            for (int d = d0; d < d1; d++) {
                int rr = r + RAY_D[d][0], cc = c + RAY_D[d][1];
                while (rr >= 0 && rr < 8 && cc >= 0 && cc < 8) {
                    const int o = at[rr * 8 + cc];
                    if (o >= 0) {
                        if (w_black(p->w[o]) != black) m |= 1ull << (rr * 8 + cc);
                        break;
                    }
                    m |= 1ull << (rr * 8 + cc);
                    rr += RAY_D[d][0]; cc += RAY_D[d][1];
                }
            }
        }
        out[s] = m;
    }
}

/* Apply `move = slot * 64 + target` (promo 0:N 1:B 2:R 3:Q, used on promotions only). */
static void apply_move(Pos* p, int move, int promo) {
    const int src = move >> 6, target = move & 63;
    const uint16_t v = p->w[src];
    const int t = w_type(v), white = p->control > 0, from = w_sq(v);
    int capture = 0;
    for (int s = 0; s < 32; s++) {
        const uint16_t w = p->w[s];
        if (s != src && w_alive(w) && w_sq(w) == target) { p->w[s] = CAPTURED; capture = 1; }
    }
    if (t == PAWN && !capture) {
        /* en passant victim: an enemy pawn flagged special directly behind the target */
        const uint16_t victim = white ? (uint16_t)(COLOR | SPECIAL | (target - 8))
                                      : (uint16_t)(SPECIAL | (target + 8));
        for (int s = 0; s < 32; s++)
            if (p->w[s] == victim) { p->w[s] = CAPTURED; capture = 1; }
    }
    uint16_t nw = (uint16_t)((v & ~SQMASK) | target);
    if (t == PAWN && (target >> 3) == (white ? 7 : 0)) nw = (uint16_t)(nw + ((promo + KNIGHT) << 6));
    p->w[src] = nw;
    const int dx = target - from;
    if (t == KING && (dx == 2 || dx == -2)) {
        const int row = white ? 0 : 56, rfrom = row + (dx > 0 ? 7 : 0), rto = row + (dx > 0 ? 5 : 3);
        for (int s = 0; s < 32; s++) {
            const uint16_t w = p->w[s];
            if (w_alive(w) && w_type(w) == ROOK && w_sq(w) == rfrom) {
                p->w[s] = (uint16_t)((w & ~SQMASK) | rto);
                break;
            }
        }
    }
    if (t == KING || t == ROOK) p->w[src] |= SPECIAL;
    for (int s = 0; s < 32; s++)
        if (w_type(p->w[s]) == PAWN) p->w[s] &= (uint16_t)~SPECIAL;
    if (t == PAWN && (dx == 16 || dx == -16)) p->w[src] |= SPECIAL;
    const int mag = (capture || t == PAWN) ? 1 : abs(p->control) + 1;
    p->control = (int16_t)(white ? -mag : mag);
}

/* Fully legal mask; returns the number of set bits. */
static int legal_moves(const Pos* p, uint64_t mask[32], int* in_check) {
    int8_t at[64];
    mailbox(p, at);
    const int black = p->control < 0;
    const int ksq = w_sq(p->w[black ? 31 : 15]);
    if (in_check) *in_check = attacked(p, at, ksq, !black);
    uint64_t ps[32];
    pseudo_moves(p, at, ps);
    int count = 0;
    for (int s = 0; s < 32; s++) {
        uint64_t m = ps[s], keep = 0;
        while (m) {
            const int tsq = __builtin_ctzll(m);
            m &= m - 1;
            Pos q = *p;
            apply_move(&q, s * 64 + tsq, 3);
            int8_t at2[64];
            mailbox(&q, at2);
            int ok;
            const int from = w_sq(p->w[s]);
            if (w_type(p->w[s]) == KING && abs(tsq - from) == 2) {
                /* start, crossed and landing squares must all be safe */
                const int lo = tsq < from ? tsq : from;
                ok = !attacked(&q, at2, lo, !black) && !attacked(&q, at2, lo + 1, !black) &&
                     !attacked(&q, at2, lo + 2, !black);
            } else {
                ok = !attacked(&q, at2, w_sq(q.w[black ? 31 : 15]), !black);
            }
            if (ok) { keep |= 1ull << tsq; count++; }
        }
        mask[s] = keep;
    }
    return count;
}

/* ------------------------------------------------------------------------ */
/* exported API                                                              */
/* ------------------------------------------------------------------------ */

static const uint16_t START[32] = {
    8, 9, 10, 11, 12, 13, 14, 15,
    (KNIGHT << 6) | 1, (KNIGHT << 6) | 6, (BISHOP << 6) | 2, (BISHOP << 6) | 5,
    (ROOK << 6) | 0, (ROOK << 6) | 7, (QUEEN << 6) | 3, (KING << 6) | 4,
    COLOR | 48, COLOR | 49, COLOR | 50, COLOR | 51, COLOR | 52, COLOR | 53, COLOR | 54, COLOR | 55,
    COLOR | (KNIGHT << 6) | 57, COLOR | (KNIGHT << 6) | 62, COLOR | (BISHOP << 6) | 58,
    COLOR | (BISHOP << 6) | 61, COLOR | (ROOK << 6) | 56, COLOR | (ROOK << 6) | 63,
    COLOR | (QUEEN << 6) | 59, COLOR | (KING << 6) | 60};

void bf_chess_initial(uint16_t* board, int16_t* control) {
    memcpy(board, START, sizeof(START));
    *control = 1;
}

void bf_chess_movegen(const uint16_t* boards, const int16_t* control, int n, uint64_t* mask,
                      uint8_t* in_check) {
    for (int i = 0; i < n; i++) {
        Pos p;
        memcpy(p.w, boards + (size_t)i * 32, 64);
        p.control = control[i];
        int chk;
        legal_moves(&p, mask + (size_t)i * 32, &chk);
        if (in_check) in_check[i] = (uint8_t)chk;
    }
}

/* In place. move -1 leaves the row untouched. */
void bf_chess_step(uint16_t* boards, int16_t* control, const int16_t* move, const uint8_t* promo,
                   int n) {
    for (int i = 0; i < n; i++) {
        if (move[i] < 0) continue;
        Pos p;
        memcpy(p.w, boards + (size_t)i * 32, 64);
        p.control = control[i];
        apply_move(&p, move[i], promo ? promo[i] & 3 : 3);
        memcpy(boards + (size_t)i * 32, p.w, 64);
        control[i] = p.control;
    }
}

/* FEN -> position. Returns 0 on success. */
int bf_chess_from_fen(const char* fen, uint16_t* board, int16_t* control) {
    char placement[128], turn[8], castle[8], ep[8];
    int half = 0, full = 1;
    int got = 0;
    {
        /* split on spaces without sscanf width surprises */
        const char* f = fen;
        char* dst[4] = {placement, turn, castle, ep};
        const size_t cap[4] = {sizeof(placement), sizeof(turn), sizeof(castle), sizeof(ep)};
        for (int k = 0; k < 4; k++) {
            size_t n = 0;
            while (*f == ' ') f++;
            while (*f && *f != ' ') { if (n + 1 < cap[k]) dst[k][n++] = *f; f++; }
            dst[k][n] = 0;
            if (n) got++;
        }
        while (*f == ' ') f++;
        if (*f) { half = atoi(f); while (*f && *f != ' ') f++; while (*f == ' ') f++; if (*f) full = atoi(f); }
        (void)full;
    }
    if (got < 4) return -1;
    const int black_to_move = turn[0] == 'b';
    int ep_victim = -1;
    if (ep[0] != '-') {
        const int sq = (ep[1] - '1') * 8 + (ep[0] - 'a');
        ep_victim = sq + (black_to_move ? 8 : -8);
    }
    for (int s = 0; s < 32; s++) board[s] = (uint16_t)(START[s] | CAPTURED);
    /* next free index per letter, slot offset, capacity */
    const char* letters = "PNBRQKpnbrqk";
    const int off[12] = {0, 8, 10, 12, 14, 15, 16, 24, 26, 28, 30, 31};
    const int cap[12] = {8, 2, 2, 2, 1, 1, 8, 2, 2, 2, 1, 1};
    int next[12] = {0};
    int row = 7, col = 0;
    for (const char* c = placement; *c; c++) {
        if (*c >= '1' && *c <= '8') { col += *c - '0'; continue; }
        if (*c == '/') { row--; col = 0; continue; }
        const char* f = strchr(letters, *c);
        if (!f) return -2;
        int li = (int)(f - letters);
        const int white = li < 6, kind = li % 6;
        int slot;
        uint16_t w;
        if (next[li] >= cap[li]) { /* promoted material goes into a pawn slot */
            const int pl = white ? 0 : 6;
            if (next[pl] >= cap[pl]) return -3;
            slot = off[pl] + next[pl]++;
            w = (uint16_t)((white ? 0 : COLOR) | (kind << 6));
        } else {
            slot = off[li] + next[li]++;
            w = (uint16_t)((white ? 0 : COLOR) | (kind << 6));
        }
        const int sq = row * 8 + col;
        w |= (uint16_t)sq;
        if (kind == PAWN && sq == ep_victim) w |= SPECIAL;
        if (kind == ROOK) {
            const int rank = sq >> 3, file = sq & 7;
            const int on_corner = rank == (white ? 0 : 7) && (file == 0 || file == 7);
            char letter = file == 7 ? 'k' : 'q';
            if (white) letter = (char)(letter - 32);
            if (!(on_corner && strchr(castle, letter))) w |= SPECIAL;
        }
        if (kind == KING) {
            const int any = white ? (strchr(castle, 'K') || strchr(castle, 'Q'))
                                  : (strchr(castle, 'k') || strchr(castle, 'q'));
            if (!any) w |= SPECIAL;
        }
        board[slot] = w;
        col++;
    }
    *control = (int16_t)((black_to_move ? -1 : 1) * (half + 1));
    return 0;
}

static uint64_t perft_rec(const Pos* p, int depth) {
    uint64_t mask[32];
    legal_moves(p, mask, NULL);
    uint64_t total = 0;
    const int white = p->control > 0;
    for (int s = 0; s < 32; s++) {
        uint64_t m = mask[s];
        while (m) {
            const int tsq = __builtin_ctzll(m);
            m &= m - 1;
            const int is_promo = w_type(p->w[s]) == PAWN && (tsq >> 3) == (white ? 7 : 0);
            if (depth == 1) { total += is_promo ? 4 : 1; continue; }
            for (int pr = is_promo ? 0 : 3; pr < 4; pr++) {
                Pos q = *p;
                apply_move(&q, s * 64 + tsq, pr);
                total += perft_rec(&q, depth - 1);
            }
        }
    }
    return total;
}

/* Number of leaf edges at `depth` (a promotion counts as four moves). */
uint64_t bf_chess_perft(const uint16_t* board, int16_t control, int depth) {
    if (depth <= 0) return 1;
    Pos p;
    memcpy(p.w, board, 64);
    p.control = control;
    return perft_rec(&p, depth);
}

static inline uint64_t splitmix64(uint64_t* s) {
    uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* Game i (counted from `first_game`) plays plies_i ~ U{0..max_plies} uniformly random
 * legal moves from the initial position (promotion piece uniform); a game with no legal
 * move stops where it is.  rep_i = i mod 3.  Each game has its own generator derived
 * from (seed, i), so the result does not depend on how the batch is split.
 * Outputs: boards [n,32], control [n], rep [n], mask [n,32] (may be NULL). */
void bf_chess_random_playouts(int n, int max_plies, uint64_t seed, uint64_t first_game,
                              uint16_t* boards, int16_t* control, uint8_t* rep, uint64_t* mask) {
#pragma omp parallel for schedule(dynamic, 16)
    for (int i = 0; i < n; i++) {
        const uint64_t game = first_game + (uint64_t)i;
        uint64_t st = seed * 0xD1342543DE82EF95ull + game * 0x9E3779B97F4A7C15ull + 0x2545F4914F6CDD1Dull;
        Pos p;
        memcpy(p.w, START, sizeof(START));
        p.control = 1;
        const int plies = (int)(splitmix64(&st) % (uint64_t)(max_plies + 1));
        uint64_t m[32];
        int count = legal_moves(&p, m, NULL);
        for (int ply = 0; ply < plies && count > 0; ply++) {
            int pick = (int)(splitmix64(&st) % (uint64_t)count);
            const int promo = (int)(splitmix64(&st) & 3);
            int mv = -1;
            for (int s = 0; s < 32 && mv < 0; s++) {
                const int c = __builtin_popcountll(m[s]);
                if (pick >= c) { pick -= c; continue; }
                uint64_t w = m[s];
                while (pick--) w &= w - 1;
                mv = s * 64 + __builtin_ctzll(w);
            }
            apply_move(&p, mv, promo);
            count = legal_moves(&p, m, NULL);
        }
        memcpy(boards + (size_t)i * 32, p.w, 64);
        control[i] = p.control;
        rep[i] = (uint8_t)(game % 3);
        if (mask) memcpy(mask + (size_t)i * 32, m, sizeof(m));
    }
}

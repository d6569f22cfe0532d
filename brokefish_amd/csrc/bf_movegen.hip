// Legal-move words on the device: packed positions -> [n, 32] x u64 masks (+ in-check flags), so
// the mask the evaluator ANDs in and the expansion walks never leaves the GPU.
// Replaces env.movegen of the reference (docs/reference/spec.md:152-172; rule behaviour
// brokefish/env/torch_impl.py:77-126 pawns / en passant, :161-181 castling, :251-289 legality by
// replaying every pseudo-legal move); the CPU generator of this repository (chessgen.c, pinned by
// the published perft counts) is its checker.
//
// One wavefront per position.  The position's bitboards (occupancy by colour, the enemy's pieces
// by kind) are built once per wave on the scalar unit from the 32 words.  Lane l < 32 generates
// slot l's pseudo-legal targets -- a slider's reach along a line is two subtractions, the other
// pieces are shift patterns: no loop over squares -- and each target is tested by "replaying" the
// move on the bitboards (occupancy, captured piece, en-passant victim, castled rook) and asking
// whether the enemy attacks the king's square -- for castling the start, crossed and landing
// squares, evaluated on the position after the move, as the checker does.  For that step the
// position's moves are dealt out evenly over the 64 lanes.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#include "bf_args.h"

namespace {

typedef unsigned long long u64;

constexpr unsigned CAPTURED = 0x800u, COLOR = 0x400u, SPECIAL = 0x200u;
enum { PAWN, KNIGHT, BISHOP, ROOK, QUEEN, KING };

struct Enemy {          // the side NOT to move, after the move under test
    u64 pawns, knights, diag, orth, king;
    bool black;
};

__device__ __forceinline__ u64 bit(int sq) { return 1ull << sq; }

constexpr u64 FILE_A = 0x0101010101010101ull, FILE_H = 0x8080808080808080ull;
constexpr u64 NOT_A = ~FILE_A, NOT_H = ~FILE_H, NOT_AB = ~(FILE_A | FILE_A << 1), NOT_GH = ~(FILE_H | FILE_H >> 1);

// The squares a slider on s (one bit) reaches along the line `m` (a rank, file or diagonal through
// s, s excluded) on occupancy occ, blockers included: o - s borrows upwards through the empty
// squares to the first blocker, so o ^ (o - s) is the ray towards the higher bits; the same on the
// bit-reversed board is the ray towards the lower ones.  No loop, no branch.
__device__ __forceinline__ u64 line_attacks(u64 occ, u64 m, u64 s) {
    const u64 o = occ & m;
    const u64 up = o - s;
    const u64 down = __brevll(__brevll(o) - __brevll(s));
    return (up ^ down) & m;
}
// the four lines through square sq (the square itself excluded)
struct Lines { u64 rank, file, diag, anti; };
__device__ __forceinline__ Lines lines_through(int sq) {
    const int r = sq >> 3, c = sq & 7;
    const u64 s = bit(sq);
    Lines l;
    l.rank = (0xFFull << (8 * r)) ^ s;
    l.file = (FILE_A << c) ^ s;
    const int d = r - c;            // a1-h8 direction: 0x8040201008040201 shifted by whole ranks
    l.diag = (d >= 0 ? 0x8040201008040201ull << (8 * d) : 0x8040201008040201ull >> (8 * -d)) ^ s;
    const int e = r + c - 7;        // a8-h1 direction
    l.anti = (e >= 0 ? 0x0102040810204080ull << (8 * e) : 0x0102040810204080ull >> (8 * -e)) ^ s;
    return l;
}
__device__ __forceinline__ u64 rook_attacks(u64 occ, int sq) {
    const Lines l = lines_through(sq);
    return line_attacks(occ, l.rank, bit(sq)) | line_attacks(occ, l.file, bit(sq));
}
__device__ __forceinline__ u64 bishop_attacks(u64 occ, int sq) {
    const Lines l = lines_through(sq);
    return line_attacks(occ, l.diag, bit(sq)) | line_attacks(occ, l.anti, bit(sq));
}
__device__ __forceinline__ u64 knight_pattern(u64 s) {
    return ((s << 17) & NOT_A) | ((s << 10) & NOT_AB) | ((s >> 6) & NOT_AB) | ((s >> 15) & NOT_A) |
           ((s << 15) & NOT_H) | ((s << 6) & NOT_GH) | ((s >> 10) & NOT_GH) | ((s >> 17) & NOT_H);
}
__device__ __forceinline__ u64 king_pattern(u64 s) {
    const u64 row = s | ((s << 1) & NOT_A) | ((s >> 1) & NOT_H);
    return (row | row << 8 | row >> 8) ^ s;
}

// Does `e` attack square sq, given occupancy occ?  Looked at from the square: a rook placed there
// sees the enemy's orthogonal sliders exactly when they see it, and so for the other kinds.
__device__ __forceinline__ bool attacked(const Enemy& e, u64 occ, int sq) {
    const u64 s = bit(sq);
    // a white pawn on (r-1, c+-1) attacks (r, c); a black one from (r+1, c+-1)
    const u64 pawn_from = e.black ? (((s << 7) & NOT_H) | ((s << 9) & NOT_A)) : (((s >> 7) & NOT_A) | ((s >> 9) & NOT_H));
    const u64 hit = (pawn_from & e.pawns) | (knight_pattern(s) & e.knights) | (king_pattern(s) & e.king) |
                    (rook_attacks(occ, sq) & e.orth) | (bishop_attacks(occ, sq) & e.diag);
    return hit != 0;
}

__global__ __launch_bounds__(256) void movegen_kernel(const uint16_t* boards, const int16_t* control, int n,
                                                      u64* mask, uint8_t* in_check) {
    const int lane = threadIdx.x & 63;
    // the position and the side to move are the same for the whole wave: said so, the bitboard
    // construction below runs on the scalar unit
    const int b = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
    if (b >= n) return;                                 // no workgroup barrier below
    const int slot = lane & 31, part = lane >> 5;
    const unsigned w = boards[(size_t)b * 32 + slot];
    const bool black = __builtin_amdgcn_readfirstlane((int)control[b]) < 0;

    // bitboards, computed by every lane from the words of all 32 slots
    u64 own = 0, opp = 0, ep_pawns = 0;
    Enemy e = {0, 0, 0, 0, 0, !black};
    bool rook_short = false, rook_long = false;         // an unmoved own rook on its corner
    const unsigned row = black ? 56u : 0u;
    const unsigned rookw = (black ? COLOR : 0u) | (ROOK << 6);
#pragma unroll
    for (int s = 0; s < 32; s++) {
        const unsigned v = (unsigned)__builtin_amdgcn_readlane((int)w, s);   // wave-uniform: the loop runs on the scalar unit
        rook_short |= v == (rookw | (row + 7));
        rook_long |= v == (rookw | row);
        if (v & CAPTURED) continue;
        const u64 sb = bit(v & 63);
        const int t = (v >> 6) & 7;
        if (((v >> 10) & 1) == (unsigned)black) {
            own |= sb;
        } else {
            opp |= sb;
            if (t == PAWN) { e.pawns |= sb; if (v & SPECIAL) ep_pawns |= sb; }
            else if (t == KNIGHT) e.knights |= sb;
            else if (t == KING) e.king |= sb;
            if (t == BISHOP || t == QUEEN) e.diag |= sb;
            if (t == ROOK || t == QUEEN) e.orth |= sb;
        }
    }
    const u64 occ = own | opp;
    const int ksq = (black ? __builtin_amdgcn_readlane((int)w, 31) : __builtin_amdgcn_readlane((int)w, 15)) & 63;
    if (lane == 0 && in_check) in_check[b] = attacked(e, occ, ksq) ? 1 : 0;

    // pseudo-legal targets of this slot
    u64 ps = 0;
    const bool mine = !(w & CAPTURED) && (((w >> 10) & 1) == (unsigned)black);
    const int sq = w & 63, r = sq >> 3, c = sq & 7, t = (w >> 6) & 7;
    if (mine) {
        if (t == PAWN) {
            const int dir = black ? -1 : 1, r1 = r + dir;
            if (r1 >= 0 && r1 < 8) {
                if (!(occ & bit(r1 * 8 + c))) {
                    ps |= bit(r1 * 8 + c);
                    const int r2 = r + 2 * dir;
                    if (r == (black ? 6 : 1) && !(occ & bit(r2 * 8 + c))) ps |= bit(r2 * 8 + c);
                }
#pragma unroll
                for (int dc = -1; dc <= 1; dc += 2) {
                    const int cc = c + dc;
                    if (cc < 0 || cc > 7) continue;
                    if (opp & bit(r1 * 8 + cc)) ps |= bit(r1 * 8 + cc);
                    // en passant: an enemy pawn that just double-pushed stands beside us on our fifth rank
                    if (r == (black ? 3 : 4) && (ep_pawns & bit(r * 8 + cc))) ps |= bit(r1 * 8 + cc);
                }
            }
        } else if (t == KNIGHT) {
            ps = knight_pattern(bit(sq)) & ~own;
        } else if (t == KING) {
            ps = king_pattern(bit(sq)) & ~own;
            if (!(w & SPECIAL)) {
                if (rook_short && !(occ & (bit(row + 5) | bit(row + 6)))) ps |= bit(row + 6);
                if (rook_long && !(occ & (bit(row + 1) | bit(row + 2) | bit(row + 3)))) ps |= bit(row + 2);
            }
        } else if (t == BISHOP || t == ROOK || t == QUEEN) {
            if (t != BISHOP) ps |= rook_attacks(occ, sq);
            if (t != ROOK) ps |= bishop_attacks(occ, sq);
            ps &= ~own;
        }
    }

    // legality: the position's pseudo-legal moves are dealt out evenly over the 64 lanes (move k of
    // the slot-major list goes to lane k % 64); each is replayed on the bitboards
    __shared__ u64 legal[4][32];
    u64* const mine_out = legal[threadIdx.x >> 6];
    if (lane < 32) mine_out[lane] = 0;
    const int cnt = part == 0 ? __popcll(ps) : 0;
    int first = cnt;                                                // exclusive prefix over slots
#pragma unroll
    for (int d = 1; d < 32; d <<= 1) {
        const int o = __shfl_up(first, d);
        if (lane >= d) first += o;
    }
    first -= cnt;
    const int total = __shfl(first + cnt, 31);
    for (int base = 0; base < total; base += 64) {
        const int k = base + lane;
        int s = 0;                                                  // the slot whose range holds move k
#pragma unroll
        for (int j = 1; j < 32; j++) s = (__shfl(first, j) <= k) ? j : s;
        const unsigned ws = (unsigned)__shfl((int)w, s);
        u64 todo = ((u64)(unsigned)__shfl((int)(unsigned)(ps >> 32), s) << 32) | (unsigned)__shfl((int)(unsigned)ps, s);
        const int skip = k - __shfl(first, s);                      // every lane takes part in the exchanges above
        if (k >= total) continue;
        for (int j = skip; j > 0; j--) todo &= todo - 1;
        const int tsq = __builtin_ctzll(todo);
        const int from = ws & 63, ts = (ws >> 6) & 7;
        const u64 tb = bit(tsq), fb = bit(from);
        u64 occ2 = (occ & ~fb) | tb;
        Enemy e2 = e;
        u64 gone = tb;                                              // a piece standing on the target is captured
        if (ts == PAWN && !(opp & tb) && (tsq & 7) != (from & 7)) { // en passant: the victim is behind the target
            const u64 vb = bit(black ? tsq + 8 : tsq - 8);
            gone |= vb;
            occ2 &= ~vb;
        }
        e2.pawns &= ~gone; e2.knights &= ~gone; e2.diag &= ~gone; e2.orth &= ~gone;
        bool ok;
        if (ts == KING && (tsq - from == 2 || tsq - from == -2)) {
            // the rook jumps too; start, crossed and landing squares must all be safe afterwards
            const int rfrom = (int)row + (tsq > from ? 7 : 0), rto = (int)row + (tsq > from ? 5 : 3);
            occ2 = (occ2 & ~bit(rfrom)) | bit(rto);
            const int lo = tsq < from ? tsq : from;
            ok = !attacked(e2, occ2, lo) && !attacked(e2, occ2, lo + 1) && !attacked(e2, occ2, lo + 2);
        } else {
            ok = !attacked(e2, occ2, ts == KING ? tsq : ksq);
        }
        if (ok) atomicOr(&mine_out[s], tb);
    }
    // same wave, LDS operations complete in order: the words are final
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (lane < 32) mask[(size_t)b * 32 + lane] = mine_out[lane];
}

}  // namespace

extern "C" int bf_movegen(const uint16_t* boards, const int16_t* control, int64_t n, uint64_t* mask,
                          uint8_t* in_check, void* stream) {
    auto fail = [](int code, const char* msg) {
        bf::set_error(msg);
        return code;
    };
    if (n < 1 || n > (1ll << 28)) return fail(BF_ERR_ARGUMENT, "n must be in [1, 2^28]");
    if (!boards || !control || !mask) return fail(BF_ERR_ARGUMENT, "boards/control/mask must not be NULL");
    if (((uintptr_t)boards & 1) || ((uintptr_t)control & 1) || ((uintptr_t)mask & 7))
        return fail(BF_ERR_ARGUMENT, "boards and control must be 2-byte and mask 8-byte aligned");
    hipLaunchKernelGGL(movegen_kernel, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, (hipStream_t)stream, boards, control,
                       (int)n, reinterpret_cast<u64*>(mask), in_check);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[256];
        snprintf(msg, sizeof(msg), "kernel launch failed: %s", hipGetErrorString(e));
        return fail(BF_ERR_LAUNCH, msg);
    }
    return BF_OK;
}

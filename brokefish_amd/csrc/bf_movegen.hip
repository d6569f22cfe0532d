// Legal-move words on the device: packed positions -> [n, 32] x u64 masks (+ in-check flags), so
// the mask the evaluator ANDs in and the expansion walks never leaves the GPU.
// Replaces env.movegen of the reference (docs/reference/spec.md:152-172; rule behaviour
// brokefish/env/torch_impl.py:77-126 pawns / en passant, :161-181 castling, :251-289 legality by
// replaying every pseudo-legal move); the CPU generator of this repository (chessgen.c, pinned by
// the published perft counts) is its checker.
//
// One wavefront per position.  Every lane first builds the position's bitboards (occupancy by
// colour, the enemy's pieces by kind) from the 32 words, broadcast lane to lane.  Lane l < 32
// generates slot l's pseudo-legal targets with bitboard walks, and each target is tested by
// "replaying" the move on the bitboards (occupancy, captured piece,
// en-passant victim, castled rook) and asking whether the enemy attacks the king's square -- for
// castling the start, crossed and landing squares, evaluated on the position after the move, as
// the checker does.  For that step the position's moves are dealt out evenly over the 64 lanes.
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

// Does `e` attack square sq, given occupancy occ?
__device__ bool attacked(const Enemy& e, u64 occ, int sq) {
    const int r = sq >> 3, c = sq & 7;
    // a white pawn on (r-1, c+-1) attacks (r, c); a black one from (r+1, c+-1)
    const int pr = e.black ? r + 1 : r - 1;
    if (pr >= 0 && pr < 8) {
        if (c > 0 && (e.pawns & bit(pr * 8 + c - 1))) return true;
        if (c < 7 && (e.pawns & bit(pr * 8 + c + 1))) return true;
    }
    const int kn[8][2] = {{1, 2}, {2, 1}, {2, -1}, {1, -2}, {-1, -2}, {-2, -1}, {-2, 1}, {-1, 2}};
    const int kg[8][2] = {{1, 0}, {1, 1}, {0, 1}, {-1, 1}, {-1, 0}, {-1, -1}, {0, -1}, {1, -1}};
#pragma unroll
    for (int i = 0; i < 8; i++) {
        int rr = r + kn[i][0], cc = c + kn[i][1];
        if (rr >= 0 && rr < 8 && cc >= 0 && cc < 8 && (e.knights & bit(rr * 8 + cc))) return true;
        rr = r + kg[i][0]; cc = c + kg[i][1];
        if (rr >= 0 && rr < 8 && cc >= 0 && cc < 8 && (e.king & bit(rr * 8 + cc))) return true;
    }
    const int ray[8][2] = {{1, 0}, {-1, 0}, {0, 1}, {0, -1}, {1, 1}, {1, -1}, {-1, 1}, {-1, -1}};
#pragma unroll
    for (int d = 0; d < 8; d++) {
        int rr = r + ray[d][0], cc = c + ray[d][1];
        while (rr >= 0 && rr < 8 && cc >= 0 && cc < 8) {
            const u64 b = bit(rr * 8 + cc);
            if (occ & b) {
                if ((d < 4 ? e.orth : e.diag) & b) return true;
                break;
            }
            rr += ray[d][0]; cc += ray[d][1];
        }
    }
    return false;
}

__global__ __launch_bounds__(256) void movegen_kernel(const uint16_t* boards, const int16_t* control, int n,
                                                      u64* mask, uint8_t* in_check) {
    const int lane = threadIdx.x & 63;
    const int b = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= n) return;                                 // no workgroup barrier below
    const int slot = lane & 31, part = lane >> 5;
    const unsigned w = boards[(size_t)b * 32 + slot];
    const bool black = control[b] < 0;

    // bitboards, computed by every lane from the words of all 32 slots
    u64 own = 0, opp = 0, ep_pawns = 0;
    Enemy e = {0, 0, 0, 0, 0, !black};
    bool rook_short = false, rook_long = false;         // an unmoved own rook on its corner
    const unsigned row = black ? 56u : 0u;
    const unsigned rookw = (black ? COLOR : 0u) | (ROOK << 6);
#pragma unroll
    for (int s = 0; s < 32; s++) {
        const unsigned v = (unsigned)__shfl((int)w, s);
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
    const int ksq = __shfl((int)w, black ? 31 : 15) & 63;
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
        } else if (t == KNIGHT || t == KING) {
            const int kn[8][2] = {{1, 2}, {2, 1}, {2, -1}, {1, -2}, {-1, -2}, {-2, -1}, {-2, 1}, {-1, 2}};
            const int kg[8][2] = {{1, 0}, {1, 1}, {0, 1}, {-1, 1}, {-1, 0}, {-1, -1}, {0, -1}, {1, -1}};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int rr = r + (t == KNIGHT ? kn[i][0] : kg[i][0]), cc = c + (t == KNIGHT ? kn[i][1] : kg[i][1]);
                if (rr < 0 || rr > 7 || cc < 0 || cc > 7) continue;
                if (!(own & bit(rr * 8 + cc))) ps |= bit(rr * 8 + cc);
            }
            if (t == KING && !(w & SPECIAL)) {
                if (rook_short && !(occ & (bit(row + 5) | bit(row + 6)))) ps |= bit(row + 6);
                if (rook_long && !(occ & (bit(row + 1) | bit(row + 2) | bit(row + 3)))) ps |= bit(row + 2);
            }
        } else if (t == BISHOP || t == ROOK || t == QUEEN) {
            const int ray[8][2] = {{1, 0}, {-1, 0}, {0, 1}, {0, -1}, {1, 1}, {1, -1}, {-1, 1}, {-1, -1}};
            const int d0 = (t == BISHOP) ? 4 : 0, d1 = (t == ROOK) ? 4 : 8;
            for (int d = d0; d < d1; d++) {
                int rr = r + ray[d][0], cc = c + ray[d][1];
                while (rr >= 0 && rr < 8 && cc >= 0 && cc < 8) {
                    const u64 sb = bit(rr * 8 + cc);
                    if (occ & sb) {
                        if (opp & sb) ps |= sb;
                        break;
                    }
                    ps |= sb;
                    rr += ray[d][0]; cc += ray[d][1];
                }
            }
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

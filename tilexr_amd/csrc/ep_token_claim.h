// Consumer side of the tile readiness flags: what a combine launch that may have to wait does about tokens whose tiles
// are not published yet.  Shared by the reduce kernels (ep_reduce_common.hip.h supplies the operations as device code:
// atomics, barriers, LDS) and by a host-side model that runs the same control flow one memory operation at a time
// under seeded schedules (flag_trace.cpp), as ep_tile_publish.h is shared on the producer side.
//
// A token needs the tiles of all its rows, and a producer that works tile by tile finishes those at unrelated times,
// so tokens become ready in no particular order.  A waiting launch therefore never sits on one group of tokens:
//   * groups are claimed, a few at a time, from a counter all workgroups share; a workgroup holds at most kClaimHeld
//     groups that are not ready yet, and whoever has nothing left to wait for takes the next ones (with fixed ownership
//     the tokens of a producer's last tiles were reduced by the few workgroups that happened to own them, one after
//     the other, while the rest had gone home);
//   * fresh groups are looked at once (kRouteCheck) and reduced at once if their tiles are there;
//   * for what is left the workgroup goes in rounds: one scan looks at every tile the held groups need, the groups that
//     have become complete are reduced without looking again (kRouteTrusted: the scan has just seen them), and a round
//     without any is followed by a sleep that grows;
//   * when nothing held has become ready for the wait bound, or another workgroup has reported an expired wait, the
//     rest is given up (kRouteGiveUp): a token with a tile that is still missing gets a row of zeros -- never the sum
//     of the rows that happened to be there -- and the launch's status word is set.
//
// `Env` supplies:
//   int  Claim(int want)                first of `want` consecutive groups nobody else has been given (any value when
//                                       groups are dealt by NextGroup alone)
//   int  NextGroup(int *next)           the next group for this workgroup: (*next)++ with a shared counter
//   void Hold(int slot, int group)      remember the group in one of the kClaimHeld slots
//   void HoldDone()                     all Hold calls of a refill are made
//   bool Try(int slot, int mode)        look at the slot's group as `mode` says and reduce it; false = "come back
//                                       later" (only in kRouteCheck), the same answer for the whole workgroup
//   uint32_t Scan(uint32_t pending)     one look at every tile the pending slots' groups need: mask of slots with a
//                                       tile that is not published
//   bool GiveUpNow()                    the wait bound has passed since Touch(), or a wait of the launch has expired
//   void Touch()                        progress was made: the wait bound starts again
//   void Sleep(int level)               level 0, 1, 2: longer each time
//   void Leave()                        this workgroup has claimed for the last time.  The claim counter is left at
//                                       zero for the next launch by whoever leaves last (a second word counts the
//                                       leavers), the way the publishers' landing counters are: no launch has to
//                                       clear anything first
#ifndef TILEXR_AMD_EP_TOKEN_CLAIM_H
#define TILEXR_AMD_EP_TOKEN_CLAIM_H

#include <cstdint>

#include "ep_tile_publish.h"

namespace TileXREp {

// what a route table holds for a slot whose wait expired / whose tile is not there yet (rows are >= 0, no row is -1)
constexpr int kRowExpired = -2;
constexpr int kRowPending = -3;
enum RouteMode : int { kRouteCheck = 0, kRouteTrusted = 1, kRouteGiveUp = 2 };
constexpr int kClaimHeld = 4;

// Whether a slot with a row looks at its tile's word when the route table is filled.  `block`: the launch waits
// (bounded) on every slot in turn instead of coming back later (the element-granular kernel).
TILEXR_EP_HD bool SlotLooksAtTile(bool block, int mode)
{
    return block || mode != kRouteTrusted;
}

// What the slot becomes after the look: its row stays, "come back later", or expired (status word set, row of zeros).
enum SlotVerdict : int { kSlotTake = 0, kSlotComeBack = 1, kSlotExpire = 2 };
TILEXR_EP_HD int JudgeSlot(bool block, int mode, bool published)
{
    if (published) {
        return kSlotTake;
    }
    return (!block && mode == kRouteCheck) ? kSlotComeBack : kSlotExpire;
}

template <typename Env>
TILEXR_EP_HD void ClaimAndReduce(Env &env, int groups)
{
    bool more = true;
    uint32_t pending = 0u;                          // slots that hold a claimed, unfinished group
    int backoff = 0;
    env.Touch();
    for (;;) {
        uint32_t fresh = 0u;
        const uint32_t freeSlots = ~pending & ((1u << kClaimHeld) - 1u);
        if (more && freeSlots != 0u) {
            int next = env.Claim(__builtin_popcount(freeSlots));
            for (uint32_t m = freeSlots; m != 0u; m &= m - 1u) {
                const int slot = __builtin_ctz(m);
                const int group = env.NextGroup(&next);
                if (group >= groups || group < 0) {
                    more = false;
                    continue;
                }
                env.Hold(slot, group);
                fresh |= 1u << slot;
            }
            pending |= fresh;
            env.HoldDone();
        }
        if (pending == 0u) {
            break;                                  // nothing held, nothing left to claim
        }
        // One loop body does the work of all stages: `todo` holds the slots to try now, `mode` says how (a first look at
        // fresh groups; after a scan: trusted; giving up).
        uint32_t todo = fresh;
        int mode = kRouteCheck;
        for (int pass = 0; pass < 2; ++pass) {
            bool done = false;
            for (; todo != 0u; todo &= todo - 1u) {
                const int slot = __builtin_ctz(todo);
                if (!env.Try(slot, mode)) {
                    continue;
                }
                pending &= ~(1u << slot);
                env.Touch();
                backoff = 0;
                done = true;
            }
            if (pass == 1 || pending == 0u || (done && more)) {
                break;                              // free slots and groups to claim: refill before looking again
            }
            todo = pending & ~env.Scan(pending);
            mode = kRouteTrusted;
            if (todo != 0u) {
                continue;
            }
            if (env.GiveUpNow()) {
                todo = pending;                     // what is held is given up: rows of zeros, status word set
                mode = kRouteGiveUp;
                continue;
            }
            env.Sleep(backoff);
            backoff += backoff < 2 ? 1 : 0;
            break;
        }
    }
    env.Leave();
}

// The leaver's part, for an Env whose two words live in memory the operations `ops` reach (FetchAdd(p) -> value
// before, Store(p, v)): the last of `workgroups` leavers puts both words back to zero.  Every claim of a workgroup has
// returned before it leaves, so nothing can claim behind the reset.  Returns whether this call did the reset.
template <typename Ops>
TILEXR_EP_HD bool LeaveClaimWords(Ops &ops, uint32_t *claimWords, uint32_t workgroups)
{
    const uint32_t before = ops.FetchAdd(&claimWords[1]);
    if (before + 1u != workgroups) {
        return false;
    }
    ops.Store(&claimWords[1], 0u);
    ops.Store(&claimWords[0], 0u);
    return true;
}

} // namespace TileXREp

#endif // TILEXR_AMD_EP_TOKEN_CLAIM_H

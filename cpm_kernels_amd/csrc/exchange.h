// Exchange of per-column partial statistics between the workgroups of a team.
//
// A column reduction whose rows do not fit one workgroup's registers is split over the P
// workgroups of a team (P workgroups that one XCD starts one after the other, see xch_member).  Each
// posts its partials as 8-byte packets {value, launch tag} with device-scope atomic stores and
// collects its team mates' packets by polling until the tag matches; a packet is valid as a
// whole or not at all, so no fence and no separate flag is needed, and the packets of an older
// launch can never be mistaken for this one's.
//
// The team member that finishes collecting last wipes the team's packets, so a launch that is
// replayed with the same arguments (a captured graph) starts from a clean slate as well.
//
// The packets live in a fixed pool in device memory owned by the library (nothing is allocated
// per call).  Its first kXchRingSlots slots of kXchVals packets are handed out as a ring.  A launch
// takes as many slots as it has (team, part) pairs (at most kXchSlots), so the ring holds the
// slots of many launches at once (128 tall layernorms of 8 x 4096 x 512); before a launch reuses
// slots that an earlier launch was given, its stream waits for that launch's completion event,
// so launches on any number of streams never share live packets.  The pool's lock is held from
// the moment a launch is given its slots until its completion event is recorded (XchScope), so
// no other host thread ever sees slots whose holder cannot be waited for.
// A launch recorded during stream capture cannot be tracked by events (a graph is replayed any
// number of times, at any time): it gets slots from a reserve of kXchCaptureSlots further slots
// that the ring never hands out.  A range of the reserve belongs to one (capture, stream) pair
// for good: the launches recorded on one stream during one capture form a chain of graph nodes
// that run one after the other, so they share a range, and no launch outside that chain, eager
// or captured, is ever given it.  When the reserve is used up XchScope::begin says so (kXchFull)
// and the caller records its kernel that needs no packets instead.
//
// Progress: a workgroup only ever waits for workgroups of its own team, which are the next ones that its own
// XCD starts for this launch (xch_member; that an XCD starts a launch's workgroups in index order is an observed
// property of the hardware queue, not a documented one).  With several launches sharing the chip at most
// (team size - 1) workgroups per launch and XCD can be waiting for a member that has not started, so the
// oldest unfinished team of every XCD gets its members as soon as compute units are free there.  Should a
// packet nevertheless not arrive within about a second the wait gives up, the caller writes NaN (0 in an int8
// output) and sets the device's sticky status word and its mirror in pinned host memory.  Every launcher of
// the library looks at the mirror before it returns (launch_status() in common.h), so the failure is
// reported by the next call, whichever it is, like an asynchronous error of the runtime itself;
// cpmk_async_status() reports and clears it: a visible failure instead of a hung GPU.
#pragma once
#include "common.h"

namespace cpmk {

constexpr int kXchRingSlots = 32768;     // slots handed out as a ring to eager launches (1 KB each)
constexpr int kXchCaptureSlots = 32768;  // slots beyond the ring, given once and for all to launches recorded during stream capture
constexpr int kXchPoolSlots = kXchRingSlots + kXchCaptureSlots;
constexpr int kXchSlots = 8192;       // (team, part) pairs per launch
constexpr int kXchVals = 128;         // packets per slot: 64 columns x 2 statistics
constexpr int kXchMaxParts = 8;
constexpr int kXchGranule = 64;       // slots are handed out in multiples of this

constexpr uint32_t kXchStatusTimeout = 1u;   // bit of the status word: a packet did not arrive in time

constexpr int kXchFull = -2;          // XchScope::begin: the capture reserve is used up (not an error: record the kernel without packets)

// What a team kernel needs of the pool; passed to the kernel by value.
struct XchLaunch {
    uint64_t* region;     // this launch's slots: slot i at region + i * kXchVals
    uint64_t* counters;   // one retire counter per team: counters[team]
    uint32_t* status;     // the device's sticky status word
    uint32_t* host_status;  // its mirror in pinned host memory (nullptr if there is none)
    uint32_t tag;         // never 0, differs from the tags of the launches that used these slots before
    int32_t first;        // host bookkeeping: first pool slot of the launch, -1 if it holds none
};
constexpr XchLaunch kXchNone = {nullptr, nullptr, nullptr, nullptr, 0, -1};     // a launch without packets

// Host: the slots of one team launch.  begin() gives `slots` slots (and as many team counters) to a launch on
// stream `st` of the current device and makes `st` wait for the launches that last held them; end(), after the
// kernel launch, records the launch's completion on `st` so that a later holder of its slots can wait for it.
// The pool stays locked in between (and is unlocked by the destructor on every path), so the launch itself
// must follow begin() directly.  begin(): 0, kXchFull (recorded during stream capture and the capture reserve
// is used up; nothing is held), or an error code.  end(): 0 or an error code.
class XchScope {
public:
    XchScope() = default;
    XchScope(const XchScope&) = delete;
    XchScope& operator=(const XchScope&) = delete;
    ~XchScope();
    int begin(int64_t slots, hipStream_t st);
    int end();
    XchLaunch xl = kXchNone;
private:
    hipStream_t st_ = nullptr;
    int32_t last_ = 0;                 // end of the slot range [xl.first, last_)
    bool locked_ = false, captured_ = false;
};
// Host: a tag for a team launch that brings its own packet slots (never 0, from the same sequence as XchScope's).
uint32_t xch_next_tag();
// Host: the addresses of the current device's status word and of its host mirror (nullptr if none), for such a
// launch.  0 or an error code.
int xch_status_words(uint32_t** device_word, uint32_t** host_word);
// Host: sets the current device's pool up (symbol addresses, the status word's host mirror) ahead of the first team launch, so
// that a process whose first team launch is recorded during stream capture has the mirror too.  Failures are left to that launch.
void xch_prepare();
// Host: slots left in the current device's capture reserve.  0 or an error code.
int xch_capture_slots_left(int32_t* slots);
// Host: reads and clears the current device's status word and its mirror (0, kXchStatus* bits; an error code on failure to read).
int xch_take_status(uint32_t* bits);

// A wait gave up: leave a mark that the host can see (launch_status, cpmk_async_status).
__device__ inline void xch_flag(const XchLaunch& xl, uint32_t bit) {
    __hip_atomic_fetch_or(xl.status, bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (xl.host_status != nullptr) __hip_atomic_fetch_or(xl.host_status, bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ inline void xch_post(uint64_t* slot, int idx, float v, uint32_t tag) {
    const uint64_t pkt = ((uint64_t)tag << 32) | (uint64_t)__builtin_bit_cast(uint32_t, v);
    __hip_atomic_store(slot + idx, pkt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Poll one packet; false if it has not arrived by `deadline` (wall_clock64 ticks).
__device__ inline bool xch_wait(const uint64_t* p, uint32_t tag, uint64_t deadline, float& v) {
    for (;;) {
        const uint64_t pkt = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((uint32_t)(pkt >> 32) == tag) {
            v = __builtin_bit_cast(float, (uint32_t)pkt);
            return true;
        }
        if ((uint64_t)wall_clock64() > deadline) {
            v = 0.0f;
            return false;
        }
        __builtin_amdgcn_s_sleep(2);
    }
}

// Packet `idx` of up to W consecutive parts q0 .. q0+W-1 (< parts) of a team, polled together so
// that their round trips to the L2 overlap instead of following one another.  v[j] receives the value
// of part q0 + j (0 where there is no such part, or none arrived in time); false on a time-out.
template <int W>
__device__ inline bool xch_gather(const uint64_t* team_slots, int parts, int q0, int idx, uint32_t tag, uint64_t deadline,
                                  float (&v)[W]) {
    uint32_t missing = 0;
#pragma unroll
    for (int j = 0; j < W; ++j) {
        v[j] = 0.0f;
        if (q0 + j < parts) missing |= 1u << j;
    }
    for (;;) {
        uint64_t pk[W];
#pragma unroll
        for (int j = 0; j < W; ++j)
            if (missing >> j & 1u)
                pk[j] = __hip_atomic_load(team_slots + (size_t)(q0 + j) * kXchVals + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int j = 0; j < W; ++j)
            if ((missing >> j & 1u) && (uint32_t)(pk[j] >> 32) == tag) {
                v[j] = __builtin_bit_cast(float, (uint32_t)pk[j]);
                missing &= ~(1u << j);
            }
        if (missing == 0) return true;
        if ((uint64_t)wall_clock64() > deadline) return false;
        __builtin_amdgcn_s_sleep(2);
    }
}

// The same for two packets of every part, `ia` and `ib`, all polled together: one round trip to the L2 where
// two calls of xch_gather would make two, one after the other.
template <int W>
__device__ inline bool xch_gather2(const uint64_t* team_slots, int parts, int q0, int ia, int ib, uint32_t tag, uint64_t deadline,
                                   float (&va)[W], float (&vb)[W]) {
    uint32_t missing = 0;           // bit j: packet ia of part q0 + j, bit W + j: packet ib
#pragma unroll
    for (int j = 0; j < W; ++j) {
        va[j] = vb[j] = 0.0f;
        if (q0 + j < parts) missing |= (1u << j) | (1u << (W + j));
    }
    for (;;) {
        uint64_t pk[2 * W];
#pragma unroll
        for (int j = 0; j < 2 * W; ++j)
            if (missing >> j & 1u)
                pk[j] = __hip_atomic_load(team_slots + (size_t)(q0 + j % W) * kXchVals + (j < W ? ia : ib), __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int j = 0; j < 2 * W; ++j)
            if ((missing >> j & 1u) && (uint32_t)(pk[j] >> 32) == tag) {
                const float x = __builtin_bit_cast(float, (uint32_t)pk[j]);
                if (j < W) va[j] = x;
                else vb[j - W] = x;
                missing &= ~(1u << j);
            }
        if (missing == 0) return true;
        if ((uint64_t)wall_clock64() > deadline) return false;
        __builtin_amdgcn_s_sleep(2);
    }
}

// Which team a workgroup belongs to.  The hardware deals the workgroups of a launch out to the chip's 8 XCDs
// round robin (workgroup i runs on XCD (i + k) % 8, k the same for the whole launch), and every XCD starts its share on its own, in index order, as its
// compute units become free: nothing orders the XCDs among each other.  A team therefore consists of workgroups of
// ONE XCD that follow one another in that XCD's order -- workgroups 8s + x for `parts` consecutive s -- so a
// member only ever waits for members that the same XCD starts next, whatever other launches keep the other XCDs
// busy with (and its packets stay in that XCD's L2).  Teams go to the XCDs in turn: team t is the (t / 8)-th
// team of XCD t % 8.  The grid holds whole teams on every XCD, xch_team_grid() workgroups; those of teams past
// the last one find `false` here and leave at once.
struct XchMember {
    uint32_t team, part;
};
__device__ inline bool xch_member(uint32_t workgroup, uint32_t parts, uint32_t nteams, XchMember& m) {
    const uint32_t x = workgroup & 7u, s = workgroup >> 3;
    const uint32_t local = s / parts;
    m.part = s - local * parts;
    m.team = local * 8u + x;
    return m.team < nteams;
}
// Host: workgroups to launch for `nteams` teams of `parts` members.
inline int64_t xch_team_grid(int64_t nteams, int64_t parts) { return ceil_div(nteams, 8) * 8 * parts; }

// To be called by the first wave of a workgroup once the whole workgroup has collected its
// packets (i.e. after the barrier that follows the xch_wait calls): counts the team members that
// are done and lets the last one clear the team's `parts` slots and the counter.
__device__ inline void xch_retire(const XchLaunch& xl, uint32_t team, int parts) {
    uint64_t* counter = xl.counters + team;
    uint64_t* team_slots = xl.region + (size_t)team * parts * kXchVals;
    const int lane = threadIdx.x & 63;
    uint64_t old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t seen = __builtin_amdgcn_readfirstlane((uint32_t)old);
    if ((int)seen == parts - 1) {
        for (int i = lane; i < parts * kXchVals; i += 64)
            __hip_atomic_store(team_slots + i, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (lane == 0) __hip_atomic_store(counter, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

constexpr uint64_t kXchTimeoutTicks = 100000000ull;   // wall_clock64 counts at 100 MHz: one second

}  // namespace cpmk

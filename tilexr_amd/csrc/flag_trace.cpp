// CPU model of the tile readiness-flag protocol (see flag_trace.h): a lock-step scheduler that runs producer and
// consumer agents on host threads, one memory operation per step, and the ordering rules that a trace must obey.
//
// The producers call PublishLanded from ep_tile_publish.h -- the code the scatter kernels compile -- through an `Ops`
// whose three memory operations are steps of the scheduler.  The consumers run ClaimAndReduce from ep_token_claim.h --
// the control flow of a combine launch that may have to wait: tokens claimed from a shared counter, at most four held,
// first look, scan, trusted pass, give-up -- through an `Env` whose looks at tile words, row reads and claims are steps
// of the scheduler, with JudgeSlot deciding what a slot does about a tile that is not there and TileWordReady as the
// acceptance test, all as on the device.  What the model cannot see is the memory system below these operations
// (write-through stores, per-XCD L2s): it checks the protocol's logic, the GPU tests check its implementation.
#include "flag_trace.h"

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <map>
#include <mutex>
#include <random>
#include <set>
#include <thread>
#include <unordered_map>
#include <vector>

#include "ep_tile_publish.h"
#include "ep_token_claim.h"

namespace {

using TileXREp::ClaimAndReduce;
using TileXREp::JudgeSlot;
using TileXREp::kClaimHeld;
using TileXREp::kRouteCheck;
using TileXREp::kRouteTrusted;
using TileXREp::kSlotComeBack;
using TileXREp::kSlotExpire;
using TileXREp::PublishLanded;
using TileXREp::SlotLooksAtTile;
using TileXREp::TileCounterWords;
using TileXREp::TilePublishArgs;
using TileXREp::TileWordReady;

constexpr uint64_t kEpochBase = 1000;

struct Agent {
    bool consumer = false;
    int queue = 0;
    int position = 0;         // on a shared queue, agents of a higher position wait for all of a lower one
    bool alive = true;
};

// One agent at a time holds the turn; it performs one memory operation, appends its event and hands the turn on.
class Scheduler {
public:
    Scheduler(std::vector<Agent> agents, int mode, uint32_t seed, std::vector<TileXREpTraceEvent> *log, int round)
        : agents_(std::move(agents)), mode_(mode), rng_(seed), log_(log), round_(round)
    {
        current_ = Pick(-1, false);
    }

    template <typename Op>
    void Step(int me, bool *failedPoll, Op op)
    {
        std::unique_lock<std::mutex> lock(mu_);
        cv_.wait(lock, [&] { return current_ == me; });
        TileXREpTraceEvent e {};
        e.agent = me;
        e.queue = agents_[static_cast<size_t>(me)].queue;
        e.round = round_;
        e.tile = e.row = e.part = e.counter = -1;
        op(e);
        e.id = static_cast<int32_t>(log_->size());
        log_->push_back(e);
        current_ = Pick(me, failedPoll != nullptr && *failedPoll);
        cv_.notify_all();
    }

    void Finish(int me)
    {
        std::unique_lock<std::mutex> lock(mu_);
        cv_.wait(lock, [&] { return current_ == me; });
        agents_[static_cast<size_t>(me)].alive = false;
        current_ = Pick(me, false);
        cv_.notify_all();
    }

private:
    bool Runnable(int a) const
    {
        const Agent &g = agents_[static_cast<size_t>(a)];
        if (!g.alive) {
            return false;
        }
        for (const Agent &o : agents_) {
            if (o.alive && o.queue == g.queue && o.position < g.position) {
                return false;      // an earlier kernel of the same queue has not finished
            }
        }
        return true;
    }

    int NextFrom(int after, int wantConsumer) const      // wantConsumer: -1 any, 0 producer, 1 consumer
    {
        const int n = static_cast<int>(agents_.size());
        for (int i = 1; i <= n; ++i) {
            const int a = ((after < 0 ? -1 : after) + i) % n;
            if (Runnable(a) && (wantConsumer < 0 || agents_[static_cast<size_t>(a)].consumer == (wantConsumer == 1))) {
                return a;
            }
        }
        return -1;
    }

    int Pick(int me, bool failedPoll)
    {
        std::vector<int> ready;
        for (int a = 0; a < static_cast<int>(agents_.size()); ++a) {
            if (Runnable(a)) {
                ready.push_back(a);
            }
        }
        if (ready.empty()) {
            return -1;
        }
        int next = -1;
        switch (mode_) {
            case TILEXR_SCHED_SERIAL:
                // lowest runnable agent keeps going; a failed poll lets the others of its kind try (they all expire)
                next = failedPoll ? NextFrom(me, -1) : ready.front();
                break;
            case TILEXR_SCHED_ROUND_ROBIN:
                next = NextFrom(me, -1);
                break;
            case TILEXR_SCHED_RANDOM:
                next = ready[rng_() % ready.size()];
                if (failedPoll && next == me && ready.size() > 1) {
                    next = NextFrom(me, -1);
                }
                break;
            default:        // consumer-eager
                if (failedPoll) {
                    lastProducer_ = NextFrom(lastProducer_, 0);
                    next = lastProducer_ >= 0 ? lastProducer_ : NextFrom(me, 1);
                } else {
                    next = NextFrom(me < 0 ? -1 : me - 1, 1);
                    if (next < 0) {
                        next = NextFrom(me, 0);
                    }
                }
                break;
        }
        return next >= 0 ? next : ready.front();
    }

    std::vector<Agent> agents_;
    int mode_;
    std::mt19937 rng_;
    std::vector<TileXREpTraceEvent> *log_;
    int round_;
    int current_ = -1;
    int lastProducer_ = -1;
    std::mutex mu_;
    std::condition_variable cv_;
};

// The three memory operations of ep_tile_publish.h as scheduler steps.
struct TraceOps {
    Scheduler *sched;
    int agent;
    uint32_t *counterBase;
    uint64_t *flagBase;

    uint32_t FetchAdd(uint32_t *p)
    {
        uint32_t before = 0;
        sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
            before = (*p)++;
            e.kind = TILEXR_TRACE_COUNTER_ADD;
            e.counter = static_cast<int32_t>(p - counterBase);
            e.word = before;
        });
        return before;
    }
    void Store(uint32_t *p, uint32_t v)
    {
        sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
            *p = v;
            e.kind = TILEXR_TRACE_COUNTER_RESET;
            e.counter = static_cast<int32_t>(p - counterBase);
            e.word = v;
        });
    }
    void Store(uint64_t *p, uint64_t v)
    {
        sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
            *p = v;
            e.kind = TILEXR_TRACE_FLAG_STORE;
            e.tile = static_cast<int32_t>(p - flagBase);
            e.word = v;
            e.epoch = v >> 32;
        });
    }
};

// The operations of ep_token_claim.h for one consumer of the model: every look at a tile word, every row read and every
// claim is a step of the scheduler and an event of the trace.  A group is one token.
struct TraceClaimEnv {
    Scheduler *sched;
    const TileXREpTraceCase *c;
    int agent;
    int me;                                 // index among the consumers
    uint64_t epoch;                         // what the rows of this round hold
    uint64_t want;                          // the epoch this consumer waits for
    const std::vector<int> *rowOf;          // [tokens, topK] rows of a token, -1 = none
    const std::vector<uint64_t> *flags;
    const std::vector<uint64_t> *contents;  // epoch that last wrote each (row, part)
    uint32_t *claimCounter;                 // two words, as on the device: next token to claim, consumers that have left
    std::atomic<int> *status;               // the launch's status word
    int *wrongTokens;
    int held[kClaimHeld] = {-1, -1, -1, -1};
    int idleScans = 0;

    int RowOf(int token, int k) const { return (*rowOf)[static_cast<size_t>(token) * c->topK + k]; }
    bool Ready(uint64_t word) const
    {
        return c->inject == TILEXR_INJECT_ACCEPT_ANY_EPOCH ? word != 0 : TileWordReady(word, want);
    }
    // one look at the word of the tile that holds `row`
    bool Look(int row, bool *yield)
    {
        const int tile = row / c->shape.tileRows;
        bool ok = false;
        sched->Step(agent, yield, [&](TileXREpTraceEvent &e) {
            const uint64_t w = (*flags)[static_cast<size_t>(tile)];
            ok = Ready(w);
            e.kind = TILEXR_TRACE_FLAG_POLL;
            e.tile = tile;
            e.row = row;
            e.word = w;
            e.epoch = want;
            e.accepted = ok ? 1 : 0;
            if (yield != nullptr) {
                *yield = !ok;
            }
        });
        return ok;
    }

    int Claim(int wantGroups)
    {
        uint32_t before = 0;
        auto record = [&](TileXREpTraceEvent &e) {
            e.kind = TILEXR_TRACE_TOKEN_CLAIM;
            e.word = before;
            e.part = wantGroups;
            e.epoch = want;
        };
        if (c->inject == TILEXR_INJECT_CLAIM_NOT_ATOMIC) {
            // read, then write back in a second step: another consumer's claim in between is lost
            sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
                before = *claimCounter;
                e.kind = TILEXR_TRACE_SLEEP;
                e.part = -1;
            });
            sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
                *claimCounter = before + static_cast<uint32_t>(wantGroups);
                record(e);
            });
            return static_cast<int>(before);
        }
        sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
            before = *claimCounter;
            *claimCounter += static_cast<uint32_t>(wantGroups);
            if (c->inject == TILEXR_INJECT_CLAIM_SKIPS && me == 0) {
                before += 1;                // takes [before + 1, before + 1 + want): one token falls through
                *claimCounter += 1;
            }
            record(e);
        });
        return static_cast<int>(before);
    }
    int NextGroup(int *next) { return (*next)++; }
    void Hold(int slot, int group) { held[slot] = group; }
    void HoldDone() {}

    bool Try(int slot, int mode)
    {
        const int token = held[slot];
        // a consumer that does not wait reads whatever is there (the injected mistake of the first consumer)
        if (c->inject == TILEXR_INJECT_READ_WITHOUT_WAIT && me == 0) {
            mode = kRouteTrusted;
        }
        // the route table of the token: every slot with a row looks at its tile as the mode says (LoadRoutes)
        bool comeBack = false;
        int expiredRow = -1;
        for (int k = 0; k < c->topK; ++k) {
            const int row = RowOf(token, k);
            if (row < 0 || !SlotLooksAtTile(false, mode)) {
                continue;
            }
            bool yield = false;
            const bool there = Look(row, mode == kRouteCheck ? &yield : nullptr);
            const int verdict = JudgeSlot(false, mode, there);
            comeBack |= verdict == kSlotComeBack;
            if (verdict == kSlotExpire && expiredRow < 0) {
                expiredRow = row;
            }
        }
        if (mode == kRouteCheck && comeBack) {
            return false;
        }
        if (expiredRow >= 0) {
            sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
                *status = 1;
                e.kind = TILEXR_TRACE_WAIT_EXPIRED;
                e.tile = expiredRow / c->shape.tileRows;
                e.row = expiredRow;
                e.epoch = want;
            });
            sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
                e.kind = TILEXR_TRACE_TOKEN_ZEROED;      // a row of zeros, never a partial sum: nothing is read
                e.row = token;
                e.epoch = want;
            });
            return true;
        }
        bool bad = false;
        for (int k = 0; k < c->topK; ++k) {
            const int row = RowOf(token, k);
            if (row < 0) {
                continue;
            }
            sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
                for (int p = 0; p < c->shape.parts; ++p) {
                    bad |= (*contents)[static_cast<size_t>(row) * c->shape.parts + p] != epoch;
                }
                e.kind = TILEXR_TRACE_ROW_READ;
                e.row = row;
                e.tile = row / c->shape.tileRows;
                e.epoch = want;
            });
        }
        sched->Step(agent, nullptr, [&](TileXREpTraceEvent &e) {
            e.kind = TILEXR_TRACE_TOKEN_REDUCED;
            e.row = token;
            e.epoch = want;
        });
        *wrongTokens += bad ? 1 : 0;
        return true;
    }

    uint32_t Scan(uint32_t pending)
    {
        if (c->inject == TILEXR_INJECT_TRUST_WITHOUT_SCAN && me == 0) {
            return 0u;                      // "all ready" without a look
        }
        uint32_t notReady = 0u;
        for (int slot = 0; slot < kClaimHeld; ++slot) {
            if (((pending >> slot) & 1u) == 0u) {
                continue;
            }
            for (int k = 0; k < c->topK; ++k) {
                const int row = RowOf(held[slot], k);
                if (row >= 0 && !Look(row, nullptr)) {
                    notReady |= 1u << slot;
                }
            }
        }
        return notReady;
    }
    bool GiveUpNow()
    {
        if (c->inject == TILEXR_INJECT_IMPATIENT_CONSUMER && me == 0) {
            return true;
        }
        return ++idleScans > c->pollBudget || *status != 0;
    }
    void Touch() { idleScans = 0; }
    void Leave()
    {
        // LeaveClaimWords of ep_token_claim.h, its memory operations as steps of the scheduler
        struct LeaveOps {
            TraceClaimEnv *env;
            uint32_t FetchAdd(uint32_t *p)
            {
                uint32_t before = 0;
                env->sched->Step(env->agent, nullptr, [&](TileXREpTraceEvent &e) {
                    before = (*p)++;
                    e.kind = TILEXR_TRACE_CONSUMER_LEAVE;
                    e.word = before;
                    e.epoch = env->want;
                });
                return before;
            }
            void Store(uint32_t *p, uint32_t v)
            {
                env->sched->Step(env->agent, nullptr, [&](TileXREpTraceEvent &e) {
                    *p = v;
                    e.kind = TILEXR_TRACE_CLAIM_RESET;
                    e.counter = static_cast<int32_t>(p - env->claimCounter);
                    e.word = v;
                    e.epoch = env->want;
                });
            }
        } ops {this};
        if (c->inject == TILEXR_INJECT_NO_CLAIM_RESET) {
            ops.FetchAdd(&claimCounter[1]);      // counts itself out, and nobody puts the words back
            return;
        }
        TileXREp::LeaveClaimWords(ops, claimCounter, static_cast<uint32_t>(c->consumers));
    }
    void Sleep(int level)
    {
        bool yield = true;                  // nothing was ready: somebody else gets the turn
        sched->Step(agent, &yield, [&](TileXREpTraceEvent &e) {
            e.kind = TILEXR_TRACE_SLEEP;
            e.part = level;
            e.epoch = want;
        });
    }
};

int Priority(int kind)
{
    switch (kind) {
        case TILEXR_FINDING_DEADLOCK: return 0;
        case TILEXR_FINDING_FLAG_STALE_EPOCH: return 1;
        case TILEXR_FINDING_FLAG_NO_PRODUCER: return 2;
        case TILEXR_FINDING_READ_BEFORE_WRITE: return 3;
        case TILEXR_FINDING_READ_WITHOUT_WAIT: return 4;
        case TILEXR_FINDING_TOKEN_REDUCED_WHILE_PENDING: return 4;
        case TILEXR_FINDING_TOKEN_CLAIMED_TWICE: return 4;
        case TILEXR_FINDING_TOKEN_NEVER_CLAIMED: return 4;
        case TILEXR_FINDING_CLAIM_WORD_NOT_RESET: return 4;
        case TILEXR_FINDING_PUBLISH_BEFORE_LANDED: return 5;
        case TILEXR_FINDING_DOUBLE_PUBLISH: return 6;
        case TILEXR_FINDING_WRONG_WORD: return 7;
        case TILEXR_FINDING_COUNTER_NOT_ZERO: return 8;
        default: return 9;
    }
}

} // namespace

extern "C" {

const char *TileXREpTraceFindingName(int32_t kind)
{
    switch (kind) {
        case TILEXR_FINDING_READ_BEFORE_WRITE: return "READ_BEFORE_WRITE";
        case TILEXR_FINDING_FLAG_STALE_EPOCH: return "FLAG_STALE_EPOCH";
        case TILEXR_FINDING_FLAG_NO_PRODUCER: return "FLAG_NO_PRODUCER";
        case TILEXR_FINDING_DEADLOCK: return "DEADLOCK";
        case TILEXR_FINDING_DOUBLE_PUBLISH: return "DOUBLE_PUBLISH";
        case TILEXR_FINDING_PUBLISH_BEFORE_LANDED: return "PUBLISH_BEFORE_LANDED";
        case TILEXR_FINDING_COUNTER_NOT_ZERO: return "COUNTER_NOT_ZERO";
        case TILEXR_FINDING_WRONG_WORD: return "WRONG_WORD";
        case TILEXR_FINDING_READ_WITHOUT_WAIT: return "READ_WITHOUT_WAIT";
        case TILEXR_FINDING_WAIT_EXPIRED_EARLY: return "WAIT_EXPIRED_EARLY";
        case TILEXR_FINDING_TOKEN_REDUCED_WHILE_PENDING: return "TOKEN_REDUCED_WHILE_PENDING";
        case TILEXR_FINDING_TOKEN_CLAIMED_TWICE: return "TOKEN_CLAIMED_TWICE";
        case TILEXR_FINDING_TOKEN_NEVER_CLAIMED: return "TOKEN_NEVER_CLAIMED";
        case TILEXR_FINDING_CLAIM_WORD_NOT_RESET: return "CLAIM_WORD_NOT_RESET";
        default: return "UNKNOWN";
    }
}

int TileXREpTraceRun(const TileXREpTraceCase *c, TileXREpTraceEvent *events, int32_t maxEvents, int32_t *numEvents,
    int32_t *wrongTokens)
{
    if (c == nullptr || numEvents == nullptr || (events == nullptr && maxEvents > 0)) {
        return -1;
    }
    const TileXREpTraceShape &sh = c->shape;
    if (sh.totalRows < 0 || sh.maxRows < sh.totalRows || sh.maxRows <= 0 || sh.tileRows <= 0 || sh.parts <= 0 ||
        sh.parts > 64 || c->topK <= 0 || c->producers <= 0 || c->consumers <= 0 || c->producers + c->consumers > 64 ||
        c->rounds <= 0 || c->pollBudget <= 0 || c->scheduler < 0 || c->scheduler > TILEXR_SCHED_CONSUMER_EAGER ||
        (sh.tokens != 0 && sh.tokens != (sh.totalRows + c->topK - 1) / c->topK)) {
        return -1;
    }
    const int maxTiles = (sh.maxRows + sh.tileRows - 1) / sh.tileRows;
    std::vector<uint32_t> counters(static_cast<size_t>(TileCounterWords(sh.maxRows, sh.tileRows)), 0u);
    std::vector<uint64_t> flags(static_cast<size_t>(maxTiles), 0ull);
    // what memory holds: the epoch that last wrote each (row, part)
    std::vector<uint64_t> contents(static_cast<size_t>(sh.maxRows) * sh.parts, 0ull);
    uint32_t claimWords[2] = {0u, 0u};      // what the waiting launches claim their tokens from: zero once, then left at
                                            // zero by every launch's last leaver
    std::vector<TileXREpTraceEvent> log;
    std::mt19937 rng(c->seed);
    int wrong = 0;
    const int tokens = (sh.totalRows + c->topK - 1) / c->topK;

    for (int round = 1; round <= c->rounds; ++round) {
        const uint64_t epoch = kEpochBase + static_cast<uint64_t>(round);
        const int agentsN = c->producers + c->consumers;
        std::vector<Agent> agents(static_cast<size_t>(agentsN));
        for (int a = 0; a < agentsN; ++a) {
            Agent &g = agents[static_cast<size_t>(a)];
            g.consumer = a >= c->producers;
            if (c->inject == TILEXR_INJECT_CONSUMER_ENQUEUED_FIRST) {
                g.queue = 0;
                g.position = g.consumer ? 0 : 1;
            } else {
                g.queue = g.consumer ? 1 : 0;
                g.position = 0;
            }
        }
        for (int a = 0; a < agentsN; ++a) {
            TileXREpTraceEvent e {};
            e.id = static_cast<int32_t>(log.size());
            e.kind = TILEXR_TRACE_LAUNCH;
            e.agent = a;
            e.queue = agents[static_cast<size_t>(a)].queue;
            e.part = agents[static_cast<size_t>(a)].position;
            e.tile = e.row = e.counter = -1;
            e.round = round;
            e.epoch = epoch;
            log.push_back(e);
        }
        // producers: every (row, part) once, in a seeded order; consumers: rows dealt to tokens by a seeded permutation
        std::vector<int> landings(static_cast<size_t>(sh.totalRows) * sh.parts);
        for (size_t i = 0; i < landings.size(); ++i) {
            landings[i] = static_cast<int>(i);
        }
        std::shuffle(landings.begin(), landings.end(), rng);
        std::vector<int> rowOf(static_cast<size_t>(tokens) * c->topK, -1);
        for (int r = 0; r < sh.totalRows; ++r) {
            rowOf[static_cast<size_t>(r)] = r;
        }
        std::shuffle(rowOf.begin(), rowOf.end(), rng);
        const int victim = landings.empty() ? -1 : landings[rng() % landings.size()];

        Scheduler sched(agents, c->scheduler, rng(), &log, round);
        std::vector<int> wrongPerConsumer(static_cast<size_t>(c->consumers), 0);
        std::atomic<int> status {0};    // the launch's status word: set by the first expired wait
        std::vector<std::thread> pool;
        for (int a = 0; a < agentsN; ++a) {
            if (a < c->producers) {
                pool.emplace_back([&, a] {
                    TilePublishArgs t {};
                    t.flags = flags.data();
                    t.counters = counters.data();
                    t.tileRows = sh.tileRows;
                    t.maxTiles = maxTiles;
                    t.totalRows = sh.totalRows;
                    t.epoch = epoch;
                    TraceOps ops {&sched, a, counters.data(), flags.data()};
                    for (size_t i = static_cast<size_t>(a); i < landings.size(); i += static_cast<size_t>(c->producers)) {
                        const int row = landings[i] / sh.parts;
                        const int part = landings[i] % sh.parts;
                        auto write = [&] {
                            sched.Step(a, nullptr, [&](TileXREpTraceEvent &e) {
                                contents[static_cast<size_t>(row) * sh.parts + part] = epoch;
                                e.kind = TILEXR_TRACE_ROW_WRITE;
                                e.row = row;
                                e.part = part;
                                e.tile = row / sh.tileRows;
                                e.epoch = epoch;
                            });
                        };
                        if (c->inject == TILEXR_INJECT_REPORT_BEFORE_WRITE) {
                            PublishLanded(ops, t, row, sh.parts);
                            write();
                            continue;
                        }
                        write();
                        if (c->inject == TILEXR_INJECT_MISSING_PRODUCER && landings[i] == victim) {
                            continue;
                        }
                        PublishLanded(ops, t, row, sh.parts);
                        if (c->inject == TILEXR_INJECT_DOUBLE_REPORT && landings[i] == victim) {
                            PublishLanded(ops, t, row, sh.parts);
                        }
                    }
                    sched.Finish(a);
                });
            } else {
                pool.emplace_back([&, a] {
                    const int me = a - c->producers;
                    TraceClaimEnv env {&sched, c, a, me, epoch, c->inject == TILEXR_INJECT_OLD_EPOCH_CONSUMER ? epoch - 1 : epoch,
                        &rowOf, &flags, &contents, claimWords, &status, &wrongPerConsumer[static_cast<size_t>(me)]};
                    ClaimAndReduce(env, tokens);
                    sched.Finish(a);
                });
            }
        }
        for (auto &th : pool) {
            th.join();
        }
        for (int w : wrongPerConsumer) {
            wrong += w;
        }
        TileXREpTraceEvent end {};
        end.id = static_cast<int32_t>(log.size());
        end.kind = TILEXR_TRACE_ROUND_END;
        end.agent = end.tile = end.row = end.part = end.counter = -1;
        end.round = round;
        end.epoch = epoch;
        log.push_back(end);
    }
    *numEvents = static_cast<int32_t>(log.size());
    if (wrongTokens != nullptr) {
        *wrongTokens = wrong;
    }
    if (static_cast<int64_t>(log.size()) > maxEvents) {
        return -2;
    }
    std::copy(log.begin(), log.end(), events);
    return 0;
}

int TileXREpTraceCheck(const TileXREpTraceShape *shape, const TileXREpTraceEvent *events, int32_t numEvents,
    TileXREpTraceFinding *findings, int32_t maxFindings)
{
    if (shape == nullptr || numEvents < 0 || (events == nullptr && numEvents > 0) || (findings == nullptr && maxFindings > 0) ||
        shape->tileRows <= 0 || shape->parts <= 0 || shape->parts > 64 || shape->totalRows < 0 || shape->tokens < 0) {
        return -1;
    }
    std::vector<TileXREpTraceFinding> out;
    auto report = [&](int kind, const TileXREpTraceEvent &e) {
        TileXREpTraceFinding f {};
        f.kind = kind;
        f.event = e.id;
        f.agent = e.agent;
        f.tile = e.tile;
        f.row = e.row;
        f.round = e.round;
        f.epoch = e.epoch;
        out.push_back(f);
    };
    const uint64_t allParts = shape->parts == 64 ? ~0ull : ((1ull << shape->parts) - 1);
    auto rowsInTile = [&](int tile) {
        const int left = shape->totalRows - tile * shape->tileRows;
        return left < shape->tileRows ? left : shape->tileRows;
    };

    // every store of a readiness word, wherever it sits in the trace: a wait is judged against all of them
    std::map<std::pair<int, uint64_t>, std::vector<int>> storesOf;      // (tile, epoch) -> event ids
    std::unordered_map<int, std::pair<int, int>> launchOf;              // agent -> (queue, position), last launch wins per round
    for (int i = 0; i < numEvents; ++i) {
        if (events[i].kind == TILEXR_TRACE_FLAG_STORE) {
            storesOf[{events[i].tile, events[i].word >> 32}].push_back(i);
        }
    }

    std::map<std::pair<uint64_t, int>, uint64_t> written;               // (epoch, row) -> mask of parts written so far
    std::map<int, uint64_t> newestStored;                               // tile -> highest epoch stored so far
    std::set<std::tuple<int, int, uint64_t>> sawReady;                  // (agent, tile, epoch) accepted polls
    std::set<std::tuple<int, int, uint64_t>> staleReported;
    std::map<int, int64_t> counterValue;
    std::set<int> counterReported;
    // the consumer side's bookkeeping, per round: who claimed which token, which tokens were finished (summed or given a
    // row of zeros), and the rows an agent has read since its last token event
    std::map<std::pair<int, int>, int> claimsOf;                        // (round, token) -> claims
    std::map<std::pair<int, int>, int> finishedOf;                      // (round, token) -> times finished
    std::map<int, std::vector<int>> readsSince;                         // agent -> ids of ROW_READ events
    std::set<int> roundsWithClaims;
    auto finish = [&](const TileXREpTraceEvent &e) {
        if (++finishedOf[{e.round, e.row}] == 2) {
            report(TILEXR_FINDING_TOKEN_CLAIMED_TWICE, e);
        }
        readsSince[e.agent].clear();
    };
    for (int i = 0; i < numEvents; ++i) {
        const TileXREpTraceEvent &e = events[i];
        switch (e.kind) {
            case TILEXR_TRACE_LAUNCH:
                launchOf[e.agent] = {e.queue, e.part};
                break;
            case TILEXR_TRACE_ROW_WRITE:
                if (e.part >= 0 && e.part < 64) {
                    written[{e.epoch, e.row}] |= 1ull << e.part;
                }
                break;
            case TILEXR_TRACE_COUNTER_ADD:
                counterValue[e.counter] += 1;
                break;
            case TILEXR_TRACE_COUNTER_RESET:
                counterValue[e.counter] = static_cast<int64_t>(e.word);
                break;
            case TILEXR_TRACE_FLAG_STORE: {
                const uint64_t epoch = e.word >> 32;
                const std::vector<int> &all = storesOf[{e.tile, epoch}];
                if (all.size() > 1 && all.front() != i) {
                    report(TILEXR_FINDING_DOUBLE_PUBLISH, e);
                }
                const int rows = rowsInTile(e.tile);
                bool landed = rows > 0;
                for (int r = 0; r < rows && landed; ++r) {
                    const auto it = written.find({epoch, e.tile * shape->tileRows + r});
                    landed = it != written.end() && it->second == allParts;
                }
                if (!landed) {
                    report(TILEXR_FINDING_PUBLISH_BEFORE_LANDED, e);
                }
                if (static_cast<int64_t>(e.word & 0xffffffffull) != rows) {
                    report(TILEXR_FINDING_WRONG_WORD, e);
                }
                uint64_t &newest = newestStored[e.tile];
                newest = std::max(newest, epoch);
                break;
            }
            case TILEXR_TRACE_FLAG_POLL: {
                const auto key = std::make_tuple(e.agent, e.tile, e.epoch);
                if (e.accepted != 0) {
                    sawReady.insert(key);
                }
                const auto newest = newestStored.find(e.tile);
                const bool acceptedOther = e.accepted != 0 && (e.word >> 32) != e.epoch;
                const bool waitsForPast = newest != newestStored.end() && newest->second > e.epoch;
                if ((acceptedOther || waitsForPast) && staleReported.insert(key).second) {
                    report(TILEXR_FINDING_FLAG_STALE_EPOCH, e);
                }
                break;
            }
            case TILEXR_TRACE_WAIT_EXPIRED: {
                const auto it = storesOf.find({e.tile, e.epoch});
                if (it == storesOf.end()) {
                    if (staleReported.count(std::make_tuple(e.agent, e.tile, e.epoch)) == 0) {
                        report(TILEXR_FINDING_FLAG_NO_PRODUCER, e);
                    }
                    break;
                }
                if (it->second.front() < i) {
                    break;      // published before this wait gave up: it gave up because an earlier wait had expired
                }
                const TileXREpTraceEvent &store = events[it->second.front()];
                const auto mine = launchOf.find(e.agent);
                const auto theirs = launchOf.find(store.agent);
                const bool behind = mine != launchOf.end() && theirs != launchOf.end() &&
                    mine->second.first == theirs->second.first && theirs->second.second > mine->second.second;
                report(behind ? TILEXR_FINDING_DEADLOCK : TILEXR_FINDING_WAIT_EXPIRED_EARLY, e);
                break;
            }
            case TILEXR_TRACE_ROW_READ: {
                const auto it = written.find({e.epoch, e.row});
                if (it == written.end() || it->second != allParts) {
                    report(TILEXR_FINDING_READ_BEFORE_WRITE, e);
                }
                if (sawReady.count(std::make_tuple(e.agent, e.row / shape->tileRows, e.epoch)) == 0) {
                    report(TILEXR_FINDING_READ_WITHOUT_WAIT, e);
                }
                readsSince[e.agent].push_back(i);
                break;
            }
            case TILEXR_TRACE_CONSUMER_LEAVE:
            case TILEXR_TRACE_CLAIM_RESET:
                break;
            case TILEXR_TRACE_TOKEN_CLAIM: {
                // the first claim of a launch finds the counter at zero: the launch before has left it so
                if (shape->tokens > 0 && roundsWithClaims.insert(e.round).second && e.word != 0) {
                    report(TILEXR_FINDING_CLAIM_WORD_NOT_RESET, e);
                }
                bool overlap = false;
                for (int64_t t = static_cast<int64_t>(e.word); t < static_cast<int64_t>(e.word) + e.part; ++t) {
                    if (t < shape->tokens) {
                        overlap |= ++claimsOf[{e.round, static_cast<int>(t)}] > 1;
                    }
                }
                if (overlap) {
                    report(TILEXR_FINDING_TOKEN_CLAIMED_TWICE, e);
                }
                break;
            }
            case TILEXR_TRACE_TOKEN_REDUCED: {
                // every row that went into the sum: had its tile been published for the epoch when it was read?
                for (int readId : readsSince[e.agent]) {
                    const TileXREpTraceEvent &r = events[readId];
                    const auto it = storesOf.find({r.tile, r.epoch});
                    if (it == storesOf.end() || it->second.front() > readId) {
                        report(TILEXR_FINDING_TOKEN_REDUCED_WHILE_PENDING, e);
                        out.back().tile = r.tile;
                        break;
                    }
                }
                finish(e);
                break;
            }
            case TILEXR_TRACE_TOKEN_ZEROED:
                finish(e);
                break;
            case TILEXR_TRACE_SLEEP:
                break;
            case TILEXR_TRACE_ROUND_END:
                for (int t = 0; t < shape->tokens; ++t) {
                    if (claimsOf.count({e.round, t}) == 0 || finishedOf.count({e.round, t}) == 0) {
                        TileXREpTraceEvent at = e;
                        at.row = t;
                        report(TILEXR_FINDING_TOKEN_NEVER_CLAIMED, at);
                    }
                }
                for (const auto &cv : counterValue) {
                    if (cv.second != 0 && counterReported.insert(cv.first).second) {
                        TileXREpTraceEvent at = e;
                        at.counter = cv.first;
                        report(TILEXR_FINDING_COUNTER_NOT_ZERO, at);
                        out.back().tile = cv.first;      // the counter's index
                    }
                }
                break;
            default:
                return -1;
        }
    }
    std::stable_sort(out.begin(), out.end(), [](const TileXREpTraceFinding &a, const TileXREpTraceFinding &b) {
        const int pa = Priority(a.kind);
        const int pb = Priority(b.kind);
        return pa != pb ? pa < pb : a.event < b.event;
    });
    for (int i = 0; i < static_cast<int>(out.size()) && i < maxFindings; ++i) {
        findings[i] = out[static_cast<size_t>(i)];
    }
    return static_cast<int>(out.size());
}

}

/* CPU model of the tile readiness-flag protocol: an abstract event trace and ordering diagnostics over it.
 *
 * Test infrastructure (it is linked into the hooks library, not into libtilexr-ep.so).  Both sides of the model run
 * the very code the kernels compile: the producers ep_tile_publish.h (PublishLanded, CountLanded), the consumers
 * ep_token_claim.h (ClaimAndReduce: tokens claimed from a shared counter, at most four held, scan, trusted pass,
 * give-up and status word; JudgeSlot: what a slot does about a tile that is not there) with the kernels' acceptance
 * test (TileWordReady).  Each memory operation is one step of a seeded scheduler and one event of the trace.  The
 * diagnostics are a pure function of a trace, so hand-written traces can be checked too.
 *
 * The idea follows the reference's no-NPU checker (tools/checker/src/diagnostics.cpp:323-440: an event log of
 * READ / WRITE / FLAG_STORE / FLAG_WAIT and rules such as READ_BEFORE_WRITE, FLAG_STALE_MAGIC, FLAG_NO_PRODUCER,
 * DEADLOCK; tools/checker/README.md:251-266, injection switches :151-152); the events and rules here are those of
 * this library's own protocol. */
#ifndef TILEXR_AMD_FLAG_TRACE_H
#define TILEXR_AMD_FLAG_TRACE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#pragma GCC visibility push(default)
#endif

enum {
    TILEXR_TRACE_LAUNCH = 0,          /* agent joins `queue` at position `part` (lower runs first on a shared queue) */
    TILEXR_TRACE_ROW_WRITE = 1,       /* part `part` of row `row` is complete in memory for epoch `epoch` */
    TILEXR_TRACE_COUNTER_ADD = 2,     /* atomic +1 on counter `counter`; `word` = value before */
    TILEXR_TRACE_COUNTER_RESET = 3,   /* counter `counter` stored back to `word` (0) */
    TILEXR_TRACE_FLAG_STORE = 4,      /* readiness word of `tile` stored as `word` */
    TILEXR_TRACE_FLAG_POLL = 5,       /* consumer read `word` from `tile`, wants `epoch`; `accepted` = took it as ready */
    TILEXR_TRACE_WAIT_EXPIRED = 6,    /* consumer gave up waiting for `tile` / `epoch` */
    TILEXR_TRACE_ROW_READ = 7,        /* consumer read row `row` expecting the contents of `epoch` */
    TILEXR_TRACE_ROUND_END = 8,       /* all agents of one dispatch + combine are done */
    TILEXR_TRACE_TOKEN_CLAIM = 9,     /* consumer took tokens [word, word + part) from the shared claim counter */
    TILEXR_TRACE_TOKEN_REDUCED = 10,  /* consumer summed token `row` from the rows it has read since its last token event */
    TILEXR_TRACE_TOKEN_ZEROED = 11,   /* consumer gave token `row` a row of zeros (a wait of its tiles expired) */
    TILEXR_TRACE_SLEEP = 12,          /* consumer found nothing ready and backs off (`part` = level) */
    TILEXR_TRACE_CONSUMER_LEAVE = 13, /* consumer has claimed for the last time: +1 on the leavers' word, `word` = value before */
    TILEXR_TRACE_CLAIM_RESET = 14     /* the last leaver stored `word` (0) to claim word `counter` (1: leavers, 0: next token) */
};

typedef struct {
    int32_t id;           /* position in the trace */
    int32_t kind;
    int32_t agent;        /* producers are 0 .. producers-1, consumers follow */
    int32_t queue;
    int32_t tile;
    int32_t row;
    int32_t part;
    int32_t counter;
    int32_t accepted;
    int32_t round;
    uint64_t word;
    uint64_t epoch;
} TileXREpTraceEvent;

enum {
    TILEXR_FINDING_READ_BEFORE_WRITE = 1,      /* a row was read before every part of it was written in that epoch */
    TILEXR_FINDING_FLAG_STALE_EPOCH = 2,       /* a poll accepted a word of another epoch, or waits for an epoch older
                                                  than one already stored on that tile */
    TILEXR_FINDING_FLAG_NO_PRODUCER = 3,       /* a wait expired and nobody ever stores that tile for that epoch */
    TILEXR_FINDING_DEADLOCK = 4,               /* a wait expired because its producer sits behind the waiting kernel on
                                                  the same queue */
    TILEXR_FINDING_DOUBLE_PUBLISH = 5,         /* a tile's word was stored twice for one epoch */
    TILEXR_FINDING_PUBLISH_BEFORE_LANDED = 6,  /* a tile's word was stored before all parts of all its rows were written */
    TILEXR_FINDING_COUNTER_NOT_ZERO = 7,       /* a landing counter did not return to zero by the end of the round */
    TILEXR_FINDING_WRONG_WORD = 8,             /* a stored word's lower half is not the tile's row count */
    TILEXR_FINDING_READ_WITHOUT_WAIT = 9,      /* a row was read by an agent that never saw its tile ready for the epoch */
    TILEXR_FINDING_WAIT_EXPIRED_EARLY = 10,    /* a wait expired although the tile is published later (bound too short) */
    TILEXR_FINDING_TOKEN_REDUCED_WHILE_PENDING = 11, /* a token was summed although a tile of one of its rows had not
                                                  been published for the epoch yet */
    TILEXR_FINDING_TOKEN_CLAIMED_TWICE = 12,   /* two claims of a round overlap, or a token was finished twice */
    TILEXR_FINDING_TOKEN_NEVER_CLAIMED = 13,   /* a token of the round was never claimed or never finished */
    TILEXR_FINDING_CLAIM_WORD_NOT_RESET = 14   /* a round's first claim did not find the claim counter at zero */
};

typedef struct {
    int32_t kind;
    int32_t event;        /* id of the event the finding is about */
    int32_t agent;
    int32_t tile;
    int32_t row;
    int32_t round;
    uint64_t epoch;
} TileXREpTraceFinding;

typedef struct {
    int32_t totalRows;    /* rows the dispatch keeps */
    int32_t maxRows;      /* rows the counters are sized for (>= totalRows) */
    int32_t tileRows;
    int32_t parts;        /* publishers per row (column slices) */
    int32_t tokens;       /* tokens a combine reduces per round; 0: unknown, the claim rules are not applied */
} TileXREpTraceShape;

enum {
    TILEXR_SCHED_SERIAL = 0,          /* producers to completion, then consumers */
    TILEXR_SCHED_ROUND_ROBIN = 1,
    TILEXR_SCHED_RANDOM = 2,          /* seeded */
    TILEXR_SCHED_CONSUMER_EAGER = 3   /* consumers run whenever they can; a failed poll lets one producer step run */
};

enum {
    TILEXR_INJECT_NONE = 0,
    TILEXR_INJECT_READ_WITHOUT_WAIT = 1,   /* one consumer reads its rows without polling */
    TILEXR_INJECT_ACCEPT_ANY_EPOCH = 2,    /* consumers take any non-zero word as ready */
    TILEXR_INJECT_MISSING_PRODUCER = 3,    /* one row's last part is written but never reported */
    TILEXR_INJECT_DOUBLE_REPORT = 4,       /* one part is reported twice */
    TILEXR_INJECT_REPORT_BEFORE_WRITE = 5, /* parts are reported before they are written */
    TILEXR_INJECT_CONSUMER_ENQUEUED_FIRST = 6, /* one shared queue, the waiting kernel ahead of its producer */
    TILEXR_INJECT_OLD_EPOCH_CONSUMER = 7,  /* consumers wait for the previous round's epoch */
    TILEXR_INJECT_TRUST_WITHOUT_SCAN = 8,  /* one consumer's scan reports every held token ready without looking */
    TILEXR_INJECT_CLAIM_NOT_ATOMIC = 9,    /* the claim counter is read and written back in two steps */
    TILEXR_INJECT_CLAIM_SKIPS = 10,        /* one consumer's claims start one token late */
    TILEXR_INJECT_IMPATIENT_CONSUMER = 11, /* one consumer gives up after its first scan without a ready token */
    TILEXR_INJECT_NO_CLAIM_RESET = 12      /* nobody puts the claim words back to zero when the launch is over */
};

typedef struct {
    TileXREpTraceShape shape;
    int32_t topK;          /* rows a consumer gathers per token: rows are dealt to tokens by a seeded permutation
                              (shape.tokens must be 0 or ceil(totalRows / topK)) */
    int32_t producers;
    int32_t consumers;
    int32_t rounds;        /* dispatch + combine pairs in a row on the same flags and counters */
    int32_t scheduler;
    int32_t inject;
    int32_t pollBudget;    /* scans without a ready token after which what a consumer holds is given up (stands for the
                              wall-clock bound) */
    uint32_t seed;
} TileXREpTraceCase;

/* Runs the model and writes its trace (at most maxEvents events; *numEvents receives the full count).  Returns 0, or
 * -1 for a bad case, -2 when the trace did not fit.  `wrongTokens` (optional) receives the number of tokens whose
 * gathered rows did not all carry the round's contents. */
int TileXREpTraceRun(const TileXREpTraceCase *c, TileXREpTraceEvent *events, int32_t maxEvents, int32_t *numEvents,
    int32_t *wrongTokens);

/* Checks a trace against the protocol's rules.  Writes at most maxFindings findings, most severe kinds first within
 * the order of the trace; returns the total number found (or -1 for bad arguments). */
int TileXREpTraceCheck(const TileXREpTraceShape *shape, const TileXREpTraceEvent *events, int32_t numEvents,
    TileXREpTraceFinding *findings, int32_t maxFindings);

const char *TileXREpTraceFindingName(int32_t kind);

#ifdef __cplusplus
#pragma GCC visibility pop
}
#endif

#endif /* TILEXR_AMD_FLAG_TRACE_H */

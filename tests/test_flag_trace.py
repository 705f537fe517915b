"""The readiness-flag protocol on the CPU: an abstract event trace of producers (the scatter kernels' own publishing
code, tilexr_amd/csrc/ep_tile_publish.h) and consumers (the reduce kernels' acceptance test) under seeded schedules,
and the ordering rules a trace must obey (tilexr_amd/csrc/flag_trace.h).

Three layers: (1) the rules on hand-written traces, one minimal trace per rule, so that each rule is pinned by
something other than the model that produces traces; (2) clean runs of the model over shapes, schedules and seeds
give no finding and no wrong token; (3) every injection switch makes its rule fire.  The reference has the same
structure for its own protocols: an event log with READ_BEFORE_WRITE / stale flag / missing producer / deadlock rules
(tools/checker/src/diagnostics.cpp:323-440) and injection switches that prove they fire
(tools/checker/README.md:146-152).
"""
import ctypes as C

import pytest

import hostlib as H

(LAUNCH, ROW_WRITE, COUNTER_ADD, COUNTER_RESET, FLAG_STORE, FLAG_POLL, WAIT_EXPIRED, ROW_READ, ROUND_END, TOKEN_CLAIM,
 TOKEN_REDUCED, TOKEN_ZEROED, SLEEP, CONSUMER_LEAVE, CLAIM_RESET) = range(15)
(READ_BEFORE_WRITE, FLAG_STALE_EPOCH, FLAG_NO_PRODUCER, DEADLOCK, DOUBLE_PUBLISH, PUBLISH_BEFORE_LANDED,
 COUNTER_NOT_ZERO, WRONG_WORD, READ_WITHOUT_WAIT, WAIT_EXPIRED_EARLY, TOKEN_REDUCED_WHILE_PENDING, TOKEN_CLAIMED_TWICE,
 TOKEN_NEVER_CLAIMED, CLAIM_WORD_NOT_RESET) = range(1, 15)
SERIAL, ROUND_ROBIN, RANDOM, CONSUMER_EAGER = range(4)
(INJECT_NONE, INJECT_READ_WITHOUT_WAIT, INJECT_ACCEPT_ANY_EPOCH, INJECT_MISSING_PRODUCER, INJECT_DOUBLE_REPORT,
 INJECT_REPORT_BEFORE_WRITE, INJECT_CONSUMER_ENQUEUED_FIRST, INJECT_OLD_EPOCH_CONSUMER, INJECT_TRUST_WITHOUT_SCAN,
 INJECT_CLAIM_NOT_ATOMIC, INJECT_CLAIM_SKIPS, INJECT_IMPATIENT_CONSUMER, INJECT_NO_CLAIM_RESET) = range(13)


class Event(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("id", "kind", "agent", "queue", "tile", "row", "part", "counter", "accepted",
                                          "round")] + [("word", C.c_uint64), ("epoch", C.c_uint64)]


class Finding(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("kind", "event", "agent", "tile", "row", "round")] + [("epoch", C.c_uint64)]


class Shape(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("totalRows", "maxRows", "tileRows", "parts", "tokens")]


class Case(C.Structure):
    _fields_ = [("shape", Shape)] + [(n, C.c_int32) for n in ("topK", "producers", "consumers", "rounds", "scheduler",
                                                               "inject", "pollBudget")] + [("seed", C.c_uint32)]


def lib():
    l = H.lib()
    l.TileXREpTraceRun.argtypes = [C.POINTER(Case), C.POINTER(Event), C.c_int32, C.POINTER(C.c_int32),
                                   C.POINTER(C.c_int32)]
    l.TileXREpTraceCheck.argtypes = [C.POINTER(Shape), C.POINTER(Event), C.c_int32, C.POINTER(Finding), C.c_int32]
    l.TileXREpTraceFindingName.restype = C.c_char_p
    return l


def check(shape, events):
    arr = (Event * max(1, len(events)))(*events)
    for i, e in enumerate(events):
        arr[i].id = i
    out = (Finding * 256)()
    n = lib().TileXREpTraceCheck(C.byref(shape), arr, len(events), out, 256)
    assert n >= 0
    return [out[i] for i in range(min(n, 256))]


def kinds(findings):
    return sorted({f.kind for f in findings})


def ev(kind, agent=0, queue=0, tile=-1, row=-1, part=-1, counter=-1, accepted=0, round_=1, word=0, epoch=0):
    return Event(0, kind, agent, queue, tile, row, part, counter, accepted, round_, word, epoch)


def word(epoch, rows):
    return (epoch << 32) | rows


# ---------------------------------------------------------------------------------------------------------------
# (1) the rules, on hand-written traces: two rows of one part in one tile, one producer (agent 0), one consumer (1)
# ---------------------------------------------------------------------------------------------------------------
SHAPE = Shape(2, 2, 2, 1, 0)
E = 7


def good_trace():
    return [
        ev(LAUNCH, agent=0, queue=0, part=0, epoch=E), ev(LAUNCH, agent=1, queue=1, part=0, epoch=E),
        ev(ROW_WRITE, 0, tile=0, row=0, part=0, epoch=E), ev(COUNTER_ADD, 0, counter=0, word=0),
        ev(FLAG_POLL, 1, 1, tile=0, row=0, word=word(E - 1, 2), epoch=E, accepted=0),
        ev(ROW_WRITE, 0, tile=0, row=1, part=0, epoch=E), ev(COUNTER_ADD, 0, counter=0, word=1),
        ev(COUNTER_RESET, 0, counter=0, word=0), ev(FLAG_STORE, 0, tile=0, word=word(E, 2), epoch=E),
        ev(FLAG_POLL, 1, 1, tile=0, row=0, word=word(E, 2), epoch=E, accepted=1),
        ev(ROW_READ, 1, 1, tile=0, row=0, epoch=E), ev(ROW_READ, 1, 1, tile=0, row=1, epoch=E),
        ev(ROUND_END, agent=-1, epoch=E),
    ]


def test_a_correct_hand_written_trace_has_no_finding():
    assert check(SHAPE, good_trace()) == []


def test_read_before_write_rule():
    t = good_trace()
    t.insert(4, ev(ROW_READ, 1, 1, tile=0, row=1, epoch=E))        # row 1 is written later in the trace
    f = check(SHAPE, t)
    assert READ_BEFORE_WRITE in kinds(f) and READ_WITHOUT_WAIT in kinds(f)
    assert [x.row for x in f if x.kind == READ_BEFORE_WRITE] == [1]
    # a read of the previous epoch's contents that were complete is not this finding: it is a stale acceptance
    t = good_trace()
    t[9] = ev(FLAG_POLL, 1, 1, tile=0, row=0, word=word(E - 1, 2), epoch=E, accepted=1)
    assert FLAG_STALE_EPOCH in kinds(check(SHAPE, t))


def test_stale_epoch_rules():
    # a consumer that still waits for an epoch older than one already stored on the tile
    t = good_trace()
    t.append(ev(FLAG_POLL, 1, 1, tile=0, row=0, word=word(E, 2), epoch=E - 1, accepted=0, round_=2))
    f = check(SHAPE, t)
    assert kinds(f) == [FLAG_STALE_EPOCH] and f[0].round == 2


def test_missing_producer_deadlock_and_early_expiry_rules():
    base = good_trace()
    # nobody ever stores the word the consumer waits for
    t = [e for e in base if e.kind not in (FLAG_STORE, ROW_READ)]
    t[-1:] = [ev(WAIT_EXPIRED, 1, 1, tile=0, row=0, epoch=E), t[-1]]
    t = [e for e in t if not (e.kind == FLAG_POLL and e.accepted)]
    assert kinds(check(SHAPE, t)) == [FLAG_NO_PRODUCER]
    # the word is stored, but only after the wait gave up, by a kernel queued behind the waiting one
    t = [ev(LAUNCH, agent=1, queue=0, part=0, epoch=E), ev(LAUNCH, agent=0, queue=0, part=1, epoch=E),
         ev(FLAG_POLL, 1, 0, tile=0, row=0, word=0, epoch=E), ev(WAIT_EXPIRED, 1, 0, tile=0, row=0, epoch=E),
         ev(ROW_WRITE, 0, tile=0, row=0, part=0, epoch=E), ev(ROW_WRITE, 0, tile=0, row=1, part=0, epoch=E),
         ev(FLAG_STORE, 0, tile=0, word=word(E, 2), epoch=E)]
    assert kinds(check(SHAPE, t)) == [DEADLOCK]
    # the same on separate queues: the producer was free to run, the bound was simply too short
    t[0] = ev(LAUNCH, agent=1, queue=1, part=0, epoch=E)
    t[1] = ev(LAUNCH, agent=0, queue=0, part=0, epoch=E)
    assert kinds(check(SHAPE, t)) == [WAIT_EXPIRED_EARLY]


def test_publisher_side_rules():
    t = good_trace()
    t.insert(9, ev(FLAG_STORE, 0, tile=0, word=word(E, 2), epoch=E))
    assert kinds(check(SHAPE, t)) == [DOUBLE_PUBLISH]
    t = good_trace()
    store = t.pop(8)
    t.insert(4, store)                     # before row 1 is written
    assert kinds(check(SHAPE, t)) == [PUBLISH_BEFORE_LANDED]
    t = good_trace()
    t[8] = ev(FLAG_STORE, 0, tile=0, word=word(E, 1), epoch=E)
    t[9] = ev(FLAG_POLL, 1, 1, tile=0, row=0, word=word(E, 1), epoch=E, accepted=1)
    assert kinds(check(SHAPE, t)) == [WRONG_WORD]
    t = [e for e in good_trace() if e.kind != COUNTER_RESET]
    f = check(SHAPE, t)
    assert kinds(f) == [COUNTER_NOT_ZERO] and f[0].tile == 0
    assert lib().TileXREpTraceFindingName(READ_BEFORE_WRITE) == b"READ_BEFORE_WRITE"
    assert lib().TileXREpTraceFindingName(DEADLOCK) == b"DEADLOCK"


def consumer_trace():
    """The good trace with the consumer's token bookkeeping: one token (0) made of the tile's two rows, claimed, found
    pending at the first look, seen ready by a scan, read and summed."""
    t = good_trace()
    t.insert(4, ev(TOKEN_CLAIM, 1, 1, part=4, word=0, epoch=E))                  # takes tokens [0, 4): only token 0 exists
    t.insert(-1, ev(TOKEN_REDUCED, 1, 1, row=0, epoch=E))
    return t


def test_consumer_side_rules():
    shape = Shape(2, 2, 2, 1, 1)
    assert check(shape, consumer_trace()) == []
    # the token is summed from a row that was read before its tile was published: the sum is the finding, on top of the read's own
    t = consumer_trace()
    store = next(i for i, e in enumerate(t) if e.kind == FLAG_STORE)
    first_read = next(i for i, e in enumerate(t) if e.kind == ROW_READ)
    t.insert(store, t.pop(first_read))
    f = check(shape, t)
    assert TOKEN_REDUCED_WHILE_PENDING in kinds(f)
    assert [(x.row, x.tile) for x in f if x.kind == TOKEN_REDUCED_WHILE_PENDING] == [(0, 0)]
    # two claims that overlap
    t = consumer_trace()
    t.insert(6, ev(TOKEN_CLAIM, 2, 1, part=2, word=0, epoch=E))
    assert kinds(check(shape, t)) == [TOKEN_CLAIMED_TWICE]
    # a token finished twice (summed, and given a row of zeros by somebody else)
    t = consumer_trace()
    t.insert(-1, ev(TOKEN_ZEROED, 2, 1, row=0, epoch=E))
    assert kinds(check(shape, t)) == [TOKEN_CLAIMED_TWICE]
    # claimed but never finished; and never claimed at all
    t = [e for e in consumer_trace() if e.kind != TOKEN_REDUCED]
    f = check(shape, t)
    assert kinds(f) == [TOKEN_NEVER_CLAIMED] and f[0].row == 0
    t = [e for e in consumer_trace() if e.kind != TOKEN_CLAIM]
    assert kinds(check(shape, t)) == [TOKEN_NEVER_CLAIMED]
    # a second round has to claim and finish its tokens again
    t = consumer_trace() + [ev(ROUND_END, agent=-1, epoch=E + 1, round_=2)]
    f = check(shape, t)
    assert kinds(f) == [TOKEN_NEVER_CLAIMED] and f[0].round == 2
    # a launch whose first claim does not find the counter at zero (the launch before did not leave it so)
    t = consumer_trace()
    t[4] = ev(TOKEN_CLAIM, 1, 1, part=4, word=1, epoch=E)
    assert CLAIM_WORD_NOT_RESET in kinds(check(shape, t))
    # without a token count the claim rules are off
    assert check(SHAPE, [e for e in consumer_trace() if e.kind != TOKEN_CLAIM]) == []
    assert lib().TileXREpTraceFindingName(TOKEN_REDUCED_WHILE_PENDING) == b"TOKEN_REDUCED_WHILE_PENDING"


# ---------------------------------------------------------------------------------------------------------------
# (2) + (3) the model
# ---------------------------------------------------------------------------------------------------------------
def run(total, max_rows, tile_rows, parts, top_k=4, producers=4, consumers=3, rounds=2, scheduler=RANDOM, inject=0,
        budget=10_000, seed=1):
    tokens = (total + top_k - 1) // top_k
    c = Case(Shape(total, max_rows, tile_rows, parts, tokens), top_k, producers, consumers, rounds, scheduler, inject, budget, seed)
    cap = 400_000
    events = (Event * cap)()
    n, wrong = C.c_int32(), C.c_int32()
    assert lib().TileXREpTraceRun(C.byref(c), events, cap, C.byref(n), C.byref(wrong)) == 0, n.value
    out = (Finding * 512)()
    found = lib().TileXREpTraceCheck(C.byref(c.shape), events, n.value, out, 512)
    assert found >= 0
    return [events[i] for i in range(n.value)], [out[i] for i in range(min(found, 512))], wrong.value


@pytest.mark.parametrize("shape", [(96, 128, 1, 1), (96, 128, 8, 1), (100, 128, 16, 2), (100, 128, 17, 2),
                                   (130, 160, 64, 4), (257, 300, 100, 2), (64, 64, 1024, 4), (5, 64, 64, 2)])
@pytest.mark.parametrize("scheduler", [SERIAL, ROUND_ROBIN, RANDOM, CONSUMER_EAGER])
def test_clean_runs_have_no_findings(shape, scheduler):
    for seed in (1, 2):
        events, findings, wrong = run(*shape, scheduler=scheduler, seed=seed, rounds=3)
        assert [lib().TileXREpTraceFindingName(f.kind) for f in findings] == []
        assert wrong == 0
        total, _, tile_rows, parts = shape
        tiles = (total + tile_rows - 1) // tile_rows
        stores = [e for e in events if e.kind == FLAG_STORE]
        assert len(stores) == 3 * tiles                                   # once per tile and round
        assert sum(e.kind == ROW_READ for e in events) == 3 * total       # every row consumed, every round
        assert sum(e.kind == ROW_WRITE for e in events) == 3 * total * parts


@pytest.mark.parametrize("scheduler", [ROUND_ROBIN, RANDOM, CONSUMER_EAGER])
def test_consumers_claim_hold_scan_and_reduce_as_the_kernels_do(scheduler):
    """What the waiting combine's control flow promises, read off the trace of a clean run: every token is claimed once
    and summed once, a consumer never holds more than four unfinished tokens, a sleep only follows a scan that found
    nothing ready, and rows are only read by a consumer that has seen their tile published."""
    total, top_k, consumers, rounds = 130, 4, 3, 2
    tokens = (total + top_k - 1) // top_k
    events, findings, wrong = run(total, 160, 16, 2, top_k=top_k, consumers=consumers, rounds=rounds, scheduler=scheduler, seed=9)
    assert findings == [] and wrong == 0
    for rnd in range(1, rounds + 1):
        ev_r = [e for e in events if e.round == rnd]
        claimed = sorted(t for e in ev_r if e.kind == TOKEN_CLAIM for t in range(e.word, e.word + e.part) if t < tokens)
        assert claimed == list(range(tokens))
        assert sorted(e.row for e in ev_r if e.kind == TOKEN_REDUCED) == list(range(tokens))
        assert not any(e.kind in (TOKEN_ZEROED, WAIT_EXPIRED) for e in ev_r)
        for agent in {e.agent for e in ev_r if e.kind == TOKEN_CLAIM}:
            held = 0
            polls_since_progress = 0
            for e in (x for x in ev_r if x.agent == agent):
                if e.kind == TOKEN_CLAIM:
                    held += sum(1 for t in range(e.word, e.word + e.part) if t < tokens)
                    assert held <= 4
                elif e.kind == TOKEN_REDUCED:
                    held -= 1
                    polls_since_progress = 0
                elif e.kind == FLAG_POLL:
                    polls_since_progress += 1
                elif e.kind == SLEEP:
                    assert polls_since_progress > 0 and held > 0      # it looked, found nothing, and still owes tokens
            assert held == 0
        leaves = [e for e in ev_r if e.kind == CONSUMER_LEAVE]
        assert sorted(e.word for e in leaves) == list(range(consumers))           # everybody leaves once
        resets = [e for e in ev_r if e.kind == CLAIM_RESET]
        assert sorted(e.counter for e in resets) == [0, 1] and all(e.word == 0 for e in resets)
        assert all(e.agent == max(leaves, key=lambda x: x.id).agent and e.id > max(x.id for x in leaves) for e in resets)
        assert not any(e.kind == TOKEN_CLAIM and e.id > min(x.id for x in resets) for e in ev_r)
    if scheduler == CONSUMER_EAGER:
        assert any(e.kind == SLEEP for e in events)       # consumers that run ahead of their producers do back off


def test_tokens_of_a_tile_that_is_never_published_get_zeros_not_partial_sums():
    events, findings, wrong = run(100, 128, 8, 2, scheduler=RANDOM, inject=INJECT_MISSING_PRODUCER, budget=40, rounds=1, seed=5)
    assert wrong == 0 and FLAG_NO_PRODUCER in kinds(findings)
    zeroed = {e.row for e in events if e.kind == TOKEN_ZEROED}
    assert zeroed
    stored = {e.tile for e in events if e.kind == FLAG_STORE}
    # a zeroed token contributes no row read, and no token was summed from a row of the tile that never came
    for agent in {e.agent for e in events if e.kind == TOKEN_ZEROED}:
        reads = 0
        for e in (x for x in events if x.agent == agent):
            if e.kind == ROW_READ:
                reads += 1
                assert e.tile in stored
            elif e.kind == TOKEN_REDUCED:
                assert reads > 0
                reads = 0
            elif e.kind == TOKEN_ZEROED:
                assert reads == 0
    assert TOKEN_REDUCED_WHILE_PENDING not in kinds(findings) and TOKEN_NEVER_CLAIMED not in kinds(findings)


def test_trace_covers_the_two_level_counters():
    # tiles wider than 16 rows count groups first: both levels show up as counters of the trace
    events, findings, _ = run(130, 160, 64, 4, rounds=1)
    assert findings == []
    max_tiles = (160 + 63) // 64
    counters = {e.counter for e in events if e.kind == COUNTER_ADD}
    assert any(c < max_tiles for c in counters) and any(c >= max_tiles for c in counters)


@pytest.mark.parametrize("inject,scheduler,expect,wrong_tokens", [
    (INJECT_READ_WITHOUT_WAIT, CONSUMER_EAGER, {READ_WITHOUT_WAIT, READ_BEFORE_WRITE}, True),
    (INJECT_READ_WITHOUT_WAIT, SERIAL, {READ_WITHOUT_WAIT}, False),      # the race is there even when nothing goes wrong
    (INJECT_ACCEPT_ANY_EPOCH, CONSUMER_EAGER, {FLAG_STALE_EPOCH, READ_BEFORE_WRITE}, True),
    (INJECT_MISSING_PRODUCER, RANDOM, {FLAG_NO_PRODUCER, COUNTER_NOT_ZERO}, False),
    (INJECT_DOUBLE_REPORT, RANDOM, None, None),
    (INJECT_REPORT_BEFORE_WRITE, RANDOM, {PUBLISH_BEFORE_LANDED}, None),
    (INJECT_CONSUMER_ENQUEUED_FIRST, RANDOM, {DEADLOCK}, False),
    (INJECT_OLD_EPOCH_CONSUMER, SERIAL, {FLAG_STALE_EPOCH}, None),          # polls meet the newer words
    (INJECT_OLD_EPOCH_CONSUMER, CONSUMER_EAGER, {FLAG_NO_PRODUCER}, None),  # the first dispatch + combine pair waits for an epoch nobody stores
    # the consumer's own logic (ep_token_claim.h runs in the model; the mistakes are planted in its operations)
    (INJECT_TRUST_WITHOUT_SCAN, CONSUMER_EAGER, {TOKEN_REDUCED_WHILE_PENDING, READ_BEFORE_WRITE, READ_WITHOUT_WAIT}, True),
    (INJECT_CLAIM_NOT_ATOMIC, ROUND_ROBIN, {TOKEN_CLAIMED_TWICE}, None),
    (INJECT_CLAIM_SKIPS, RANDOM, {TOKEN_NEVER_CLAIMED}, False),
    (INJECT_IMPATIENT_CONSUMER, CONSUMER_EAGER, {WAIT_EXPIRED_EARLY}, False),
    (INJECT_NO_CLAIM_RESET, RANDOM, {CLAIM_WORD_NOT_RESET, TOKEN_NEVER_CLAIMED}, False),   # the second launch claims from where the first stopped
])
def test_each_planted_mistake_is_reported(inject, scheduler, expect, wrong_tokens):
    events, findings, wrong = run(100, 128, 8, 2, scheduler=scheduler, inject=inject, budget=60, rounds=2, seed=5)
    got = set(kinds(findings))
    if inject == INJECT_DOUBLE_REPORT:
        # the tile's counter overshoots: depending on the order the tile is published early, twice or never
        assert got & {PUBLISH_BEFORE_LANDED, DOUBLE_PUBLISH, COUNTER_NOT_ZERO, FLAG_NO_PRODUCER}
        return
    assert expect <= got, [lib().TileXREpTraceFindingName(k) for k in got]
    if wrong_tokens is True:
        assert wrong > 0          # the mistake is not only a rule violation: consumers really saw old contents
    elif wrong_tokens is False:
        assert wrong == 0
    if inject == INJECT_CONSUMER_ENQUEUED_FIRST:
        # every consumer finished (by expiry) before the first producer step ran: the model's queue really blocks
        first_write = min(e.id for e in events if e.kind == ROW_WRITE and e.round == 1)
        assert all(e.id < first_write for e in events if e.kind == WAIT_EXPIRED and e.round == 1)
        assert not any(e.kind == ROW_READ for e in events)


def test_bad_cases_are_rejected():
    c = Case(Shape(10, 5, 4, 1, 0), 2, 1, 1, 1, 0, 0, 10, 1)          # maxRows < totalRows
    n = C.c_int32()
    assert lib().TileXREpTraceRun(C.byref(c), None, 0, C.byref(n), None) == -1
    c = Case(Shape(10, 16, 4, 1, 5), 2, 1, 1, 1, 0, 0, 10, 1)
    assert lib().TileXREpTraceRun(C.byref(c), None, 0, C.byref(n), None) == -2 and n.value > 0     # trace does not fit

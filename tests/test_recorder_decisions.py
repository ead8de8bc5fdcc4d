"""Which steps of prompt portions are recorded, and when a recording goes (gesso_amd/engine/planned.py: StepRecorder),
on stand-ins for the engine and for the recording itself: no GPU."""
from types import SimpleNamespace

import pytest

from gesso_amd.engine import planned
from gesso_amd.engine.batch import StepEntry
from gesso_amd.errors import InvalidPlan


class Recording:
    """Stands for RecordedStep: remembers what it was made for; ``refuse`` makes the recording fail as a part would."""

    made = []
    refuse = set()

    def __init__(self, engine, T, seq_cap, kv_cap, key, single=False):
        self.T, self.seq_cap, self.kv_cap, self.key, self.single = T, seq_cap, kv_cap, key, single

    def record(self):
        if self.T in self.refuse:
            raise InvalidPlan(f"a part refuses steps of {self.T} tokens")
        Recording.made.append((self.T, self.kv_cap))


@pytest.fixture
def recorder(monkeypatch):
    Recording.made, Recording.refuse = [], set()
    monkeypatch.setattr(planned, "RecordedStep", Recording)
    held = {}
    manager = SimpleNamespace(get=lambda rid: SimpleNamespace(length=held.get(rid, 0)))
    # the model records steps whose longest portion has 64 tokens or more, and walks sequences of 4,096 keys another way
    # (steps of single tokens it walks in a way of their own)
    model = SimpleNamespace(replay_key=lambda lens, longest: ("single",) if max(lens) == 1 else
                            (2 if longest < 4096 else 1,) if max(lens) >= 64 else None)
    rec = planned.StepRecorder(SimpleNamespace(manager=manager, model=model, DECODE_MAX_BATCH=64))
    rec.held = held
    return rec


def step(*lens):
    return [StepEntry(i, [0] * n, []) for i, n in enumerate(lens)]


def test_the_fourth_step_of_a_kind_is_recorded_and_serves_from_then_on(recorder):
    for _ in range(recorder.SEEN_BEFORE):
        assert recorder.recording_for(step(1, 1, 98)) is None
    first = recorder.recording_for(step(1, 99))            # the same kind: 100 tokens, however they divide
    assert first is not None and Recording.made == [(100, 4096)]
    assert recorder.recording_for(step(1, 1, 1, 97)) is first and Recording.made == [(100, 4096)]


def test_steps_that_are_never_recorded(recorder):
    for _ in range(6):
        assert recorder.recording_for(step(1, 1, 1)) is None                       # decoded tokens only
        assert recorder.recording_for(step(1, 30, 40)) is None                     # the model says no (short portions)
        assert recorder.recording_for(step(*([1] * recorder.MAX_SEQ_CAP + [80]))) is None  # more sequences than a recording holds
    assert Recording.made == [] and recorder.seen == {}


def test_single_tokens_are_recorded_when_there_are_more_than_the_decode_loop_takes(recorder):
    for _ in range(6):
        assert recorder.recording_for(step(*[1] * 64)) is None           # the recorded decode loop's business
        assert recorder.recording_for(step(*[1] * (recorder.MAX_SINGLE + 1))) is None
    for _ in range(recorder.SEEN_BEFORE):
        assert recorder.recording_for(step(*[1] * 200)) is None
    rec = recorder.recording_for(step(*[1] * 200))
    assert rec.single and rec.T == rec.seq_cap == 200 and rec.key == ("single",)
    # 200 tokens with a portion among them are another kind, with room for the usual number of sequences
    for _ in range(4):
        other = recorder.recording_for(step(*[1] * 30, 170))
    assert not other.single and other.seq_cap == recorder.SEQ_CAP and other.T == 200
    # more sequences than that beside a portion: room for twice as many, a kind of its own
    for _ in range(4):
        more = recorder.recording_for(step(*[1] * 100, 100))
    assert more is not other and more.seq_cap == 128 and more.T == 200


def test_room_for_keys_and_the_walk_make_kinds_of_their_own(recorder):
    for _ in range(4):
        recorder.recording_for(step(128))
    recorder.held[0] = 4000                                  # the sequence has grown: 4,128 keys after the step
    for _ in range(3):
        assert recorder.recording_for(step(128)) is None
    assert recorder.recording_for(step(128)).kv_cap == 8192
    assert Recording.made == [(128, 4096), (128, 8192)]
    assert {k[2] for k in recorder.recordings} == {(2,), (1,)}


def test_a_recording_that_a_part_refuses_is_not_tried_again(recorder):
    Recording.refuse = {100}
    for _ in range(8):
        assert recorder.recording_for(step(100)) is None
    (kind, err), = recorder.refused.items()
    assert kind[0] == 100 and "refuses" in str(err)
    assert recorder.seen[kind] == recorder.SEEN_BEFORE + 1        # counted until the attempt, not after
    for _ in range(4):
        recorder.recording_for(step(200))
    assert Recording.made == [(200, 4096)]                  # and a refusal takes none of the room


def test_when_full_a_kind_waits_until_a_recording_has_lain_idle(recorder):
    recorder.MAX_RECORDINGS, recorder.IDLE_STEPS = 2, 10
    for T in (100, 200):
        for _ in range(4):
            recorder.recording_for(step(T))
    assert Recording.made == [(100, 4096), (200, 4096)]
    for i in range(9):                                       # 200 keeps serving, 100 lies idle, 300 comes again and again
        assert recorder.recording_for(step(200)) is not None
        got = recorder.recording_for(step(300))
        if 2 * (i + 1) + 4 < 10:
            assert got is None, i                            # 100 has not been idle for ten steps yet
    assert Recording.made == [(100, 4096), (200, 4096), (300, 4096)]
    assert sorted(k[0] for k, r in recorder.recordings.items() if r is not None) == [200, 300]
    # the kind that went starts its count again
    assert recorder.recording_for(step(100)) is None


def test_the_tally_of_kinds_starts_over_when_it_is_full(recorder):
    recorder.MAX_SEEN = 5
    for T in range(100, 105):
        recorder.recording_for(step(T))
    assert len(recorder.seen) == 5
    recorder.recording_for(step(105))
    assert list(recorder.seen) == [(105, 4096, (2,), 64)]

"""A CPU model of how the workgroups of the single sweep meet (csrc/fcr.hip, col_fused_kernel, step 3).

The workgroups that share a (batch, head) pair exchange one value per query row and round.  A value and
the number of its round travel as ONE 64-bit word, stored and loaded atomically; readers poll a slot
until it carries the round they are in; there are two sets of slots, used by even and odd rounds; the
slots start at zero and round numbers start at 1; a reader gives up after a bounded number of polls.
The model runs that protocol under random interleavings of the individual loads and stores and checks
what the kernel relies on:

  * every value a workgroup takes from a slot is the value its writer published for that very round,
  * a workgroup is never more than one round ahead of the slowest of its team, which is why two sets of
    slots are enough (and one set is not: the model shows the overwritten slot),
  * nobody waits for ever: with a member that never arrives the others give up after the bound.
"""
import random

import pytest


class Member:
    """One workgroup of a team: publish, then poll every slot of the round's set, then go on."""

    def __init__(self, index, team_size, rounds, sets, poll_limit):
        self.index, self.team_size, self.rounds, self.sets, self.poll_limit = index, team_size, rounds, sets, poll_limit
        self.round = 0          # 0-based; the tag it writes and waits for is round + 1
        self.phase = "publish"
        self.next_slot = 0
        self.polls = 0
        self.taken = []         # (round, writer, value) of every slot it accepted
        self.gave_up = False
        self.done = rounds == 0

    @staticmethod
    def value(writer, rnd):
        return 1000 * rnd + writer

    def step(self, slots):
        """One atomic access to the slots (or one local transition)."""
        if self.done:
            return
        which = self.round % self.sets
        if self.phase == "publish":
            slots[which][self.index] = (self.round + 1, self.value(self.index, self.round))   # one 64-bit store
            self.phase, self.next_slot, self.polls = "poll", 0, 0
            return
        tag, val = slots[which][self.next_slot]                                               # one 64-bit load
        if tag == self.round + 1:
            self.taken.append((self.round, self.next_slot, val))
            self.next_slot += 1
            if self.next_slot == self.team_size:
                self.round += 1
                self.phase = "publish"
                self.done = self.round == self.rounds
        else:
            self.polls += 1
            if self.polls > self.poll_limit:
                self.gave_up = True     # the kernel stores NaN columns, raises the status word and goes on;
                self.done = True        # here the member simply stops


def run(team_size, rounds, sets, seed, poll_limit=10**9, absent=()):
    rng = random.Random(seed)
    slots = [[(0, 0)] * team_size for _ in range(sets)]
    members = [Member(i, team_size, rounds, sets, poll_limit) for i in range(team_size)]
    lead = 0
    steps = 0
    while True:
        live = [m for m in members if not m.done and m.index not in absent]
        if not live:
            break
        # a schedule with long bursts: one member races ahead as far as the protocol lets it
        m = rng.choice(live)
        for _ in range(rng.choice([1, 1, 2, 5, 50])):
            m.step(slots)
            steps += 1
        present = [x.round for x in members if x.index not in absent]
        lead = max(lead, max(present) - min(present))
        assert steps < 10**7, "the model does not terminate"
    return members, lead


@pytest.mark.parametrize("team_size", [1, 2, 3, 8, 16])
def test_every_slot_read_belongs_to_the_readers_round(team_size):
    for seed in range(40):
        members, lead = run(team_size, rounds=7, sets=2, seed=seed)
        assert lead <= 1
        for m in members:
            assert not m.gave_up and m.round == 7
            assert len(m.taken) == 7 * team_size
            for rnd, writer, val in m.taken:
                assert val == Member.value(writer, rnd)


def test_one_set_of_slots_would_not_be_enough():
    """With a single set a member that has finished round r may publish round r + 1 into the slot that a
    slower member has not read yet; the slower one then never sees the tag it waits for."""
    stuck = 0
    for seed in range(40):
        members, _ = run(4, rounds=5, sets=1, seed=seed, poll_limit=2000)
        stuck += any(m.gave_up for m in members)
    assert stuck > 0


def test_a_member_that_never_arrives_ends_the_wait_of_the_others():
    members, _ = run(4, rounds=3, sets=2, seed=1, poll_limit=500, absent={2})
    for m in members:
        if m.index != 2:
            assert m.gave_up and m.round == 0   # nobody got past the first round, and nobody spins for ever

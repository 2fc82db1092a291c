"""The rule by which the weighted race on key halves decides that a row is settled, checked by
brute force on the CPU.

The kernels (csrc/race.h) first race on the upper 32 bits of the 64-bit keys and fall back to full
(key, position) pairs only when the halves "left the row open".  Whether that rule has a hole is a
property of the rule, not of the GPU: this file restates it step by step in Python (same order of
operations as half_race_seed / half_race_offer / half_race_open and the block-per-row variant
with shared bars and the listed merge) and drives it with keys from a tiny alphabet, so that ties
of every kind are the norm.  The claim under test: whenever the rule says "settled", the picks
equal the k smallest (key, position) pairs in order.  The sort network of the kernels is not
stable, so equal halves are ordered at random here.
"""
import random

NONE = 1 << 40  # above every half


def brute(cands, k):
    """cands: (half, low, pos).  The k smallest by full key, then position."""
    return [c[2] for c in sorted(cands, key=lambda c: (c[0], c[1], c[2]))[:k]]


class HalfRace:
    def __init__(self, k, width, rng):
        self.k, self.width, self.rng = k, width, rng
        self.entries = []  # (half, pos), ascending halves, at most k
        self.last = NONE
        self.tie = NONE
        self.seeded = False

    def seed(self, chunk):
        lanes = [(h, p) for h, p in chunk] + [(NONE, -1)] * (self.width - len(chunk))
        self.rng.shuffle(lanes)                 # an unstable sort: equal halves in any order
        lanes.sort(key=lambda e: e[0])
        self.last = lanes[self.k - 1][0]
        cut = lanes[self.k][0] if self.k < self.width else NONE
        self.tie = cut if (self.k < self.width and cut == self.last) else NONE
        self.entries = lanes[:self.k]
        self.seeded = True

    def offer(self, chunk):
        hits = [(h, p) for h, p in chunk if h < self.last]
        if any(h == self.last for h, _ in chunk):
            self.tie = self.last
        for v, p in hits:
            if v >= self.last:
                if v == self.last:
                    self.tie = v
                continue
            at = next((i for i, e in enumerate(self.entries) if v < e[0]), len(self.entries))
            pushed_out = self.last
            self.entries = (self.entries[:at] + [(v, p)] + self.entries[at:])[:self.k]
            self.last = self.entries[self.k - 1][0]
            if self.last == pushed_out:
                self.tie = pushed_out

    def feed(self, chunk):
        if not self.seeded:
            self.seed(chunk)
        else:
            self.offer(chunk)

    def open(self):
        halves = [e[0] for e in self.entries[:self.k]]
        return self.tie == self.last or any(a == b for a, b in zip(halves, halves[1:]))


def group_row(cands, k, width, rng):
    race = HalfRace(k, width, rng)
    for at in range(0, len(cands), width):
        race.feed([(c[0], c[2]) for c in cands[at:at + width]])
    return race.open(), [e[1] for e in race.entries[:k]]


def block_row(cands, k, width, waves, rng):
    """Waves race interleaved stretches of 4 * width positions, drop candidates strictly above
    the lowest bar published so far (possibly a stale, higher value), list what survives the
    final lowest bar, and wave 0 races the list."""
    stretch = 4 * width
    races = [HalfRace(k, width, rng) for _ in range(waves)]
    published = [NONE] * waves
    history = [NONE]  # lowest bars seen so far: a wave may read any earlier one
    n_rounds = (len(cands) + stretch * waves - 1) // (stretch * waves)
    for rnd in range(n_rounds):
        order = list(range(waves))
        rng.shuffle(order)  # the waves of a block run in no particular order
        for w in order:
            begin = (rnd * waves + w) * stretch
            if begin >= len(cands):
                continue
            bar = rng.choice(history[-3:])
            for at in range(begin, min(begin + stretch, len(cands)), width):
                chunk = [(c[0], c[2]) for c in cands[at:at + width]]
                if races[w].seeded:
                    chunk = [(h if h <= bar else NONE, p) for h, p in chunk]
                races[w].feed(chunk)
            if races[w].last < published[w]:
                published[w] = races[w].last
                history.append(min(published))
    ties = [r.tie for r in races]
    bar = min(published)
    listed = [e for r in races for e in r.entries[:k] if e[0] <= bar]
    rng.shuffle(listed)  # the list is filled through an atomic counter
    final = HalfRace(k, width, rng)
    for at in range(0, len(listed), width):
        final.feed(listed[at:at + width])
    is_open = final.open() or any(t == final.last for t in ties)
    return is_open, [e[1] for e in final.entries[:k]]


def _row(rng, n, alphabet):
    return [(rng.randrange(alphabet), rng.randrange(4), p) for p in range(n)]


def test_group_race_on_halves_is_right_whenever_it_says_settled():
    rng = random.Random(1)
    settled = 0
    for trial in range(6000):
        width = rng.choice([4, 8])
        k = rng.randrange(1, width + 1)
        n = rng.randrange(k + 1, 6 * width)
        cands = _row(rng, n, rng.choice([3, 8, 40, 400]))
        is_open, picks = group_row(cands, k, width, rng)
        if not is_open:
            settled += 1
            assert picks == brute(cands, k), (trial, width, k, cands)
    assert settled > 1500  # the rule is not vacuous


def test_block_race_on_halves_is_right_whenever_it_says_settled():
    rng = random.Random(2)
    settled = 0
    for trial in range(3000):
        width = rng.choice([4, 8])
        waves = rng.choice([2, 4])
        k = rng.randrange(1, width + 1)
        n = rng.randrange(4 * width * waves, 16 * width * waves)  # every wave holds at least k
        cands = _row(rng, n, rng.choice([8, 40, 400, 4000]))
        is_open, picks = block_row(cands, k, width, waves, rng)
        if not is_open:
            settled += 1
            assert picks == brute(cands, k), (trial, width, waves, k, cands)
    assert settled > 700


def test_race_on_halves_settles_whenever_the_smallest_halves_are_distinct():
    # no needless repeats: if the k + 1 smallest halves of a row differ from each other, nothing
    # is open, whatever ties there are further up (unusable weights all share one half there)
    rng = random.Random(3)
    unusable = 10 ** 6
    seen = 0
    for trial in range(3000):
        width = 8
        k = rng.randrange(1, 7)
        n = rng.randrange(3 * width, 10 * width)
        cands = [(unusable if rng.random() < 0.5 else rng.randrange(60), rng.randrange(4), p) for p in range(n)]
        smallest = sorted(c[0] for c in cands)[:k + 1]
        if len(set(smallest)) < k + 1:
            continue
        seen += 1
        is_open, picks = group_row(cands, k, width, rng)
        assert not is_open, (trial, k, cands)
        assert picks == brute(cands, k)
        if n >= 4 * width * 2:
            is_open, picks = block_row(cands, k, width, 2, rng)
            assert not is_open, (trial, k, cands)
            assert picks == brute(cands, k)
    assert seen > 300

"""Host-side pieces above ForwardPipe::forward: Go rules, symmetries and input
planes.  The plain-Python restatement in oracle/go_oracle.py is first pinned
against hand-worked positions and closed forms, then the library is compared
with it on random games (no GPU needed: these entry points compute on the host)."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import oracle.go_oracle as G  # noqa: E402
from __graft_entry__ import ensure_built  # noqa: E402

lz = ensure_built()

B, W, E, PASS = G.BLACK, G.WHITE, G.EMPTY, G.PASS


def P(x, y):
    return y * 19 + x


def replay_oracle(moves):
    b = G.Board()
    for m in moves:
        b.play(m)
    return b


def check_same(moves, komi=7.5):
    """Library and restatement agree on everything after `moves`."""
    b = replay_oracle(moves)
    r = lz.board_replay(moves, komi)
    assert list(r["stones"]) == b.sq
    assert list(r["legal"]) == b.legal_mask()
    assert r["ko_point"] == b.ko
    last_is_stone = bool(moves) and moves[-1] != PASS
    assert r["superko"] == (last_is_stone and b.superko())
    assert r["score"] == b.area_score(komi)
    return b, r


# ---- hand-worked positions: these pin the restatement AND the library ------------

def test_empty_board_and_single_stone_scores():
    b, r = check_same([])
    assert r["score"] == -7.5 and r["legal"].all()
    b, r = check_same([P(3, 3)], komi=0.5)
    assert r["score"] == 361 - 0.5          # every empty point reaches black only
    b, r = check_same([P(3, 3), P(15, 15)])
    assert r["score"] == 1 - 1 - 7.5        # empty points reach both colours


def test_corner_capture_and_suicide():
    moves = [P(1, 0), P(0, 0), P(0, 1)]     # black takes the corner stone
    b, r = check_same(moves)
    assert r["stones"][P(0, 0)] == E
    assert r["stones"][P(1, 0)] == B and r["stones"][P(0, 1)] == B
    assert not r["legal"][P(0, 0)]          # white may not jump back in: suicide
    assert r["ko_point"] == -1              # the capturing stone has other liberties
    # black itself may fill its own eye point (not suicide: the string keeps liberties)
    b, r = check_same(moves + [PASS])
    assert r["legal"][P(0, 0)]


def test_multi_stone_suicide_and_capture_beats_suicide():
    # white string (0,0),(1,0) with last liberty (2,0) after black surrounds it
    moves = [P(0, 1), P(0, 0), P(1, 1), P(1, 0), P(10, 10), PASS]
    # white: (0,0),(1,0); black: (0,1),(1,1),(10,10); liberty of white string: (2,0)
    b, r = check_same(moves)
    assert r["legal"][P(2, 0)]              # black captures two stones there
    b, r = check_same(moves + [P(2, 0)])
    assert r["stones"][P(0, 0)] == E and r["stones"][P(1, 0)] == E
    assert r["ko_point"] == -1              # two stones taken: never a ko
    # white to move: (0,0) is now empty with neighbours (1,0) empty -> legal
    assert r["legal"][P(0, 0)]


KO_SETUP = [P(2, 3), P(5, 3), P(3, 2), P(4, 2), P(3, 4), P(4, 4), P(10, 10), P(3, 3)]


def test_simple_ko():
    b, r = check_same(KO_SETUP)
    assert r["legal"][P(4, 3)]              # black may capture the stone at (3,3)
    b, r = check_same(KO_SETUP + [P(4, 3)])
    assert r["stones"][P(3, 3)] == E and r["stones"][P(4, 3)] == B
    assert r["ko_point"] == P(3, 3)
    assert not r["legal"][P(3, 3)]          # white may not retake at once
    b, r = check_same(KO_SETUP + [P(4, 3), P(10, 11), P(10, 12)])
    assert r["ko_point"] == -1 and r["legal"][P(3, 3)]
    b, r = check_same(KO_SETUP + [P(4, 3), P(10, 11), P(10, 12), P(3, 3)])
    assert r["stones"][P(4, 3)] == E and r["ko_point"] == P(4, 3)
    assert not r["superko"]                 # the two exchanged stones make it new


def test_positional_superko_after_passes():
    # black takes the ko, both pass, white retakes: the stones repeat the
    # position before black's capture although the simple-ko point was cleared.
    moves = KO_SETUP + [P(4, 3), PASS, PASS]
    b, r = check_same(moves)
    assert r["ko_point"] == -1 and r["legal"][P(3, 3)]
    b, r = check_same(moves + [P(3, 3)])
    assert r["superko"]


def test_snapback():
    # white (1,0) is taken by black (2,0)?  Build: black (0,1),(1,1),(2,1)... a
    # one-stone capture that is NOT a ko because the capturing stone joins a string.
    moves = [P(0, 1), P(1, 0), P(1, 1), P(12, 12), P(2, 0)]
    # white (1,0): neighbours (0,0) empty -> still one liberty
    b, r = check_same(moves)
    assert r["stones"][P(1, 0)] == W
    b, r = check_same(moves + [P(12, 13), P(0, 0)])   # black fills the last liberty
    assert r["stones"][P(1, 0)] == E
    assert r["ko_point"] == -1              # (0,0) touches a friendly stone: no eye play


def test_illegal_move_is_rejected():
    with pytest.raises(ValueError):
        lz.board_replay([P(3, 3), P(3, 3)])
    with pytest.raises(ValueError):
        lz.board_replay(KO_SETUP + [P(4, 3), P(3, 3)])
    with pytest.raises(ValueError):
        lz.board_replay([400])


# ---- library against the restatement on random games ---------------------------

@pytest.mark.parametrize("seed,plies", [(1, 250), (2, 250), (3, 420), (4, 420)])
def test_random_games_agree(seed, plies):
    rng = np.random.default_rng(seed)
    b = G.Board()
    moves = []
    captures = kos = 0
    for ply in range(plies):
        mask = b.legal_mask()
        r = lz.board_replay(moves)
        assert list(r["legal"]) == mask, "ply %d" % ply
        assert list(r["stones"]) == b.sq, "ply %d" % ply
        assert r["ko_point"] == b.ko
        assert r["score"] == b.area_score(7.5)
        cand = [v for v in range(361) if mask[v]]
        # no superko filter here: replay reports it, the search avoids such moves
        mv = int(rng.choice(cand)) if cand and rng.random() > 0.02 else PASS
        before = sum(1 for s in b.sq if s != E)
        b.play(mv)
        moves.append(mv)
        after = sum(1 for s in b.sq if s != E)
        captures += int(mv != PASS and after <= before)
        kos += int(b.ko >= 0)
        rr = lz.board_replay(moves)
        assert rr["superko"] == (mv != PASS and b.superko())
    assert captures > 0          # the games did exercise captures


# ---- the reference's own board code, compiled from its sources ------------------

def test_rules_against_the_reference_board():
    """oracle/_ref/ref_board drives the reference's FullBoard (built by oracle/Makefile,
    target ref, from the reference tree where that is present).  Every prefix of random
    games and the hand-worked sequences above give the same stones, legal moves, ko
    point, repetition flag and score in the reference, in the restatement and in the
    library; an illegal move is refused by all three at the same index."""
    if G.build_ref_board() is None:
        pytest.skip("the reference tree is not present and oracle/_ref/ref_board is not built")
    games = [KO_SETUP + [P(4, 3), PASS, PASS, P(3, 3)],
             [P(1, 0), P(0, 0), P(0, 1), PASS],
             [P(0, 1), P(0, 0), P(1, 1), P(1, 0), P(10, 10), PASS, P(2, 0)]]
    for seed in (11, 12, 13):
        rng = np.random.default_rng(seed)
        b = G.Board()
        moves = []
        for ply in range(330):
            mask = b.legal_mask()
            cand = [v for v in range(361) if mask[v]]
            mv = int(rng.choice(cand)) if cand and rng.random() > 0.03 else PASS
            b.play(mv)
            moves.append(mv)
        games.append(moves)
    prefixes, owner = [], []
    for g in games:
        for n in range(len(g) + 1):
            prefixes.append(g[:n])
            owner.append(g)
    ref = G.ref_board_replay(prefixes)
    assert len(ref) == len(prefixes)
    for moves, r in zip(prefixes, ref):
        assert "illegal" not in r, (len(moves), r)
        b = replay_oracle(moves)
        assert r["stones"] == b.sq
        assert r["legal"] == b.legal_mask()
        assert r["ko"] == b.ko
        assert r["score"] == b.area_score(7.5)
        last_is_stone = bool(moves) and moves[-1] != PASS
        assert r["superko"] == (last_is_stone and b.superko())
    # the library on the longest prefixes (every ply was already compared with the
    # restatement in the tests above)
    for g in games:
        r = G.ref_board_replay([g])[0]
        l = lz.board_replay(g)
        assert list(l["stones"]) == r["stones"] and list(l["legal"]) == r["legal"]
        assert l["ko_point"] == r["ko"] and l["superko"] == r["superko"] and l["score"] == r["score"]
    # illegal moves: same verdict, same index
    bad = [[P(3, 3), P(3, 3)], KO_SETUP + [P(4, 3), P(3, 3)], [P(1, 0), P(0, 0), P(0, 1), P(0, 0)]]
    for g, r in zip(bad, G.ref_board_replay(bad)):
        assert r == {"illegal": len(g) - 1}
        with pytest.raises(ValueError):
            lz.board_replay(g)


def test_cache_against_the_reference_cache(tmp_path):
    """The same script of inserts and lookups (more distinct keys than capacity, repeated
    keys, re-inserts of present keys) through the reference's NNCache and through the
    driver's EvalCache: every lookup has the same outcome, i.e. the same entries are
    evicted in the same order."""
    import shutil
    import subprocess
    if G.build_ref_board() is None or not os.path.exists(G.REF_CACHE):
        pytest.skip("the reference tree is not present and oracle/_ref/ref_cache is not built")
    if shutil.which("g++") is None:
        pytest.skip("needs g++")
    csrc = os.path.join(ROOT, "leela-zero_amd", "csrc")
    exe = str(tmp_path / "cache_trace")
    cmd = ["g++", "-std=c++17", "-O1", "-pthread", "-I", os.path.join(ROOT, "include"), "-I", csrc,
           os.path.join(ROOT, "tests", "cpp", "cache_trace.cpp")] + \
          [os.path.join(csrc, f) for f in ("search.cpp", "goboard.cpp", "hip_scheduler.cpp")] + \
          ["-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    rng = np.random.default_rng(3)
    for capacity in (1, 7, 64):
        lines = [str(capacity)]
        for step in range(4000):
            key = int(rng.integers(0, 3 * capacity + 2))
            if rng.random() < 0.45:
                lines.append("i %d %.3f" % (key, step % 1000 / 1000.0))
            else:
                lines.append("l %d" % key)
        script = "\n".join(lines) + "\n"
        want = G.ref_cache_trace(script)
        env = dict(os.environ)
        env.pop("LD_PRELOAD", None)
        got = subprocess.run([exe], input=script, capture_output=True, text=True, env=env,
                             timeout=120).stdout.splitlines()
        assert len(want) > 1000 and got == want
        assert any(l != "0" for l in want) and any(l == "0" for l in want)


# ---- symmetries ------------------------------------------------------------------

def test_symmetry_closed_forms():
    for idx in range(361):
        x, y = idx % 19, idx // 19
        assert lz.symmetry_index(0, idx) == idx
        assert lz.symmetry_index(1, idx) == P(x, 18 - y)
        assert lz.symmetry_index(2, idx) == P(18 - x, y)
        assert lz.symmetry_index(3, idx) == P(18 - x, 18 - y)
        assert lz.symmetry_index(4, idx) == P(y, x)
    perms = [tuple(lz.symmetry_index(s, i) for i in range(361)) for s in range(8)]
    assert len(set(perms)) == 8
    for p in perms:
        assert sorted(p) == list(range(361))
    # the eight maps form a group: closed under composition
    for a in perms:
        for b in perms:
            assert tuple(a[b[i]] for i in range(361)) in perms
    for s in range(8):
        assert list(perms[s]) == [G.symmetry_index(s, i) for i in range(361)]
    with pytest.raises(ValueError):
        lz.symmetry_index(8, 0)
    with pytest.raises(ValueError):
        lz.symmetry_index(0, 361)


# ---- input planes ----------------------------------------------------------------

def test_features_hand_cases():
    empty = np.full((1, 361), E, np.uint8)
    f = lz.gather_features(empty, B)
    assert f[16].min() == 1.0 and np.count_nonzero(f[:16]) == 0 and np.count_nonzero(f[17]) == 0
    f = lz.gather_features(empty, W)
    assert f[17].min() == 1.0 and np.count_nonzero(f[:17]) == 0
    # one black stone, white to move: it is an opponent stone of the newest board
    b = empty.copy()
    b[0, P(2, 5)] = B
    f = lz.gather_features(b, W)
    assert f[8, P(2, 5)] == 1.0 and np.count_nonzero(f[:16]) == 1
    f = lz.gather_features(b, B)
    assert f[0, P(2, 5)] == 1.0 and np.count_nonzero(f[:16]) == 1
    # mirrored in x: the plane shows the stone at (16,5)
    f = lz.gather_features(b, B, symmetry=2)
    assert f[0, P(16, 5)] == 1.0 and np.count_nonzero(f[:16]) == 1
    # transposed
    f = lz.gather_features(b, B, symmetry=4)
    assert f[0, P(5, 2)] == 1.0
    # history slot: two boards, the older one holds a white stone too
    hist = np.full((2, 361), E, np.uint8)
    hist[0, P(2, 5)] = B
    hist[1, P(2, 5)] = B
    hist[1, P(7, 7)] = W
    f = lz.gather_features(hist, B)
    assert f[0, P(2, 5)] == 1.0 and f[1, P(2, 5)] == 1.0 and f[9, P(7, 7)] == 1.0
    assert np.count_nonzero(f[:16]) == 3


@pytest.mark.parametrize("seed", [0, 1])
def test_features_agree_with_restatement(seed):
    rng = np.random.default_rng(seed)
    for n in (1, 3, 8):
        boards = rng.choice([B, W, E], size=(n, 361), p=[0.25, 0.25, 0.5]).astype(np.uint8)
        for to_move in (B, W):
            for sym in range(8):
                got = lz.gather_features(boards, to_move, sym)
                want = np.array(G.gather_features([list(b) for b in boards], to_move, sym),
                                dtype=np.float32)
                assert np.array_equal(got, want)


def test_features_argument_checks():
    e = np.full((9, 361), E, np.uint8)
    with pytest.raises(ValueError):
        lz.gather_features(e, B)          # more than 8 boards
    with pytest.raises(ValueError):
        lz.gather_features(e[:1], 2)
    with pytest.raises(ValueError):
        lz.gather_features(e[:1], B, symmetry=8)

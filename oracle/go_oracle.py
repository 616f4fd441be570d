"""TEST INFRASTRUCTURE ONLY -- not part of the product path.

Plain-Python restatement of what the search driver asks of the reference's
board and of `Network`'s input encoding, written for clarity, not speed:

* Go rules on 19x19: captures, suicide, simple ko, positional superko, area
  score (reference src/FastBoard.cpp:168-195 is_suicide, :260-296
  calc_reach_color / area_score; src/FullBoard.cpp:150-210 update_board with
  the ko rule at :159 and :203-207; src/FastState.cpp:76-83 is_move_legal,
  :89-110 play_move; src/KoState.cpp:51-58 superko).
* Symmetries and input planes (reference src/Network.cpp:968-993
  get_symmetry, :518-531 symmetry_nn_idx_table, :913-966 gather_features).

Pinned by tests/test_search_host.py against hand-worked positions (corner
capture, ko, a one-stone capture that is no ko, suicide, a repetition through
passes, small scored boards), against closed forms of the symmetry group, and,
where the reference tree is at hand, against the reference's own board code
compiled from its sources (oracle/Makefile target `ref`, oracle/_ref/ref_board)
on every ply of random games.
"""
import os
import subprocess

N = 19
NPTS = N * N
PASS = NPTS
BLACK, WHITE, EMPTY = 0, 1, 2


def neighbours(v):
    x, y = v % N, v // N
    out = []
    if x > 0:
        out.append(v - 1)
    if x < N - 1:
        out.append(v + 1)
    if y > 0:
        out.append(v - N)
    if y < N - 1:
        out.append(v + N)
    return out


class Board:
    def __init__(self):
        self.sq = [EMPTY] * NPTS
        self.to_move = BLACK
        self.ko = -1
        self.passes = 0
        self.history = [tuple(self.sq)]   # every position so far, oldest first

    def group(self, v):
        """(stones, liberties) of the string at v."""
        color = self.sq[v]
        stones, libs, todo = {v}, set(), [v]
        while todo:
            p = todo.pop()
            for n in neighbours(p):
                if self.sq[n] == EMPTY:
                    libs.add(n)
                elif self.sq[n] == color and n not in stones:
                    stones.add(n)
                    todo.append(n)
        return stones, libs

    def is_suicide(self, color, v):
        """True when placing `color` at the empty point v leaves its string
        without liberties and captures nothing."""
        self.sq[v] = color
        try:
            for n in neighbours(v):
                if self.sq[n] == (color ^ 1) and not self.group(n)[1]:
                    return False
            return not self.group(v)[1]
        finally:
            self.sq[v] = EMPTY

    def is_legal(self, color, v):
        if v == PASS:
            return True
        return self.sq[v] == EMPTY and v != self.ko and not self.is_suicide(color, v)

    def legal_mask(self):
        return [self.is_legal(self.to_move, v) for v in range(NPTS + 1)]

    def play(self, v):
        color = self.to_move
        if v == PASS:
            self.passes += 1
            self.ko = -1
        else:
            assert self.is_legal(color, v)
            self.passes = 0
            # "eye play": every neighbour is an enemy stone (or the edge)
            eyeplay = all(self.sq[n] == (color ^ 1) for n in neighbours(v))
            self.sq[v] = color
            captured = []
            for n in neighbours(v):
                if self.sq[n] == (color ^ 1):
                    stones, libs = self.group(n)
                    if not libs:
                        for s in stones:
                            self.sq[s] = EMPTY
                        captured += list(stones)
            self.ko = captured[0] if (len(captured) == 1 and eyeplay) else -1
        self.to_move = color ^ 1
        self.history.append(tuple(self.sq))

    def superko(self):
        """The present stones repeat an earlier position."""
        return self.history[-1] in self.history[:-1]

    def area_score(self, komi):
        reach = []
        for color in (BLACK, WHITE):
            seen = {v for v in range(NPTS) if self.sq[v] == color}
            todo = list(seen)
            while todo:
                p = todo.pop()
                for n in neighbours(p):
                    if self.sq[n] == EMPTY and n not in seen:
                        seen.add(n)
                        todo.append(n)
            reach.append(len(seen))
        return reach[BLACK] - reach[WHITE] - komi


def get_symmetry(x, y, symmetry):
    if symmetry & 4:
        x, y = y, x
    if symmetry & 2:
        x = N - 1 - x
    if symmetry & 1:
        y = N - 1 - y
    return x, y


def symmetry_index(symmetry, idx):
    x, y = get_symmetry(idx % N, idx // N, symmetry)
    return y * N + x


def gather_features(boards, to_move, symmetry):
    """boards: newest first, each a sequence of 361 BLACK/WHITE/EMPTY ->
    list of 18 planes of 361 floats."""
    planes = [[0.0] * NPTS for _ in range(18)]
    for h, b in enumerate(boards[:8]):
        for idx in range(NPTS):
            c = b[symmetry_index(symmetry, idx)]
            if c == EMPTY:
                continue
            plane = h if c == to_move else 8 + h
            planes[plane][idx] = 1.0
    planes[16 if to_move == BLACK else 17] = [1.0] * NPTS
    return planes


# ---- the reference's own board code, when it has been built (oracle/Makefile, target ref)

HERE = os.path.dirname(os.path.abspath(__file__))
REF_BOARD = os.path.join(HERE, "_ref", "ref_board")
REF_CACHE = os.path.join(HERE, "_ref", "ref_cache")
REF_SRC = "/root/reference/src"


def build_ref_board():
    """Builds oracle/_ref/ref_board from the reference tree if that tree is present.
    Returns the path, or None when neither the binary nor the tree exists."""
    if os.path.exists(os.path.join(REF_SRC, "FullBoard.cpp")):
        r = subprocess.run(["make", "-C", HERE, "ref"], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("building the reference board failed:\n" + r.stderr)
    return REF_BOARD if os.path.exists(REF_BOARD) else None


def ref_cache_trace(script):
    """Feeds a script (capacity line, then "i hash winrate" / "l hash" lines) to the
    reference's NNCache and returns its answers, one line per lookup."""
    env = dict(os.environ)
    env.pop("LD_PRELOAD", None)
    r = subprocess.run([REF_CACHE], input=script, capture_output=True, text=True, env=env,
                       timeout=600)
    if r.returncode != 0:
        raise RuntimeError("ref_cache failed: " + r.stderr[-500:])
    return r.stdout.splitlines()


def ref_board_replay(games):
    """Replays move lists through the reference's FullBoard.  Returns one dict per game:
    {"illegal": index} or {"ko", "superko", "score", "stones"[361], "legal"[362]}."""
    text = "".join("%d %s\n" % (len(g), " ".join(str(int(m)) for m in g)) for g in games)
    env = dict(os.environ)
    env.pop("LD_PRELOAD", None)
    r = subprocess.run([REF_BOARD], input=text, capture_output=True, text=True, env=env,
                       timeout=600)
    if r.returncode != 0:
        raise RuntimeError("ref_board failed: " + r.stderr[-500:])
    out = []
    for line in r.stdout.splitlines():
        f = line.split()
        if f[0] == "illegal":
            out.append({"illegal": int(f[1])})
        else:
            out.append({"ko": int(f[1]), "superko": f[2] == "1", "score": float(f[3]),
                        "stones": [int(c) for c in f[4]], "legal": [c == "1" for c in f[5]]})
    return out

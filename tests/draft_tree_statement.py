"""An independent statement of the draft selector's tree (after the reference's own test reference,
dev/tests/engine/draft_selector_metal_test.mm:276-516): every entry the tree could ever push is listed by walking all
paths in fp64, the list is sorted by estimate (stable), and rows are taken from it in order. Returns None where the order
hangs on less than one part in 10^4 (float sums decide there), which callers set aside."""
import math

import numpy as np

M64 = (1 << 64) - 1


def mix(v):
    v = ((v ^ (v >> 30)) * 0xbf58476d1ce4e5b9) & M64
    v = ((v ^ (v >> 27)) * 0x94d049bb133111eb) & M64
    return v ^ (v >> 31)


def child_key(parent, token):
    return mix((parent + 0x9e3779b97f4a7c15 * (token + 1)) & M64)


def gumbel(key, token):
    v = mix(key ^ ((0xd1b54a32d192ed03 * (token + 1)) & M64))
    uniform = float(np.float32((np.float32(v >> 41) + np.float32(0.5)) * np.float32(2.0 ** -23)))
    return -math.log(-math.log(uniform))


def lattice(candidates, unary, edges):
    """(q fp64 [7][16][16], ranked [7][16][16]: candidate indices by score, the lower index first among equal scores)."""
    score = unary.astype(np.float32)[:, None, :] + edges.astype(np.float32)      # fp32, as the kernel adds them
    s = score.astype(np.float64)
    w = np.exp(s - s.max(axis=2, keepdims=True))
    q = w / w.sum(axis=2, keepdims=True)
    ranked = np.argsort(-s, axis=2, kind="stable")
    return q, ranked


def tree(candidates, unary, edges, lane, chain_tokens=None, chain_rates=None):
    q_all, ranked = lattice(candidates, unary, edges)
    ids = np.asarray(candidates)
    T, children, depth, chained = float(lane.temperature), lane.children, lane.depth, lane.chain
    slope, intercept = float(lane.slope), [float(v) for v in lane.intercept]
    noise = lane.noise[0] | lane.noise[1] << 32

    tempered = {}

    def q_t(q, i):
        if T == 0.0:
            return q[i]
        if id(q) not in tempered:      # (q is a row of q_all, which lives as long as this call)
            top = q.max()
            w = np.array([math.exp((math.log(v) - math.log(top)) / T) if v > 0 else v for v in q])
            tempered[id(q)] = w / w.sum()
        return tempered[id(q)][i]

    def estimate(q, position):
        q = min(max(q, 1e-6), 1 - 1e-6)
        return 1.0 / (1.0 + math.exp(-(slope * math.log(q / (1 - q)) + intercept[position])))

    def agreement(token, d):
        if d >= 7:
            return 3
        if token == ids[d][0]:
            return 0
        return 1 if token in ids[d][1:] else 2
    rate_of = lambda d: float(chain_rates[d][agreement(chain_tokens[d], d)])
    entries, ambiguous, expansions = [], set(), {}
    rows_of_q = [[q_all[p][c] for c in range(16)] for p in range(7)]      # one array object a (position, predecessor)

    def expand(path, key, position, predecessor, score):
        q = rows_of_q[position][predecessor]
        if T == 0.0:
            taken = list(ranked[position][predecessor][:children])
        else:
            keys = sorted(((math.log(q_t(q, i)) + gumbel(key, int(ids[position][i])), i) for i in range(16) if q_t(q, i) > 0),
                          key=lambda k: -k[0])
            taken = []
            for n, (value, i) in enumerate(keys[:children]):
                taken.append(i)
                if n + 1 < len(keys) and value - keys[n + 1][0] < 1e-4:
                    ambiguous.add(tuple(path))
        draws = []
        expansions[tuple(path)] = (draws, [q_t(q, i) for i in range(16)])
        on_chain = position < chained and list(path) == [int(t) for t in chain_tokens[:len(path)]]
        rate = rate_of(position) if on_chain else 0.0
        bound, left, reserved = score, 1.0 - rate, rate
        for index in taken:
            if not q[index] > 0:
                break
            draws.append(index)
            token = int(ids[position][index])
            joins = on_chain and token == int(chain_tokens[position])
            cap = left + reserved if joins else left
            own = min(estimate(q_t(q, index), position), cap)
            bound = min(bound, score * own)
            entries.append((tuple(path) + (token,), bound, False, cap))
            left = cap - max(own, reserved) if joins else left - own
            reserved = 0.0 if joins else reserved
            if position + 1 < depth and position + 1 < 7:
                expand(list(path) + [token], child_key(key, token), position + 1, index, bound)
    if depth > 0:
        expand([], noise, 0, 0, 1.0)
    score = 1.0
    for d in range(min(chained, depth)):
        score *= rate_of(d)
        entries.append((tuple(int(t) for t in chain_tokens[:d + 1]), score, True, 1.0))
    order = sorted(range(len(entries)), key=lambda e: -entries[e][1])     # stable: equal estimates keep their order
    entries = [entries[e] for e in order]
    rows = [dict(path=(), parent=None, estimate=1.0, q=1.0, cap=1.0, draws=[], next=None)]
    if depth > 0:
        rows[0]["draws"], rows[0]["next"] = expansions[()]
    made = {(): 0}

    def drafted(path):
        position = len(path) - 1
        own = list(ids[position]).index(path[-1])
        predecessor = list(ids[position - 1]).index(path[-2]) if position else 0
        return q_t(rows_of_q[position][predecessor], own)
    most = min(16, depth + 1)
    for n, (path, estimate_, from_chain, cap) in enumerate(entries):
        if len(rows) >= most:
            break
        if n + 1 < len(entries):
            after = entries[n + 1]
            siblings = len(after[0]) == len(path) and after[0][:-1] == path[:-1]
            if after[0] != path and after[1] >= estimate_ * (1 - 1e-4) and not (siblings and after[1] == estimate_):
                return None
        if path in made:
            row = rows[made[path]]
            if not from_chain and row["q"] < 0:
                row["q"], row["cap"] = drafted(path), cap
            if not from_chain and not row["draws"] and path in expansions:
                row["draws"], row["next"] = expansions[path]
            continue
        row = dict(path=path, parent=made[path[:-1]], estimate=estimate_, q=-1.0 if from_chain else drafted(path),
                   cap=1.0 if from_chain else cap, draws=[], next=None)
        if not from_chain and path in expansions:
            row["draws"], row["next"] = expansions[path]
        made[path] = len(rows)
        rows.append(row)
    if any(row["path"] in ambiguous for row in rows):
        return None
    return rows

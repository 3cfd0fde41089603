"""Draft trees for the verify-rows layout's tests, and the layout told another way (a stable sort, a recursive
preorder) for pinning the oracle. Test infrastructure only."""
import numpy as np

from tests import oracle as orc


def grown_trees(rng, lanes, ties=False):
    """Each lane's tree as a selector leaves it: rows in the order taken, best first, a row's parent among the rows before
    it, estimates that fall along every path (a child is no likelier than its parent) and in take order."""
    tokens = rng.integers(0, 50000, (lanes, 16)).astype(np.uint32)
    trees = np.zeros((lanes, 16), dtype=orc.TREE_DTYPE)
    scores = np.zeros((lanes, 16, 2), dtype=np.float32)
    sizes = rng.integers(1, 17, lanes).astype(np.uint32)
    for lane in range(lanes):
        estimates = np.sort(rng.uniform(0.02, 1.0, 16).astype(np.float32))[::-1]
        if ties:
            estimates = np.round(estimates * 4) / 4
        for row in range(16):
            parent = 0xFFFF if row == 0 else int(rng.integers(0, row))
            depth = 0 if row == 0 else int(trees[lane, parent]["depth"]) + 1
            ancestors = (1 << row) | (0 if row == 0 else int(trees[lane, parent]["ancestors"]))
            trees[lane, row] = (ancestors, parent, depth)
            scores[lane, row] = (rng.uniform(0, 1), 1.0 if row == 0 else estimates[row])
    return tokens, trees, scores, sizes


def layout_by_sorting(tokens, trees, scores, sizes, rows, lane_cap, floor):
    """The same layout: candidates (every row past an anchor) in a stable descending sort of their estimates, taken while
    rows remain, lanes under their cap skipped over, ended by the first below the floor; a lane keeps the first rows of
    its tree, as many as it took; preorder by recursion, children in the order taken."""
    lanes = len(sizes)
    candidates = [(float(scores[lane, row, 1]), lane, row) for lane in range(lanes) for row in range(1, int(sizes[lane]))]
    candidates.sort(key=lambda c: -c[0])          # stable: lane order, then row order, among equals
    taken_of, taken = [1] * lanes, lanes
    for estimate, lane, _ in candidates:
        if taken >= rows or estimate < floor:
            break
        if taken_of[lane] == lane_cap:
            continue
        taken_of[lane] += 1
        taken += 1
    out_tokens, out_tree, out_sources, lane_rows = [], [], [], []
    for lane in range(lanes):
        mine = taken_of[lane]
        children = {r: [c for c in range(r + 1, mine) if int(trees[lane, c]["parent"]) == r] for r in range(mine)}
        order = []

        def visit(row, up, ancestors, depth):
            at = len(order)
            ancestors |= 1 << at
            order.append((row, up, ancestors, depth))
            for child in children[row]:
                visit(child, at, ancestors, depth + 1)
        visit(0, 0xFFFF, 0, 0)
        lane_rows.append((len(out_tokens), len(order)))
        for row, up, ancestors, depth in order:
            out_tokens.append(int(tokens[lane, row])); out_tree.append((ancestors, up, depth)); out_sources.append(row)
    while len(out_tokens) < rows:
        out_tokens.append(int(tokens[0, 0])); out_tree.append((0, 0xFFFF, 0)); out_sources.append(0xFFFFFFFF)
    return (np.array(out_tokens, np.uint32), np.array(out_tree, dtype=orc.TREE_DTYPE), np.array(lane_rows, np.uint32),
            np.array(out_sources, np.uint32))


def bf16_bits(values):
    """fp32 values truncated to bf16 bit patterns (uint16): test data need no rounding."""
    return (np.ascontiguousarray(values, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def bf16_values(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def proposal_logits(rng, lanes, columns, kind):
    """fp32 [lanes * 8][columns] draft logits: plain, heavily tied (few distinct values, signed zeros among them), or
    mostly -infinity so that a row has fewer than sixteen finite columns."""
    shape = (lanes * 8, columns)
    if kind == "tied":
        return rng.choice(np.array([-2.0, -0.0, 0.0, 1.5, 3.0], np.float32), shape)
    logits = (rng.standard_normal(shape) * 4).astype(np.float32)
    if kind == "sparse":
        logits[rng.random(shape) < 0.999] = -np.inf
    return logits


def candidates_by_sorting(logits, lanes, leading, trailing):
    """The same candidates from a lexicographic sort: logit descending, column ascending; -0 equals +0."""
    columns = logits.shape[1]
    candidates, unary = np.full((lanes * 7, 16), 0xFFFFFFFF, np.uint32), np.full((lanes * 7, 16), -np.inf, np.float32)
    for row in range(lanes * 7):
        x = logits[row // 7 * 8 + row % 7 + 1]
        order = np.lexsort((np.arange(columns), -(x.astype(np.float64) + 0.0)))[:16]
        tokens = np.where(order < leading, order, order - leading + trailing)
        candidates[row, :len(order)] = tokens
        unary[row, :len(order)] = x[order]
    return candidates, unary


def edges_by_einsum(candidates, anchors, vocabulary, hidden, before, after):
    """fp64 sum over the rank of predecessor x hidden x successor of the decoded bf16 factors; NaN where the kernel writes
    nothing (position 0's rows past the anchor's)."""
    h, b, a = (bf16_values(x).astype(np.float64) for x in (hidden, before, after))
    out = np.full((candidates.shape[0], 16, 16), np.nan)
    for row in range(candidates.shape[0]):
        lane, position = divmod(row, 7)
        previous = candidates[row - 1] if position else np.array([anchors[lane]], np.uint32)
        previous, tokens = np.minimum(previous, vocabulary - 1), np.minimum(candidates[row], vocabulary - 1)
        scores = np.einsum("pd,d,cd->pc", b[previous], h[lane * 8 + position + 1], a[tokens])
        out[row, :len(previous)] = scores
    return out

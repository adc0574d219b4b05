"""TEST INFRASTRUCTURE -- brute-force pins for tiny DAGs (pure Python, float64).

Enumerates every strictly increasing node sequence 0 = a_0 < ... < a_{T_b-1} = L_b-1 and
sums / maximises exp(sum_t match[t][a_t] + sum_t links[a_t][a_{t+1}]).  This is the
definition the dynamic programs of fs_plugins/custom_ops/dag_loss.py:259-353 evaluate;
it shares no code with them.
"""
import itertools
import math


def paths(Lb, Tb):
    if Tb == 1:
        if Lb == 1:
            yield (0,)
        return
    for mid in itertools.combinations(range(1, Lb - 1), Tb - 2):
        yield (0,) + mid + (Lb - 1,)


def path_score(match, links_sq, p):
    s = 0.0
    for t, j in enumerate(p):
        s += float(match[t][j])
    for a, b in zip(p[:-1], p[1:]):
        s += float(links_sq[a][b])
    return s


def log_likelihood(match, links_sq, Lb, Tb):
    """log sum over all paths (float64, via max-shifted sum); -inf when no path is finite."""
    scores = [path_score(match, links_sq, p) for p in paths(Lb, Tb)]
    scores = [s for s in scores if s > -math.inf]
    if not scores:
        return -math.inf
    top = max(scores)
    return top + math.log(sum(math.exp(s - top) for s in scores))


def posteriors(match, links_sq, Lb, Tb):
    """node posterior[t][j] and edge posterior[i][j] under the path distribution."""
    T = len(match); L = len(match[0])
    z = log_likelihood(match, links_sq, Lb, Tb)
    node = [[0.0] * L for _ in range(T)]
    edge = [[0.0] * L for _ in range(L)]
    if z == -math.inf:
        return node, edge
    for p in paths(Lb, Tb):
        s = path_score(match, links_sq, p)
        if s == -math.inf:
            continue
        w = math.exp(s - z)
        for t, j in enumerate(p):
            node[t][j] += w
        for a, b in zip(p[:-1], p[1:]):
            edge[a][b] += w
    return node, edge


def best_path(match, links_sq, Lb, Tb):
    """(best score, list of paths attaining it) -- callers use it on tie-free inputs or
    inspect the whole arg-max set."""
    best, arg = -math.inf, []
    for p in paths(Lb, Tb):
        s = path_score(match, links_sq, p)
        if s > best:
            best, arg = s, [p]
        elif s == best and s > -math.inf:
            arg.append(p)
    return best, arg

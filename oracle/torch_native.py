"""TEST INFRASTRUCTURE -- CPU oracle, never a product path.

Torch restatement of DA-Transformer's torch-native DAG operators.  Only the test
suite, the smoke check and the CPU-baseline leg of the benchmark may import this
module; the shipped operators never call into it.

Every function names the reference lines it restates
(paths relative to the DA-Transformer checkout):

    logsumexp_keepdim                   fs_plugins/custom_ops/dag_loss.py:237-245
    torch_dag_loss                      fs_plugins/custom_ops/dag_loss.py:247-251, 259-300
    torch_dag_max_score                 fs_plugins/custom_ops/dag_loss.py:253-257, 303-320
    torch_dag_best_alignment            fs_plugins/custom_ops/dag_loss.py:322-353
    torch_dag_logsoftmax_gather_inplace fs_plugins/custom_ops/dag_loss.py:355-359
    restore_valid_links                 fs_plugins/models/glat_decomposed_with_link.py:337-349
                                        (same as fs_plugins/custom_ops/dag_loss.py:373-382)
    extract_valid_links                 fs_plugins/models/glat_decomposed_with_link.py:319-335
    force_alignment                     fs_plugins/criterions/nat_dag_loss.py:111-120
    multihead_links                     fs_plugins/models/glat_decomposed_with_link.py:319-335, 380-404
                                        (the tail of extract_links, shifted branch)
    glat_glance                         fs_plugins/criterions/nat_dag_loss.py:273-278, 307-311
                                        (glat_function after the alignment, glance_strategy None)
    glat_mix                            fs_plugins/criterions/nat_dag_loss.py:307-311
    inference_viterbi                   fs_plugins/models/glat_decomposed_with_link.py:720-777
                                        (decode_strategy viterbi / jointviterbi)
    inference_lookahead_simple          fs_plugins/models/glat_decomposed_with_link.py:691-718
                                        (decode_strategy lookahead / greedy without n-gram blocking)

How each one is pinned (the reference holds no golden vectors for this path):

    torch_dag_loss           brute-force path enumeration (oracle/brute.py), closed forms
                             (T_b=2, T_b=L_b), posterior-mass invariants, fp64 gradcheck,
                             the plain-C fp64 restatement (oracle/dagref.c)
    logsumexp_keepdim        torch.logsumexp + the all -inf special case
    torch_dag_best_alignment brute-force argmax on tie-free inputs, hand-derived tie
                             cases, path-score re-summation, the C restatement
    torch_dag_logsoftmax_gather_inplace   torch.log_softmax + gather (library routine)
    layout converters        round trip on the valid band
    force_alignment          fragment-sum identity of nat_dag_loss.py:122-152
    multihead_links          rows sum to one (sum_d exp(links) = 1 wherever a transition exists), one head
                             reduces to torch.log_softmax over the window, float64 loops on tiny shapes,
                             fp64 gradcheck -- tests/test_oracle_links.py
    glat_glance, glat_mix    a case worked by hand, the limits context_p = 0 (nothing but the
                             already pinned nodes is kept) and rand = 0 with context_p >= 1 and no
                             correct prediction (every assigned node is kept), pure-Python loops
                             on random cases -- tests/test_oracle_glat.py
    inference_viterbi        exhaustive enumeration of every path through tiny graphs (score, length
                             penalty, token collapsing), a case worked by hand
                             -- tests/test_oracle_viterbi.py
    inference_lookahead_simple   a case worked by hand, numpy float32 loops over the definition
                             -- tests/test_oracle_viterbi.py
"""

import torch

NEG_INF = float("-inf")


def logsumexp_keepdim(x, dim):
    """log-sum-exp along `dim` (kept), with all -inf slices giving -inf and a zero
    (not NaN) gradient.  Restates dag_loss.py:237-245."""
    top = x.max(dim=dim, keepdim=True).values.detach()
    dead = top == NEG_INF
    shift = top.masked_fill(dead, 0.0)
    total = (x - shift).exp().sum(dim=dim, keepdim=True)
    return total.masked_fill(dead, 1.0).log() + shift.masked_fill(dead, NEG_INF)


def _check_square(links):
    assert links.dim() == 3 and links.shape[1] == links.shape[2], \
        "links should be batch_size * prelen * prelen"


def torch_dag_loss(match_all, links, output_length, target_length):
    """log P(target | graph) per sample, square links [B,L,L] (links[b,i,j] = log P(i->j),
    -inf where there is no edge).  match_all is [B,T,L].  Restates dag_loss.py:259-300:
    f[0] = -inf except node 0; f[k][j] = LSE_i(f[k-1][i] + links[i][j]) + match[k][j];
    the answer is read at (target_length-1, output_length-1).  Differentiable through
    autograd in match_all and links."""
    _check_square(links)
    bsz, tarlen, prelen = match_all.shape
    f = match_all.new_full((bsz, prelen), NEG_INF)
    f[:, 0] = match_all[:, 0, 0]
    steps = [f]
    for k in range(1, tarlen):
        nxt = logsumexp_keepdim(steps[-1].unsqueeze(2) + links, 1).squeeze(1)  # [B,L]
        steps.append(nxt + match_all[:, k, :])
    table = torch.stack(steps, dim=1)  # [B,T,L]
    rows = torch.arange(bsz, device=match_all.device)
    return table[rows, target_length - 1, output_length - 1]


def torch_dag_max_score(match_all, links, output_length, target_length):
    """Max-semiring version of torch_dag_loss: score of the single best path.
    Restates dag_loss.py:253-257 and 303-320 (add, then max over predecessors,
    then add the match term: two roundings per cell)."""
    _check_square(links)
    bsz, tarlen, prelen = match_all.shape
    f = match_all.new_full((bsz, prelen), NEG_INF)
    f[:, 0] = match_all[:, 0, 0]
    steps = [f]
    for k in range(1, tarlen):
        best = torch.max(steps[-1].unsqueeze(2) + links, dim=1)[0]
        steps.append(best + match_all[:, k, :])
    table = torch.stack(steps, dim=1)
    rows = torch.arange(bsz, device=match_all.device)
    return table[rows, target_length - 1, output_length - 1]


def torch_dag_best_alignment(match_all, links, output_length, target_length):
    """Best alignment as [B,L] int64: entry j holds the target position emitted by node j
    on the best path, -1 for nodes off the path.  Restates dag_loss.py:322-353: the path
    is recovered as the gradient of the summed best score w.r.t. match_all (one-hot on the
    path; torch.max(dim) routes ties to the lowest predecessor index).  Unlike the
    reference this does not flip requires_grad on the caller's tensor."""
    with torch.enable_grad():
        leaf = match_all.detach().requires_grad_()
        score = torch_dag_max_score(leaf, links.detach(), output_length, target_length)
        onehot = torch.autograd.grad(score.sum(), [leaf])[0]  # [B,T,L]
    weight, path = onehot.max(dim=1)
    path.masked_fill_(weight < 0.5, -1)
    return path


def torch_dag_logsoftmax_gather_inplace(word_ins_out, select_idx):
    """(word_ins_out, log_softmax(word_ins_out, fp32).gather(-1, select_idx)).
    Restates dag_loss.py:355-359; the logits are left untouched."""
    logp = torch.log_softmax(word_ins_out, -1, dtype=torch.float32)
    return word_ins_out, logp.gather(dim=-1, index=select_idx)


def restore_valid_links(links):
    """shifted [B,L,translen] (entry [i,d] = log P(i -> i+d+1)) -> square [B,L,L].
    Restates glat_decomposed_with_link.py:337-349."""
    bsz, prelen, translen = links.shape
    dst = torch.arange(prelen, device=links.device).unsqueeze(1) \
        + torch.arange(translen, device=links.device).unsqueeze(0) + 1
    dst = dst.clamp(max=prelen)  # out-of-range targets are parked in a spare column
    wide = links.new_full((bsz, prelen, prelen + 1), NEG_INF)
    wide.scatter_(2, dst.unsqueeze(0).expand(bsz, -1, -1), links)
    return wide[:, :, :prelen]


def extract_valid_links(square, translen=None):
    """square [B,L,L] -> shifted [B,L,translen]; positions that would point past the last
    node hold -inf.  Restates the gather of glat_decomposed_with_link.py:319-335 (without
    the head dimension and the validity mask, which belong to the model)."""
    bsz, prelen, _ = square.shape
    if translen is None or translen > prelen - 1:
        translen = prelen - 1
    dst = torch.arange(prelen, device=square.device).unsqueeze(1) \
        + torch.arange(translen, device=square.device).unsqueeze(0) + 1
    beyond = dst >= prelen
    out = square.gather(2, dst.clamp(max=prelen - 1).unsqueeze(0).expand(bsz, -1, -1))
    return out.masked_fill(beyond.unsqueeze(0), NEG_INF)


def force_alignment(match, force_emit):
    """Pin node j to target force_emit[b,j] (>= 0): that target's row of match becomes 0 at
    node j and -inf elsewhere; rows of unforced targets are unchanged and forced rows carry
    no gradient.  Restates nat_dag_loss.py:111-120."""
    bsz, tarlen, prelen = match.shape
    hit = torch.zeros(bsz, tarlen + 1, prelen, dtype=torch.bool, device=match.device)
    hit.scatter_(1, force_emit.unsqueeze(1) + 1, True)
    hit = hit[:, 1:]
    forced_row = hit.any(dim=-1, keepdim=True)
    pinned = torch.zeros_like(match).masked_fill_(~hit, NEG_INF).masked_fill_(~forced_row, 0.0)
    return match.masked_fill(forced_row, 0.0) + pinned


def multihead_links(content, log_gates, transition_valid_mask, translen):
    """Transition log-probabilities in the shifted layout from per-head scores.

    content [B,L,L,H]: score of i -> j for every head;  log_gates [B,L,H]: log-probability of
    every head at node i;  transition_valid_mask [B,L,L] bool: allowed (i, j), already restricted
    to j > i.  Every head's scores are normalised over the allowed targets inside the window
    j - i <= translen (log_softmax), the heads are mixed with the gates (logsumexp).  Rows without
    any allowed transition are -inf.  Restates glat_decomposed_with_link.py:319-335
    (extract_valid_links) and :397-404."""
    bsz, prelen, _, heads = content.shape
    translen = min(translen, prelen - 1)
    dst = torch.arange(prelen, device=content.device).unsqueeze(1) \
        + torch.arange(translen, device=content.device).unsqueeze(0) + 1           # [L, translen]
    masked = content.masked_fill(~transition_valid_mask.unsqueeze(-1), NEG_INF)
    window = masked.gather(2, dst.clamp(max=prelen - 1)[None, :, :, None].expand(bsz, -1, -1, heads))
    window = window.masked_fill((dst >= prelen)[None, :, :, None], NEG_INF)
    nouse = ~transition_valid_mask.any(-1)                                         # [B, L]
    window = window.masked_fill(nouse[:, :, None, None], 0.0)                      # (keeps log_softmax finite; overwritten below)
    logp = torch.log_softmax(window, dim=2).masked_fill(nouse[:, :, None, None], NEG_INF)
    return logsumexp_keepdim(logp + log_gates.unsqueeze(2), dim=-1).squeeze(-1)


def glat_mix(path, oracle, prev_output_tokens, keep_prob, rand, glat_prev_mask):
    """Which nodes get their reference token revealed: keep = rand < keep_prob or already pinned;
    the decoder input takes the oracle token there; force_emit for the second pass is the path
    on kept nodes and -1 elsewhere.  Restates nat_dag_loss.py:307-311."""
    keep_word_mask = (rand < keep_prob).bool() | glat_prev_mask
    glat_prev_output_tokens = prev_output_tokens.masked_fill(keep_word_mask, 0) + oracle.masked_fill(~keep_word_mask, 0)
    next_force_emit = path.masked_fill(~keep_word_mask, -1)
    return keep_word_mask, glat_prev_output_tokens, next_force_emit


def glat_glance(path, tgt_tokens, pred_tokens, prev_output_tokens, glat_prev_mask, target_length, context_p, rand):
    """Glancing after the best alignment (glance_strategy None).  oracle[b,j] = the target token
    node j emits on the path (target 0's token for unassigned nodes); same_num[b] = assigned,
    not yet pinned nodes whose argmax prediction is already that token; every assigned node is
    kept with probability (T_b - pinned - same_num) / T_b * context_p.
    Returns (oracle, same_num, keep_prob, keep_word_mask, glat_prev_output_tokens, next_force_emit).
    Restates nat_dag_loss.py:273-278 and :307-311."""
    predict_assigned_mask = path >= 0
    oracle = tgt_tokens.gather(-1, path.clip(min=0))
    same_num = ((pred_tokens == oracle) & predict_assigned_mask & ~glat_prev_mask).sum(1)
    keep_prob = ((target_length - glat_prev_mask.sum(dim=-1) - same_num) / target_length * context_p).unsqueeze(-1) \
        * predict_assigned_mask.float()
    return (oracle, same_num, keep_prob) + glat_mix(path, oracle, prev_output_tokens, keep_prob, rand, glat_prev_mask)


def inference_viterbi(links, unreduced_logits, unreduced_tokens, output_length, upsample_scale, viterbibeta,
                      joint, pad_index):
    """Length-penalised Viterbi decoding of the graph.  links [B,L,L] square transition
    log-probabilities, unreduced_logits / unreduced_tokens [B,L] the best token of every node and
    its log-probability, output_length [B] nodes per graph (node 0 and node L_b-1 are the two
    ends and emit nothing here).  A path 0 -> x_0 -> ... -> x_{n-1} -> L_b-1 with
    n <= int(2 L / upsample_scale) scores the sum of its transitions plus, in the joint form, the
    token log-probabilities of node 0 and of every x_k (the plain form adds that of x_0 only),
    divided by n ** viterbibeta; the best one is read back and its tokens are collapsed (pads and
    immediate repeats dropped, the last token always kept).  Like the reference it works on the
    first row of `links` in place, so it takes a copy.
    Returns (output_tokens [B, longest] padded with pad_index, pred_length [B], nodes: list of the
    x_k per sample).  Restates glat_decomposed_with_link.py:720-777."""
    links = links.clone()
    bsz, graph_length, _ = links.shape
    tokens = unreduced_tokens.tolist()
    reach = links[:, 0]                                  # a view: the updates below land in `links`
    if joint:
        reach += unreduced_logits[:, 0].unsqueeze(1)
    reach += unreduced_logits
    per_step, back = [reach], []
    max_length = int(2 * graph_length / upsample_scale)
    for _ in range(max_length - 1):
        reach, source = torch.max(reach.unsqueeze(-1) + links, dim=1)
        if joint:
            reach += unreduced_logits
        per_step.append(reach)
        back.append(source)
    back = torch.stack(back, dim=0)                      # [max_length-1, B, L]
    per_step = torch.stack(per_step, dim=0)              # [max_length, B, L]
    to_end = torch.gather(links, -1, (output_length - 1).view(bsz, 1, 1).repeat(1, graph_length, 1))
    per_step += to_end.view(1, bsz, graph_length)
    best, last_node = torch.max(per_step, dim=-1)        # [max_length, B]
    lengths = torch.arange(max_length).unsqueeze(-1).repeat(1, bsz) + 1
    best = best / (lengths ** viterbibeta)
    _, pred_length = torch.max(best, dim=0)
    pred_length = pred_length + 1
    start = torch.gather(last_node, 0, (pred_length - 1).view(1, bsz)).view(bsz).tolist()
    back = back.tolist()
    out, nodes = [], []
    for b, n in enumerate(pred_length.tolist()):
        j = start[b]
        seen = tokens[b][j]
        res, walk = [seen], [j]
        for k in range(n - 1):
            j = back[n - k - 2][b][j]
            walk.insert(0, j)
            tok = tokens[b][j]
            if tok != pad_index and tok != seen:
                res.insert(0, tok)
            seen = tok
        out.append(res)
        nodes.append(walk)
    longest = max(len(r) for r in out)
    output_tokens = torch.tensor([r + [pad_index] * (longest - len(r)) for r in out])
    return output_tokens, pred_length, nodes


def inference_lookahead_simple(links, unreduced_logits, unreduced_tokens, output_length, decode_beta, greedy, pad_index):
    """Greedy walk through the graph: from node 0 always to the successor with the best
    transition log-probability (greedy) or transition + decode_beta * token log-probability
    (lookahead), until the last node; the tokens on the way are collapsed (pads and immediate
    repeats dropped, the first token always kept).  links [B,L,L] square.
    Returns (output_tokens [B, longest] padded with pad_index, nodes: list of the visited nodes).
    Restates glat_decomposed_with_link.py:691-718."""
    tokens = unreduced_tokens.tolist()
    if greedy:
        successor = links.max(dim=-1)[1].tolist()
    else:
        successor = (links + unreduced_logits.unsqueeze(1) * decode_beta).max(dim=-1)[1].tolist()
    out, nodes = [], []
    for b, length in enumerate(output_length.tolist()):
        seen = tokens[b][0]
        j, res, walk = 0, [seen], [0]
        while j != length - 1:
            j = successor[b][j]
            walk.append(j)
            tok = tokens[b][j]
            if tok != pad_index and tok != seen:
                res.append(tok)
            seen = tok
        out.append(res)
        nodes.append(walk)
    longest = max(len(r) for r in out)
    return torch.tensor([r + [pad_index] * (longest - len(r)) for r in out]), nodes

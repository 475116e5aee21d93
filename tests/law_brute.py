"""The drafter's proposal law restated in double precision from its definition, without looking at how
the oracle or the kernels compute it (src/engine/gemma3_draft.mm:186-395 states the rule per kernel):

  score_i = logit_i / T
  support = every token whose score is >= the top_k-th best score (ties stay; top_k = 0: all tokens)
  w_i     = exp(score_i - max score) over the support, sorted by (score desc, token asc)
  tail_i  = sum of w_j over the entries from the last one up to and including i
  entry i stays if it is the best one, or if (top_p >= 1 or tail_i / total > 1 - top_p)
                                          and (min_p <= 0 or w_i >= min_p)
  mass_i  = w_i / sum of the w that stay

Every comparison that decides membership reports its margin, so a test can leave out the cases where
single and double precision may legitimately decide differently."""
import math

import numpy as np


def law(logits, temperature, top_k, top_p, min_p):
    """Returns (tokens that stay -> mass, smallest relative margin of any membership decision)."""
    scores = np.asarray(logits, np.float64) / float(np.float32(temperature))
    vocab = scores.size
    order = np.lexsort((np.arange(vocab), -scores))        # score descending, token ascending
    margin = math.inf
    if top_k and top_k < vocab:
        cutoff = scores[order[top_k - 1]]
        support = order[scores[order] >= cutoff]
        below = scores[scores < cutoff]
        if below.size:                                      # distance of the best excluded score from the cutoff
            margin = min(margin, abs(cutoff - below.max()) / max(1.0, abs(cutoff)))
    else:
        support = order
    top = scores[support[0]]
    w = np.exp(scores[support] - top)
    total = float(w.sum())
    tails = np.cumsum(w[::-1])[::-1]
    stays = {}
    kept_weight = 0.0
    for i, token in enumerate(support.tolist()):
        keep = True
        if i > 0:
            if top_p < 1.0:
                edge = 1.0 - float(np.float32(top_p))
                margin = min(margin, abs(tails[i] / total - edge))
                keep = keep and tails[i] / total > edge
            if min_p > 0.0:
                edge = float(np.float32(min_p))
                margin = min(margin, abs(w[i] - edge) / edge)
                keep = keep and w[i] >= edge
        if keep:
            stays[token] = float(w[i])
            kept_weight += float(w[i])
    return {t: v / kept_weight for t, v in stays.items()}, margin


def random_case(rng, vocab):
    """(logits, T, top_k, top_p, min_p) with exact ties, plateaus and heavy or light tails in the mix."""
    sigma = float(rng.choice([0.5, 1.5, 3.0, 6.0]))
    logits = rng.normal(0, sigma, vocab).astype(np.float32)
    kind = int(rng.integers(0, 4))
    if kind == 1:      # exact ties around the cutoff
        logits[rng.integers(0, vocab, 40)] = np.sort(logits)[-int(rng.integers(2, 60))]
    elif kind == 2:    # a plateau at the very top
        logits[rng.integers(0, vocab, int(rng.integers(2, 30)))] = logits.max() + np.float32(0.25)
    temperature = float(rng.choice([0.3, 0.7, 1.0, 1.3, 2.0]))
    top_k = int(rng.choice([1, 2, 8, 40, 64]))
    top_p = float(rng.choice([1.0, 0.99, 0.95, 0.9, 0.5]))
    min_p = float(rng.choice([0.0, 0.0, 0.02, 0.05, 0.3]))
    return logits, temperature, top_k, top_p, min_p

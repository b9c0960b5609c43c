"""Host-side token selection of globals.js:47-74."""
import math
import random


def selectTopK(probs, top_k):
    """Stable descending sort by value, first top_k (globals.js:66-74): ties keep the
    lower index first."""
    order = sorted(range(len(probs)), key=lambda i: -float(probs[i]))
    topKIndices = order[:top_k]
    return {"topKIndices": topKIndices, "topKProbs": [float(probs[i]) for i in topKIndices]}


def cpuSoftmax(logits, temperature=1.0):
    """float64 softmax with the temperature inside the exponent (globals.js:59-64)."""
    m = max(logits)
    e = [math.exp((x - m) / temperature) for x in logits]
    s = 0.0
    for v in e:
        s += v
    return [v / s for v in e]


def sampleFromDistribution(probs, rand=None):
    """Inverse-CDF sampling (globals.js:47-57)."""
    r = random.random() if rand is None else rand
    c = 0.0
    for i, p in enumerate(probs):
        c += p
        if r < c:
            return i
    return len(probs) - 1

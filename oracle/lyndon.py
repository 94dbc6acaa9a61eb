"""Lyndon-word and Lyndon-basis coordinates of the log signature: CPU restatement (test infrastructure only).

Restates siglib/shared/preparation/log_sig/lyndon_words.cpp and the two compressed log-signature methods of
siglib/cpsig/cp_tensor_log.h:140-170.  Pinned by the reference's third-party golden vectors (``logsig_words__d*`` from
signatory, ``logsig_basis__d*`` from iisignature, and the path gradients through them) in tests/test_oracle_ops.py.
Nothing outside tests/, the smoke check and the benchmark's CPU leg may import this module.

* Lyndon words of length n over d letters in lexicographic order, lengths ascending
  (lyndon_words.cpp:25-49, 72-83: Duval's successor rule).
* method 1: the expanded log signature read off at the Lyndon words (cp_tensor_log.h:140-158).
* method 2: coordinates in the Lyndon (standard-bracketing) basis.  The bracket of a Lyndon word w = uv, v its longest
  proper Lyndon suffix, is P_w = [P_u, P_v]; expanded into words it equals w plus lexicographically larger words of
  the same letters, so the matrix M[i][j] = (coefficient of Lyndon word i in P_j) is unit lower triangular in the
  enumeration order and the coordinates solve M beta = x, x the Lyndon-word coefficients (lyndon_words.cpp:150-244,
  cp_tensor_log.h:161-170 apply the precomputed inverse).
"""
import numpy as np


def lyndon_words(dimension, degree):
    """All Lyndon words of length 1..degree over {0..dimension-1}: lengths ascending, lexicographic inside a length."""
    out = []
    for n in range(1, degree + 1):
        w = [0]
        while w:
            m = len(w)
            if m == n:
                out.append(tuple(w))
            while len(w) < n:
                w.append(w[len(w) - m])
            while w and w[-1] == dimension - 1:
                w.pop()
            if w:
                w[-1] += 1
    return out


def word_index(word, dimension):
    """Index of a word in a scalar-free signature row (levels end to end, words row-major inside a level)."""
    idx = 0
    for letter in word:
        idx = idx * dimension + letter + 1
    return idx - 1


def log_sig_length(dimension, degree):
    return len(lyndon_words(dimension, degree))


def _bracket_polynomials(words):
    """word -> {word: coefficient} expansion of the standard bracketing of every Lyndon word in `words`."""
    known = set(words)
    poly = {}
    for w in words:                      # lengths ascending: both factors are expanded before their product
        if len(w) == 1:
            poly[w] = {w: 1}
            continue
        split = next(i for i in range(1, len(w)) if w[i:] in known)       # longest proper Lyndon suffix
        u, v = w[:split], w[split:]
        acc = {}
        for wu, cu in poly[u].items():
            for wv, cv in poly[v].items():
                acc[wu + wv] = acc.get(wu + wv, 0) + cu * cv
                acc[wv + wu] = acc.get(wv + wu, 0) - cu * cv
        poly[w] = {k: c for k, c in acc.items() if c}
    return poly


def projection_matrix(dimension, degree):
    """Dense M with M[i][j] = coefficient of Lyndon word i in the bracket of Lyndon word j (unit lower triangular)."""
    words = lyndon_words(dimension, degree)
    pos = {w: i for i, w in enumerate(words)}
    poly = _bracket_polynomials(words)
    m = np.zeros((len(words), len(words)))
    for j, w in enumerate(words):
        for word, c in poly[w].items():
            i = pos.get(word)
            if i is not None:
                m[i, j] = c
    return m


def compress(expanded, dimension, degree, method):
    """Expanded (scalar-free) log signature rows -> method 1 (Lyndon words) or method 2 (Lyndon basis) coordinates."""
    words = lyndon_words(dimension, degree)
    idx = np.array([word_index(w, dimension) for w in words], dtype=np.int64)
    x = np.asarray(expanded)[..., idx]
    if method == 1:
        return x
    m = projection_matrix(dimension, degree)
    beta = np.array(x, dtype=np.float64, copy=True)
    for i in range(len(words)):          # forward substitution, unit diagonal
        beta[..., i] -= beta[..., :i] @ m[i, :i]
    return beta.astype(np.asarray(expanded).dtype)


def compress_backprop(derivs, dimension, degree, method):
    """Gradient w.r.t. the expanded (scalar-free) log signature rows given the gradient w.r.t. the coordinates."""
    words = lyndon_words(dimension, degree)
    idx = np.array([word_index(w, dimension) for w in words], dtype=np.int64)
    g = np.array(derivs, dtype=np.float64, copy=True)
    if method == 2:
        m = projection_matrix(dimension, degree)
        for i in range(len(words) - 1, -1, -1):      # transpose solve: dx = M^-T dbeta
            g[..., :i] -= g[..., i:i + 1] * m[i, :i]
    n = 0
    size = dimension
    for _ in range(degree):
        n += size
        size *= dimension
    out = np.zeros(g.shape[:-1] + (n,))
    out[..., idx] = g
    return out.astype(np.asarray(derivs).dtype)

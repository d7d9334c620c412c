"""Independent float64 numpy statement of the model mathematics (textbook LSTM, Luong attention,
softmax, sort-based beam search).  It shares no code with the oracle: it exists to pin the oracle
(tests/test_oracle_pins.py) -- a dropped term, a wrong gate order or a transposed weight in the
oracle shows up as a mismatch here."""
import numpy as np

GATES = ["i", "f", "c", "o"]


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def make_params(rng, layers, H, V_src, V_tgt, attention=True, feed_input=True, scale=0.08, E=None):
    """Reference initialisation: uniform[-scale, scale], forget-gate bias 1
    (src/utility_cu.cu:77-78, src/layer_input_to_hidden.h:651-655).  E: embedding size (default H,
    the reference's only case); the tables are E x V and the first layer's M_* are H x E."""
    P = {}
    E = H if E is None else E

    def u(*shape):
        return rng.uniform(-scale, scale, size=shape).astype(np.float32)

    for side, V in (("src", V_src), ("tgt", V_tgt)):
        for l in range(layers):
            pfx = f"{side}.{l}."
            for g in GATES:
                P[pfx + "W_h" + g] = u(H, H)
                P[pfx + "M_" + g] = u(H, E if l == 0 else H)
                P[pfx + "b_" + g] = u(H)
                if side == "tgt" and l == 0 and attention and feed_input:
                    P[pfx + "Q_" + g] = u(H, H)
            P[pfx + "b_f"] = np.ones(H, np.float32)
            if l == 0:
                P[pfx + "W"] = u(E, V)
    if attention:
        for n in ("W_a", "W_p", "W_c1", "W_c2"):
            P["attn." + n] = u(H, H)
        P["attn.v_p"] = u(H)
        P["attn.b_out"] = u(H)
    P["softmax.D"] = u(V_tgt, H)
    P["softmax.b_d"] = u(V_tgt)
    return P


def lstm_step(P, pfx, x, h, c, h_tild=None, mask=None):
    P = {k: v.astype(np.float64) for k, v in P.items() if k.startswith(pfx)}
    s = {}
    for g in GATES:
        v = P[pfx + "M_" + g] @ x + P[pfx + "W_h" + g] @ h + P[pfx + "b_" + g][:, None]
        if h_tild is not None:
            v = v + P[pfx + "Q_" + g] @ h_tild
        s[g] = v
    i, f, o, g = sigmoid(s["i"]), sigmoid(s["f"]), sigmoid(s["o"]), np.tanh(s["c"])
    c_new = f * c + i * g
    h_new = o * np.tanh(c_new)
    if mask is not None:
        c_new = c_new * mask[None, :]
        h_new = h_new * mask[None, :]
    return h_new, c_new, (i, f, g, o)


def attention_local_p(P, h_t, hs_of, lens, mask, D):
    """hs_of(b, pos) -> encoder top state (H,) of ORIGINAL source position pos of column b."""
    H, B = h_t.shape
    Wp, Wa = P["attn.W_p"].astype(np.float64), P["attn.W_a"].astype(np.float64)
    Wc1, Wc2 = P["attn.W_c1"].astype(np.float64), P["attn.W_c2"].astype(np.float64)
    vp, bo = P["attn.v_p"].astype(np.float64), P["attn.b_out"].astype(np.float64)
    out = np.zeros((H, B))
    aligns = []
    for b in range(B):
        ha = h_t[:, b]
        p = lens[b] * sigmoid(vp @ np.tanh(Wp @ ha))
        # window on the fp32 position the kernels truncate
        pf = np.float32(lens[b]) * np.float32(sigmoid(vp @ np.tanh(Wp @ ha)))
        lo = max(0, int(pf) - D) if D >= 0 else 0
        hi = min(lens[b] - 1, int(pf) + D) if D >= 0 else lens[b] - 1
        pos = list(range(lo, hi + 1))[: (2 * D + 1) if D >= 0 else None]
        ctx = np.zeros(H)
        a_full = {}
        if mask[b] == 1 and pos:
            hs = np.stack([hs_of(b, s) for s in pos], axis=1)  # H x n
            sc = ha @ Wa @ hs
            e = np.exp(sc - sc.max())
            a = e / e.sum()
            if D >= 0:
                a = a * np.exp(-((p - np.array(pos)) ** 2) / (2 * (D * D / 4.0)))
            ctx = hs @ a
            a_full = dict(zip(pos, a))
        out[:, b] = np.tanh(Wc1 @ ctx + Wc2 @ ha + bo) * mask[b]
        aligns.append(a_full)
    return out, aligns


def log_softmax(z):
    z = z - z.max(axis=0, keepdims=True)
    return z - np.log(np.exp(z).sum(axis=0, keepdims=True))


def encode(P, layers, H, src_ids):
    """Single sentence: returns per-layer final (h,c) and the top states by ORIGINAL position."""
    S = len(src_ids)
    h = [np.zeros((H, 1)) for _ in range(layers)]
    c = [np.zeros((H, 1)) for _ in range(layers)]
    top = {}
    for t in range(S):
        pos = S - 1 - t  # the source is fed reversed
        x = P["src.0.W"].astype(np.float64)[:, [src_ids[pos]]]
        for l in range(layers):
            h[l], c[l], _ = lstm_step(P, f"src.{l}.", x, h[l], c[l])
            x = h[l]
        top[pos] = h[layers - 1][:, 0].copy()
    return h, c, top


def beam_decode(P, layers, H, V, src_ids, beam, D, attention=True, feed_input=True, max_ratio=1.5,
                min_ratio=0.5, penalty=0.0, diversity=0.0, lp_alpha=0.65, cp_beta=0.2,
                longest=104, margins=None, alignments=False, ensemble=()):
    """Sort-based beam search with the reference's rules (src/decoder.h:355-699).  Returns
    (best_tokens, best_score, hyps); margins (list) collects the smallest score gaps seen, so a test
    can skip seeds whose decisions are closer than fp32 can resolve.
    alignments=True (the reference's unk_replacement_mode__): every token carries the attention
    weights over the source positions of the step that produced it; the coverage penalty is computed
    from them and a fourth result holds, per 1-best token, the source position of the largest
    weight (-1 if none is positive).
    ensemble: parameter sets of further models of the same shape (EnsembleFactory with several
    models): the step's distribution is the mean of the models' distributions, a token's alignment
    weights are the sum of the models' weights."""
    if ensemble:
        return _beam_decode_ensemble([P] + list(ensemble), layers, H, V, src_ids, beam, D, attention,
                                     feed_input, max_ratio, min_ratio, penalty, diversity, lp_alpha,
                                     cp_beta, longest, margins, alignments)
    return _beam_decode_ensemble([P], layers, H, V, src_ids, beam, D, attention, feed_input,
                                 max_ratio, min_ratio, penalty, diversity, lp_alpha, cp_beta, longest,
                                 margins, alignments)


def _beam_decode_ensemble(Ps, layers, H, V, src_ids, beam, D, attention, feed_input, max_ratio,
                          min_ratio, penalty, diversity, lp_alpha, cp_beta, longest, margins,
                          alignments):
    S = len(src_ids)
    beam = min(beam, int(np.sqrt(V)))
    M = len(Ps)
    enc = [encode(P, layers, H, src_ids) for P in Ps]
    hs = [[np.repeat(enc[k][0][l], beam, axis=1) for l in range(layers)] for k in range(M)]
    cs = [[np.repeat(enc[k][1][l], beam, axis=1) for l in range(layers)] for k in range(M)]
    h_tilds = [np.zeros((H, beam)) for _ in range(M)]
    tokens = np.zeros(beam, int)
    scores = np.zeros(beam)
    hist = [[0] for _ in range(beam)]
    ahist = [[] for _ in range(beam)]  # per token: dict source position -> attention weight
    hyps, hyp_align = [], []
    ones = np.ones(beam, int)
    limit = min(int(np.float32(max_ratio) * S), longest - 2)

    def forward_one(k, step):
        P, top = Ps[k], enc[k][2]
        x = P["tgt.0.W"].astype(np.float64)[:, tokens]
        nh, nc = [], []
        for l in range(layers):
            ht = h_tilds[k] if (l == 0 and feed_input and attention and step != 0) else None
            a, b_, _ = lstm_step(P, f"tgt.{l}.", x, hs[k][l], cs[k][l], ht)
            nh.append(a)
            nc.append(b_)
            x = a
        topv = x
        ht_new, al = None, [{} for _ in range(beam)]
        if attention:
            ht_new, al = attention_local_p(P, topv, lambda b, s: top[s], [S] * beam, ones, D)
            topv = ht_new
        lp = log_softmax(P["softmax.D"].astype(np.float64) @ topv + P["softmax.b_d"].astype(np.float64)[:, None])
        return nh, nc, ht_new, lp, al

    def forward(step):
        outs = [forward_one(k, step) for k in range(M)]
        if M == 1:
            lp, al = outs[0][3], outs[0][4]
        else:
            lp = np.log(np.mean([np.exp(o[3]) for o in outs], axis=0))
            al = [{} for _ in range(beam)]
            for o in outs:
                for b in range(beam):
                    for pos, a in o[4][b].items():
                        al[b][pos] = al[b].get(pos, 0.0) + a
        return [o[0] for o in outs], [o[1] for o in outs], [o[2] for o in outs], lp, al

    for step in range(limit):
        nh, nc, ht_new, lp, al = forward(step)
        cands = []
        for i in range(1 if step == 0 else beam):
            order = np.lexsort((np.arange(V), -lp[:, i]))[: beam + 1]
            if margins is not None:
                full = np.sort(lp[:, i])[::-1]
                margins.append(full[beam] - full[beam + 1])
            for rank, v in enumerate(order):
                cands.append((lp[v, i] + scores[i] - (rank + 1) * diversity, i, int(v)))
        cands.sort(key=lambda t: (-t[0], t[1], t[2]))
        if margins is not None:
            sc = np.array([t[0] for t in cands])
            margins.append(np.min(sc[:-1] - sc[1:]))
        new_tok, new_bp, new_sc = [], [], []
        for s_, i, v in cands:
            if len(new_tok) == beam:
                break
            if v == 0:
                continue
            if v == 1:
                hyps.append((hist[i] + [1], s_ + penalty))
                hyp_align.append(ahist[i] + [al[i]])
                continue
            new_tok.append(v)
            new_bp.append(i)
            new_sc.append(s_ + penalty)
        assert len(new_tok) == beam
        hist = [hist[i] + [v] for i, v in zip(new_bp, new_tok)]
        ahist = [ahist[i] + [al[i]] for i in new_bp]
        tokens = np.array(new_tok)
        scores = np.array(new_sc)
        for k in range(M):
            hs[k] = [x[:, new_bp] for x in nh[k]]
            cs[k] = [x[:, new_bp] for x in nc[k]]
            if attention:
                h_tilds[k] = ht_new[k][:, new_bp]
    _, _, _, lp, al = forward(limit if limit > 0 else 1)
    for i in range(beam):
        hyps.append((hist[i] + [1], scores[i] + lp[1, i] + penalty))
        hyp_align.append(ahist[i] + [al[i]])

    best, best_s, best_al = None, None, None
    for (toks, s_), al_h in zip(hyps, hyp_align):
        n = len(toks)
        r = s_
        if lp_alpha != 0:
            r = r / (((5.0 + n) ** lp_alpha) / (6.0 ** lp_alpha))
        if cp_beta != 0 and alignments:
            # rows = the n-2 real tokens (al_h[j] belongs to token j+1; <EOF>'s row is left out),
            # smoothed by 0.01 and normalised over the source; coverage = capped column sums
            rows = np.zeros((max(n - 2, 0), S))
            for j in range(n - 2):
                for pos, a in al_h[j].items():
                    rows[j, pos] = a
            rows = rows + 0.01
            rows = rows / rows.sum(axis=1, keepdims=True) if n > 2 else rows
            cp = cp_beta * np.sum(np.log(np.minimum(rows.sum(axis=0), 1.0))) if n > 2 else -np.inf
            r = r + max(cp, -20.0)
        elif cp_beta != 0:
            cp = cp_beta * S * np.log(min((n - 2) / S, 1.0)) if n > 2 else -np.inf
            r = r + max(cp, -20.0)
        if n / S > min_ratio and (best is None or r > best_s):
            best, best_s, best_al = toks, r, al_h
    if alignments:
        vit = []
        for j in range(len(best) - 2 if best is not None else 0):
            pos = sorted(best_al[j].items())
            top_a = max([a for _, a in pos], default=0.0)
            vit.append(next((p for p, a in pos if a == top_a), -1) if top_a > 0 else -1)
        return (best[1:-1] if best is not None else []), best_s, hyps, vit
    return (best[1:-1] if best is not None else []), best_s, hyps


def minibatch_loglik(P, layers, H, D, sents, attention=True, feed_input=True, drop=None):
    """Teacher-forced sum of log p(target) over a list of (source ids, target ids without
    <START>/<EOF>) sentence pairs, float64, one sentence at a time (no padding involved).
    drop = dict(keep, src_embed (S,B,H), tgt_embed (T,B,H), src_out (L,S,B,H), tgt_out (L,T,B,H)):
    uniform masks indexed by the minibatch's own timestep (source sentences sit right-aligned in
    their S steps); an element is kept when mask < keep and scaled by 1/keep.  Inverted dropout on
    the embeddings and on what each layer hands UP (to the next layer, the attention node, or the
    softmax when there is no attention); the recurrent path and the encoder states read by the
    attention are not dropped."""
    P = {k: np.asarray(v, np.float64) for k, v in P.items()}
    total = 0.0
    S_max = max(len(s) for s, _ in sents)

    def dr(x, mask):
        if drop is None:
            return x
        return x * ((mask < drop["keep"]) / drop["keep"])[:, None]

    for b, (s, t) in enumerate(sents):
        if drop is None:
            he, ce, top = encode(P, layers, H, s)
        else:
            S = len(s)
            he = [np.zeros((H, 1)) for _ in range(layers)]
            ce = [np.zeros((H, 1)) for _ in range(layers)]
            top = {}
            for k in range(S):
                pos, step = S - 1 - k, S_max - S + k
                x = dr(P["src.0.W"][:, [int(s[pos])]], drop["src_embed"][step, b])
                for l in range(layers):
                    he[l], ce[l], _ = lstm_step(P, f"src.{l}.", x, he[l], ce[l])
                    x = dr(he[l], drop["src_out"][l, step, b])
                top[pos] = he[layers - 1][:, 0].copy()
        h, c = [x.copy() for x in he], [x.copy() for x in ce]
        h_tild = None
        for step, (wi, wo) in enumerate(zip(np.concatenate([[0], t]), np.concatenate([t, [1]]))):
            x = P["tgt.0.W"][:, [int(wi)]]
            if drop is not None:
                x = dr(x, drop["tgt_embed"][step, b])
            for l in range(layers):
                ht = h_tild if (l == 0 and step != 0 and attention and feed_input) else None
                h[l], c[l], _ = lstm_step(P, f"tgt.{l}.", x, h[l], c[l], ht)
                x = h[l] if drop is None else dr(h[l], drop["tgt_out"][l, step, b])
            if attention:
                h_tild, _ = attention_local_p(P, x, lambda _b, pos: top[pos], [len(s)], [1], D)
                x = h_tild
            lp = log_softmax(P["softmax.D"] @ x + P["softmax.b_d"][:, None])
            total += lp[int(wo), 0]
    return total


def pack_minibatch(sents):
    """Reference minibatch layout (src/file_helper.cc:113-381): source reversed and left-padded,
    target right-padded, -1 padding, batch_info = [len..., S - len...], unique non-pad input ids in
    first-occurrence order."""
    B = len(sents)
    S = max(len(s) for s, _ in sents)
    T = max(len(t) + 1 for _, t in sents)
    src = np.full((B, S), -1, np.int32)
    tin = np.full((B, T), -1, np.int32)
    tout = np.full((B, T), -1, np.int32)
    for b, (s, t) in enumerate(sents):
        src[b, S - len(s):] = np.asarray(s)[::-1]
        tin[b, :len(t) + 1] = np.concatenate([[0], t])
        tout[b, :len(t) + 1] = np.concatenate([t, [1]])
    lens = np.array([len(s) for s, _ in sents])
    bi = np.concatenate([lens, S - lens]).astype(np.int32)

    def uniq(a):
        seen = []
        for v in a.ravel(order="F"):
            if v != -1 and v not in seen:
                seen.append(int(v))
        return np.array(seen, np.int32)

    return src, tin, tout, bi, uniq(src), uniq(tin)

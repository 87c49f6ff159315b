"""Pins the oracle's forward pass (llama_cu.cu:1073-1210) with an independent float64 numpy
LLaMA forward on a tiny model, plus the invariants the KV cache must satisfy."""
import numpy as np
import pytest

import oracle_lib as O

CFG = dict(dim=256, multiple_of=128, n_heads=2, n_layers=2, n_vocab=320)


def np_forward64(model, tokens, eps):
    """Textbook LLaMA forward in float64 (no intermediate rounding); returns logits of the last row."""
    dim, H = model.dim, model.n_heads
    hd = dim // H

    def W(stream, rows, cols):
        w, s = model.tensor(stream, rows, cols)
        if s is None:
            return w.astype(np.float64)
        return (w.astype(np.float64) - 127.5) * np.repeat(s.astype(np.float64), model.qblock, axis=1)

    def norm(x):
        return x / np.sqrt((x ** 2).mean(axis=1, keepdims=True) + eps)

    def rope(x):
        n = x.shape[0]
        z = x.reshape(n, H, hd // 2, 2)
        zc = z[..., 0] + 1j * z[..., 1]
        freq = 1.0 / (10000.0 ** (np.arange(0, hd, 2) / hd))
        zc = zc * np.exp(1j * np.arange(n)[:, None, None] * freq[None, None, :])
        return np.stack([zc.real, zc.imag], axis=-1).reshape(n, dim)

    x = W(1, model.n_vocab, dim)[tokens]
    n = len(tokens)
    for l in range(model.n_layers):
        b = 16 + 16 * l
        h = norm(x)
        q, k, v = rope(h @ W(b, dim, dim).T), rope(h @ W(b + 1, dim, dim).T), h @ W(b + 2, dim, dim).T
        att = np.zeros_like(x)
        for hh in range(H):
            sl = slice(hh * hd, (hh + 1) * hd)
            s = q[:, sl] @ k[:, sl].T / np.sqrt(hd)
            s[np.triu_indices(n, 1)] = -np.inf
            p = np.exp(s - s.max(axis=1, keepdims=True))
            p /= p.sum(axis=1, keepdims=True)
            att[:, sl] = p @ v[:, sl]
        x = x + att @ W(b + 3, dim, dim).T
        h = norm(x)
        a = h @ W(b + 4, model.ffn, dim).T
        g = h @ W(b + 6, model.ffn, dim).T
        x = x + ((a / (1 + np.exp(-a))) * g) @ W(b + 5, dim, model.ffn).T
    return norm(x)[-1] @ W(2, model.n_vocab, dim).T, x


@pytest.mark.parametrize("q_type", [0, 1])
@pytest.mark.parametrize("flavour", [0, 1])
def test_forward_vs_float64(q_type, flavour):
    m = O.Model(**CFG, q_type=q_type, seed=11, weight_std=0.05)
    assert m.ffn == 768  # round_up(256*8//3 = 682, 128)
    ctx = O.Context(m, context_len=32, temperature=0.8, flavour=flavour)
    toks = np.random.default_rng(0).integers(0, CFG["n_vocab"], 9)
    tok, hidden, logits, probs = ctx.next_token(toks, want=True)
    ref_logits, ref_hidden = np_forward64(m, toks, 1e-6)
    assert np.max(np.abs(hidden.astype(np.float64) - ref_hidden)) < 1e-2 * np.max(np.abs(ref_hidden))
    assert np.max(np.abs(logits.astype(np.float64) - ref_logits)) < 1e-2 * np.max(np.abs(ref_logits))
    e = np.exp((ref_logits - ref_logits.max()) / np.float64(np.float32(0.8)))
    assert np.max(np.abs(probs.astype(np.float64) - e / e.sum())) < 2e-2 * (e / e.sum()).max()
    assert tok == O.argmax_first(probs)
    assert ctx.start_pos == 9


@pytest.mark.parametrize("q_type", [0, 1])
def test_prefill_then_decode_equals_longer_prefill(q_type):
    m = O.Model(**CFG, q_type=q_type, seed=5, weight_std=0.05)
    toks = np.random.default_rng(1).integers(0, CFG["n_vocab"], 12)
    a = O.Context(m, context_len=16)
    a.next_token(toks[:7])
    a.next_token(toks[7:11])
    ta, ha, la, pa = a.next_token(toks[11:], want=True)
    b = O.Context(m, context_len=16)
    tb, hb, lb, pb = b.next_token(toks, want=True)
    # every op in the oracle is row-independent with a fixed summation order, so this is bit-exact
    assert ta == tb
    assert (la.view(np.uint16) == lb.view(np.uint16)).all()
    assert (ha[-1].view(np.uint16) == hb[-1].view(np.uint16)).all()
    ka, va = a.kv(1, 12)
    kb, vb = b.kv(1, 12)
    assert (ka.view(np.uint16) == kb.view(np.uint16)).all() and (va.view(np.uint16) == vb.view(np.uint16)).all()


def test_literal_rope_mode_is_bit_identical():
    # llama_cu.cu:1150-1153 keeps K unrotated and re-rotates every cached row per call; rotating
    # once at write time gives the same bits because RoPE depends only on (value, position)
    m = O.Model(**CFG, seed=7, weight_std=0.05)
    toks = np.random.default_rng(2).integers(0, CFG["n_vocab"], 10)
    outs = []
    for literal in (0, 1):
        c = O.Context(m, context_len=16, literal_rope=literal)
        c.next_token(toks[:6])
        for t in toks[6:9]:
            c.next_token([t])
        outs.append(c.next_token(toks[9:], want=True) + c.kv(0, 10))
    for x, y in zip(outs[0][1:], outs[1][1:]):
        assert (x.view(np.uint16) == y.view(np.uint16)).all()
    assert outs[0][0] == outs[1][0]


def test_clear_and_overflow():
    m = O.Model(**CFG, seed=7)
    c = O.Context(m, context_len=8)
    t1 = c.next_token([1, 2, 3])
    assert c.next_token(list(range(6))) == -1  # 3 + 6 > 8: the reference asserts here
    c.clear()
    assert c.start_pos == 0 and c.next_token([1, 2, 3]) == t1

"""LM head GEMV and device argmax (crates/xabe-cuda/src/kernels/lm_head.rs) against the CPU oracle, following
crates/xabe-engine/tests/lm_head_differential.rs: logits over the whole vocabulary at the reference's gate
(max_abs 5e-5, cosine 1 - 1e-9), argmax exact for every token, batches bit-identical to single tokens, the
device argmax on the reference's case list."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MAX_ABS, MIN_COS = 5e-5, 1.0 - 1e-9   # lm_head_differential.rs:134-139


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _weights(X, oracle, fmt, vocab, hidden, seed):
    """(device tensor in `fmt`, host f32 [vocab][hidden] of the values it encodes)."""
    import torch

    F = X.HeadFormat
    n = vocab * hidden
    if fmt in (F.Q8_0, F.Q6K):
        q = X.ExpertQuant.Q8_0 if fmt == F.Q8_0 else X.ExpertQuant.Q6K
        dev = X.synth_quant(q, seed, n, 0.02)
        torch.cuda.synchronize()
        host = np.empty((vocab, hidden), np.float32)
        raw = dev.cpu().numpy()
        rb = len(raw) // vocab
        step = 8192
        for r0 in range(0, vocab, step):   # chunked: the full head is 2 GB as f32
            r1 = min(vocab, r0 + step)
            host[r0:r1] = oracle.dequantize_row(int(q), raw[r0 * rb:r1 * rb]).reshape(r1 - r0, hidden)
        return dev, host
    f = X.synth_normal_f32(seed, n, 0.02)
    dev = f.to(torch.bfloat16 if fmt == F.Bf16 else torch.float16)
    torch.cuda.synchronize()
    return dev, dev.float().cpu().numpy().reshape(vocab, hidden)


def _check(oracle, got, ref, label):
    r = oracle.compare(got, ref)
    assert np.abs(got - ref).max() <= MAX_ABS and r.cosine_similarity >= MIN_COS, (label, str(r))
    assert int(np.argmax(got)) == oracle.argmax(ref) == oracle.argmax(got), label


def _run(X, k, w, fmt, x, tokens):
    import torch

    g = k.geometry()
    logits = torch.full((g.max_tokens, g.vocab), -7.0, device="cuda")
    k.forward(X.HeadTensor(w, fmt), x, tokens, logits)
    torch.cuda.synchronize()
    return logits.cpu().numpy()


def test_whole_vocabulary_q8_0_one_token_and_a_batch(oracle, X):
    # lm_head_differential.rs:338-446 (one token) and :450-560 (a 5-token batch, bit-identical rows)
    import torch

    g = X.LmHeadGeometry.qwen3_6(8)
    w, host = _weights(X, oracle, X.HeadFormat.Q8_0, g.vocab, g.hidden, 31000)
    k = X.LmHeadKernels(g)
    x = X.synth_normal_f32(31001, g.max_tokens * g.hidden, 1.0).view(g.max_tokens, g.hidden)
    xs = x.cpu().numpy()
    one = _run(X, k, w, X.HeadFormat.Q8_0, x, 1)
    ref0 = oracle.gemv(host, g.vocab, g.hidden, xs[0])
    _check(oracle, one[0], ref0, "1 token")
    assert np.all(one[1:] == -7.0)            # rows past `tokens` are not written
    five = _run(X, k, w, X.HeadFormat.Q8_0, x, 5)
    assert np.array_equal(five[0].view(np.uint32), one[0].view(np.uint32))   # same bits alone and in a batch
    picks = []
    for t in range(1, 5):
        _check(oracle, five[t], oracle.gemv(host, g.vocab, g.hidden, xs[t]), f"token {t}")
        picks.append(int(np.argmax(five[t])))
    assert len(set(picks)) > 1                # distinct hidden states give distinct argmaxes
    assert np.all(five[5:] == -7.0)
    # every batch width gives every token the same bits (tiles of 1, 2 and 4, two passes at 5..8)
    eight = _run(X, k, w, X.HeadFormat.Q8_0, x, 8)
    for tokens in (2, 3, 4, 7):
        out = _run(X, k, w, X.HeadFormat.Q8_0, x, tokens)
        assert np.array_equal(out[:tokens].view(np.uint32), eight[:tokens].view(np.uint32)), tokens
    assert np.array_equal(five[:5].view(np.uint32), eight[:5].view(np.uint32))
    # device argmax over the device logits
    dl = torch.from_numpy(eight).cuda()
    pv, pi, out = torch.zeros(512, device="cuda"), torch.zeros(512, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    for t in range(8):
        k.argmax(dl[t], g.vocab, pv, pi, out)
        assert int(out.item()) == oracle.argmax(eight[t])


@pytest.mark.parametrize("fmt", ["Q8_0", "Q6K", "Bf16", "F16"])
@pytest.mark.parametrize("vocab,hidden,max_tokens,tokens", [(4099, 2048, 6, 5), (1000, 512, 3, 3), (777, 1024, 2, 1),
                                                            (513, 1536, 4, 4), (300, 5120, 5, 5), (64, 4096, 1, 1)])
def test_formats_and_shapes(oracle, X, fmt, vocab, hidden, max_tokens, tokens):
    # lm_head_formats_differential.rs: every format, ragged vocabularies, rows of one step and of several
    fmt = getattr(X.HeadFormat, fmt)
    g = X.LmHeadGeometry(hidden, vocab, max_tokens)
    # Q6_K at (777, 1024) and (513, 1536) ends 8 and 12 bytes into a 16-byte piece: the last row goes through the bounded loader
    w, host = _weights(X, oracle, fmt, vocab, hidden, 32000 + vocab)
    k = X.LmHeadKernels(g)
    x = X.synth_normal_f32(32001, max_tokens * hidden, 1.0).view(max_tokens, hidden)
    got = _run(X, k, w, fmt, x, tokens)
    xs = x.cpu().numpy()
    for t in range(tokens):
        _check(oracle, got[t], oracle.gemv(host, vocab, hidden, xs[t]), (str(fmt), t))
    assert np.all(got[tokens:] == -7.0)
    alone = _run(X, k, w, fmt, x, 1)
    assert np.array_equal(alone[0].view(np.uint32), got[0].view(np.uint32))


def test_forward_error_paths(oracle, X):
    import torch

    g = X.LmHeadGeometry(512, 64, 4)
    k = X.LmHeadKernels(g)
    F = X.HeadFormat
    w = X.synth_quant(X.ExpertQuant.Q8_0, 5, 64 * 512, 0.02)
    x = torch.zeros(4, 512, device="cuda")
    logits = torch.zeros(4, 64, device="cuda")
    k.forward(X.HeadTensor.q8_0(w), x, 4, logits)
    with pytest.raises(X.moe.RaggedWeights, match="not a whole number of 34 B blocks"):
        k.forward(X.HeadTensor.q8_0(w[:-1]), x, 1, logits)
    with pytest.raises(X.moe.WrongElementCount, match="expected 32768 elements"):
        k.forward(X.HeadTensor.q8_0(w[:-34 * 16]), x, 1, logits)
    with pytest.raises(X.moe.WrongElementCount):
        k.forward(X.HeadTensor.bf16(w), x, 1, logits)         # 34816 bytes read as bf16 is 17408 elements
    for tokens in (0, 5):
        with pytest.raises(X.moe.TooManyTokens, match="outside 1..=4"):
            k.forward(X.HeadTensor.q8_0(w), x, tokens, logits)
    with pytest.raises(X.gguf.ShapeMismatch, match="hidden states: expected 2048 elements, got 1536"):
        k.forward(X.HeadTensor.q8_0(w), x[:3], 1, logits)
    with pytest.raises(X.gguf.ShapeMismatch, match="logits: expected 256 elements"):
        k.forward(X.HeadTensor.q8_0(w), x, 1, logits[:2])
    with pytest.raises(X.moe.UnsupportedExpertType):
        k.forward(X.HeadTensor(w, F.Q4K), x, 1, logits)
    torch.cuda.synchronize()


def test_device_argmax_agrees_with_the_scalar_reference(oracle, X):
    # lm_head_differential.rs:765-833: the same case list
    import torch

    g = X.LmHeadGeometry.qwen3_6(1)
    k = X.LmHeadKernels(g)
    rng = oracle.Xorshift64Star(0x5EED_A46E_A700_0001)
    cases = [(f"random n={n}", rng.vec_f32(n, -8.0, 8.0)) for n in (1, 2, 31, 255, 256, 257, 1023, 4096, 131073, g.vocab)]
    cases.append(("all equal", np.full(g.vocab, 0.5, np.float32)))
    cases.append(("all zero", np.zeros(g.vocab, np.float32)))
    cases.append(("all NaN", np.full(4096, np.nan, np.float32)))
    tied = rng.vec_f32(g.vocab, -1.0, 1.0); tied[7] = 9.0; tied[g.vocab - 3] = 9.0
    cases.append(("tie across partitions", tied))
    last = rng.vec_f32(g.vocab, -1.0, 1.0); last[-1] = 100.0
    cases.append(("max at the end", last))
    first = rng.vec_f32(g.vocab, -1.0, 1.0); first[0] = 100.0
    cases.append(("max at index 0", first))
    infs = rng.vec_f32(g.vocab, -1.0, 1.0); infs[11] = -np.inf; infs[g.vocab // 2] = np.inf
    cases.append(("with infinities", infs))
    nan0 = rng.vec_f32(5000, -1.0, 1.0); nan0[0] = np.nan
    cases.append(("NaN at index 0", nan0))
    nans = rng.vec_f32(5000, -1.0, 1.0); nans[1::3] = np.nan
    cases.append(("NaNs among the values", nans))
    cases.append(("all -inf", np.full(777, -np.inf, np.float32)))
    pv, pi = torch.zeros(512, device="cuda"), torch.zeros(512, dtype=torch.int32, device="cuda")
    out = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    for label, v in cases:
        d = torch.from_numpy(np.ascontiguousarray(v)).cuda()
        k.argmax(d, len(v), pv, pi, out)
        assert int(out.item()) == oracle.argmax(v), label
    # a prefix of a longer buffer
    d = torch.from_numpy(np.ascontiguousarray(last)).cuda()
    k.argmax(d, 1000, pv, pi, out)
    assert int(out.item()) == oracle.argmax(last[:1000])
    with pytest.raises(X.gguf.ShapeMismatch, match="argmax length"):
        k.argmax(d, 0, pv, pi, out)
    with pytest.raises(X.gguf.ShapeMismatch, match="argmax partial values"):
        k.argmax(d, 10, pv[:100], pi, out)


def test_argmax_prob(oracle, X):
    # lm_head.rs:2012-2044: 1 / sum(exp(x - max)), against float64
    import torch

    k = X.LmHeadKernels(X.LmHeadGeometry.qwen3_6(1))
    rng = np.random.default_rng(3)
    out = torch.zeros(1, device="cuda")
    for n, scale in ((1, 1.0), (100, 3.0), (4097, 1.0), (248320, 2.0)):
        v = (rng.standard_normal(n) * scale).astype(np.float32)
        k.argmax_prob(torch.from_numpy(v).cuda(), n, out)
        want = 1.0 / np.exp(v.astype(np.float64) - v.max()).sum()
        assert abs(out.item() - want) <= 2e-6 * want, (n, out.item(), want)

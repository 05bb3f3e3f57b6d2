"""Where weight stacks may start.  Blocks are 210 and 34 bytes long, so inside a stack they sit at every even
offset; the stack itself must start on a 16-byte boundary (include/xabe_hip.h, `xabe_quant_tensor`).  Every
regime gives the same bits for the same bytes at any such start, and refuses a start off the boundary loudly
instead of reading it some other way (the reference's stacks are whole `CudaSlice<u8>` allocations,
crates/xabe-cuda/src/kernels/moe.rs:448-464)."""
import pytest

from util import activations, make_layer

pytestmark = pytest.mark.gpu


def _shifted(torch, t, off):
    """The same bytes (or floats), starting `off` bytes into a fresh allocation."""
    raw = t.view(torch.uint8) if t.dtype != torch.uint8 else t
    buf = torch.zeros(raw.numel() + 256, dtype=torch.uint8, device=t.device)
    view = buf[off:off + raw.numel()]
    view.copy_(raw.reshape(-1))
    assert view.data_ptr() % 256 == off and view.is_contiguous()
    return view if t.dtype == torch.uint8 else view.view(t.dtype).view(t.shape)


def _shift_layer(torch, X, w, off, which=None):
    q = lambda name, qt: X.QuantTensor(_shifted(torch, qt.bytes, off), qt.quant) if which in (None, name) else qt
    router = _shifted(torch, w.router, off) if which in (None, "router") else w.router
    return X.MoeLayerWeights(w.post_norm, router, w.router_quant, q("gate", w.gate_exps), q("up", w.up_exps),
                             q("down", w.down_exps), w.shared_gate_inp, q("shared_gate", w.shared_gate),
                             q("shared_up", w.shared_up), q("shared_down", w.shared_down))


REGIMES = [(3, 3), (12, 11), (32, 29), (40, 37), (128, 100)]   # decode block (two format mixes, widest), dispatch table, matrix cores


def _layer(oracle, X, max_tokens):
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(max_tokens), max_tokens)
    # the shipped mix at 12 tokens: Q8_0 down stacks, fp32 router
    return g, make_layer(oracle, g, seed=9100 + max_tokens, router_q8=(max_tokens != 12),
                         down_quant=X.ExpertQuant.Q8_0 if max_tokens == 12 else None)


@pytest.mark.parametrize("max_tokens,tokens", REGIMES)
@pytest.mark.parametrize("off", [16, 48, 208])
def test_moe_block_is_the_same_bits_wherever_the_stacks_start(oracle, max_tokens, tokens, off):
    import torch
    import llmxabe_amd as X

    g, layer = _layer(oracle, X, max_tokens)
    x = activations(9101, max_tokens, 2048, tokens)
    blk = X.MoeBlock(g)
    out = []
    for w in (layer.dev, _shift_layer(torch, X, layer.dev, off)):
        ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
        blk.forward(w, x, tokens, ffn, lout)
        torch.cuda.synchronize()
        out.append((ffn[:tokens].view(torch.int32).clone(), lout[:tokens].view(torch.int32).clone(),
                    blk.buffers().topk_ids().clone()))
    for a, b, what in zip(out[0], out[1], ("ffn_out", "l_out", "topk_ids")):
        assert torch.equal(a, b), f"{what} differs with the stacks {off} bytes into their allocation"


@pytest.mark.parametrize("max_tokens,tokens", REGIMES)
@pytest.mark.parametrize("which", ["gate", "down", "shared_up", "router"])
def test_a_stack_off_the_16_byte_boundary_is_refused(oracle, max_tokens, tokens, which):
    import torch
    import llmxabe_amd as X

    g, layer = _layer(oracle, X, max_tokens)
    x = activations(9101, max_tokens, 2048, tokens)
    blk = X.MoeBlock(g)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    off = 4 if which == "router" else 2   # (an fp32 router cannot start off a float)
    with pytest.raises(X.moe.InvalidArgument, match="16-byte"):
        blk.forward(_shift_layer(torch, X, layer.dev, off, which), x, tokens, ffn, lout)
    torch.cuda.synchronize()
    assert not ffn.any() and not lout.any()   # nothing was launched


@pytest.mark.parametrize("tokens", [1, 2])
def test_dense_block_is_the_same_bits_wherever_the_matrices_start(tokens):
    import torch
    import llmxabe_amd as X

    H, I = 4096, 4096
    q = X.ExpertQuant.Q6K
    t = [X.synth_quant(q, 71 + j, H * I, 0.02) for j in range(3)]
    norm = 1.0 + X.synth_normal_f32(70, H, 0.1)
    x = X.synth_normal_f32(75, tokens * H, 1.0).view(tokens, H)
    blk = X.DenseFfnBlock(H, I, tokens)
    out = []
    for off in (0, 16, 112):
        w = X.DenseFfnLayerWeights(norm, *[X.QuantTensor(_shifted(torch, b, off), q) for b in t])
        ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
        blk.forward(w, x, tokens, ffn, lout)
        torch.cuda.synchronize()
        out.append((ffn.view(torch.int32).clone(), lout.view(torch.int32).clone()))
    for o in out[1:]:
        assert torch.equal(out[0][0], o[0]) and torch.equal(out[0][1], o[1])
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    w = X.DenseFfnLayerWeights(norm, X.QuantTensor(_shifted(torch, t[0], 2), q), X.QuantTensor(t[1], q), X.QuantTensor(t[2], q))
    with pytest.raises(X.moe.InvalidArgument, match="16-byte"):
        blk.forward(w, x, tokens, ffn, lout)


@pytest.mark.parametrize("max_tokens,tokens", REGIMES)
def test_a_short_or_ragged_stack_is_refused_at_every_width(oracle, max_tokens, tokens):
    """The block-level entry point makes the stack checks of `grouped_forward_partial` / `shared_expert`
    (crates/xabe-cuda/src/kernels/moe.rs:6729-6746) whichever launches it goes on to issue: a stack one expert
    short is a wrong element count, one cut inside a block is ragged; nothing is launched."""
    import torch
    import llmxabe_amd as X

    g, layer = _layer(oracle, X, max_tokens)
    w = layer.dev
    x = activations(9101, max_tokens, 2048, tokens)
    blk = X.MoeBlock(g)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    one_expert = w.gate_exps.bytes.numel() // g.num_experts
    import dataclasses
    short = dataclasses.replace(w, gate_exps=X.QuantTensor(w.gate_exps.bytes[:-one_expert], w.gate_exps.quant))
    with pytest.raises(X.moe.WrongElementCount):
        blk.forward(short, x, tokens, ffn, lout)
    ragged = dataclasses.replace(w, shared_down=X.QuantTensor(w.shared_down.bytes[:-2], w.shared_down.quant))
    with pytest.raises(X.moe.RaggedWeights):
        blk.forward(ragged, x, tokens, ffn, lout)
    torch.cuda.synchronize()
    assert not ffn.any() and not lout.any()

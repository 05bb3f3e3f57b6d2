"""Layer upload from a GGUF file (crates/xabe-engine/src/block/moe.rs:660-892, dense_ffn.rs:663-760): the block
run on tensors uploaded from a file equals, bit for bit, the block run on the same tensors handed over
directly, for the shipped per-tensor layouts (gate/up Q6_K, down Q8_0, f32 router; all-Q8_0 with bf16 router and
shared-gate vectors) and against the CPU oracle; the upload's own checks (missing tensor, shape, dense and
expert types) answer with the reference's error variants."""
import numpy as np
import pytest

import gguf_build as G
from gguf_build import GgufWriter
from util import activations, rel_to_peak

pytestmark = pytest.mark.gpu

GGML = {0: G.Q6K, 1: G.Q8_0}   # ExpertQuant -> ggml type id


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _bf16_round(t):
    import torch
    return t.to(torch.bfloat16)


def _layer_tensors(X, g, seed, eq, dq, sq, sdq, bf16_router):
    """Device tensors of one layer, plus the bytes each takes in a file."""
    import torch

    E, H, I = g.num_experts, g.hidden, g.intermediate
    q = lambda quant, s, n: X.synth_quant(quant, seed + s, n, 0.02)
    t = dict(gate=q(eq, 1, E * I * H), up=q(eq, 2, E * I * H), down=q(dq, 3, E * I * H),
             sgate=q(sq, 4, I * H), sup=q(sq, 5, I * H), sdown=q(sdq, 6, I * H),
             post_norm=1.0 + X.synth_normal_f32(seed + 7, H, 0.1), router=X.synth_normal_f32(seed + 8, E * H, 0.02),
             sgi=X.synth_normal_f32(seed + 9, H, 0.02))
    if bf16_router:   # the file holds bf16: the values the block sees are the widened ones
        t["router_file"], t["sgi_file"] = _bf16_round(t["router"]), _bf16_round(t["sgi"])
        t["router"], t["sgi"] = t["router_file"].float(), t["sgi_file"].float()
    torch.cuda.synchronize()
    return t


def _raw(t):
    import torch
    return t.contiguous().view(torch.uint8).cpu().numpy().tobytes()


def _add_moe_layer(w, X, g, layer, t, eq, dq, sq, sdq, bf16_router):
    E, H, I = g.num_experts, g.hidden, g.intermediate
    p = f"blk.{layer}."
    w.tensor(p + "attn_norm.weight", [H], G.F32)            # a neighbour the upload must not touch
    w.tensor(p + "post_attention_norm.weight", [H], G.F32, _raw(t["post_norm"]))
    if bf16_router:
        w.tensor(p + "ffn_gate_inp.weight", [H, E], G.BF16, _raw(t["router_file"]))
        w.tensor(p + "ffn_gate_inp_shexp.weight", [H], G.BF16, _raw(t["sgi_file"]))
    else:
        w.tensor(p + "ffn_gate_inp.weight", [H, E], G.F32, _raw(t["router"]))
        w.tensor(p + "ffn_gate_inp_shexp.weight", [H], G.F32, _raw(t["sgi"]))
    w.tensor(p + "ffn_gate_exps.weight", [H, I, E], GGML[int(eq)], _raw(t["gate"]))
    w.tensor(p + "ffn_up_exps.weight", [H, I, E], GGML[int(eq)], _raw(t["up"]))
    w.tensor(p + "ffn_down_exps.weight", [I, H, E], GGML[int(dq)], _raw(t["down"]))
    w.tensor(p + "ffn_gate_shexp.weight", [H, I], GGML[int(sq)], _raw(t["sgate"]))
    w.tensor(p + "ffn_up_shexp.weight", [H, I], GGML[int(sq)], _raw(t["sup"]))
    w.tensor(p + "ffn_down_shexp.weight", [I, H], GGML[int(sdq)], _raw(t["sdown"]))


def _direct(X, t, eq, dq, sq, sdq):
    return X.MoeLayerWeights(t["post_norm"], t["router"], None, X.QuantTensor(t["gate"], eq), X.QuantTensor(t["up"], eq),
                             X.QuantTensor(t["down"], dq), t["sgi"], X.QuantTensor(t["sgate"], sq),
                             X.QuantTensor(t["sup"], sq), X.QuantTensor(t["sdown"], sdq))


def _forward(X, g, w, x, tokens):
    import torch

    blk = X.MoeBlock(g)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    blk.forward(w, x, tokens, ffn, lout)
    torch.cuda.synchronize()
    ids = blk.buffers().topk_ids().view(g.max_tokens, g.experts_per_token)[:tokens].cpu().numpy()
    logits = blk.router_logits().view(g.max_tokens, g.num_experts)[:tokens].cpu().numpy()
    return ffn.cpu().numpy(), lout.cpu().numpy(), ids, logits


LAYOUTS = {  # gate/up, down, shared gate/up, shared down, bf16 router
    "shipped": ("Q6K", "Q8_0", "Q8_0", "Q8_0", False),      # block/moe.rs:53-73: blocks 0..38
    "all_q8_0_bf16_router": ("Q8_0", "Q8_0", "Q8_0", "Q8_0", True),  # the last blocks of the shipped file
    "all_q6k": ("Q6K", "Q6K", "Q6K", "Q6K", False),
}


@pytest.mark.parametrize("max_tokens,tokens", [(3, 3), (32, 20), (96, 96)])
def test_small_geometry_two_layers_from_one_file(oracle, X, tmp_path, max_tokens, tokens):
    g = X.MoeGeometry(8, 2, 512, 256, 32, max_tokens)
    q = lambda n: getattr(X.ExpertQuant, n)
    w = GgufWriter().kv("general.architecture", G.T_STRING, "qwen35moe")
    layers = {}
    for layer, name in ((0, "shipped"), (1, "all_q8_0_bf16_router"), (5, "all_q6k")):
        eq, dq, sq, sdq, bf = LAYOUTS[name]
        t = _layer_tensors(X, g, 9000 + 50 * layer, q(eq), q(dq), q(sq), q(sdq), bf)
        _add_moe_layer(w, X, g, layer, t, q(eq), q(dq), q(sq), q(sdq), bf)
        layers[layer] = (t, q(eq), q(dq), q(sq), q(sdq), bf)
    path = tmp_path / "two_layers.gguf"
    path.write_bytes(w.build())
    f = X.GgufFile.open(path)
    x = activations(9100, max_tokens, g.hidden, tokens)
    for layer, (t, eq, dq, sq, sdq, bf) in layers.items():
        up = X.UploadedMoeLayer.upload(f, layer, g)
        assert up.layer() == layer and up.expert_quants() == [eq, eq, dq] and up.shared_quants() == [sq, sq, sdq]
        assert up.router_types() == ((X.GgmlType.Bf16,) * 2 if bf else (X.GgmlType.F32,) * 2)
        E, H, I = g.num_experts, g.hidden, g.intermediate
        assert up.bytes() == (H + E * H + H) * 4 + sum(int(t[k].numel()) for k in ("gate", "up", "down", "sgate", "sup", "sdown"))
        a = _forward(X, g, up, x, tokens)
        b = _forward(X, g, _direct(X, t, eq, dq, sq, sdq), x, tokens)
        for u, v in zip(a, b):
            assert np.array_equal(u.view(np.uint32) if u.dtype == np.float32 else u, v.view(np.uint32) if v.dtype == np.float32 else v)
        # and against the oracle on the file's values
        c = lambda k: t[k].cpu().numpy()
        host = oracle.MoeWeights(num_experts=E, top_k=g.experts_per_token, hidden=H, intermediate=I, eps=1e-6,
                                 post_norm=c("post_norm"), router_f32=c("router"), router_q8=None, gate_exps=c("gate"),
                                 up_exps=c("up"), down_exps=c("down"), shared_gate_inp=c("sgi"), shared_gate=c("sgate"),
                                 shared_up=c("sup"), shared_down=c("sdown"), gate_quant=int(eq), up_quant=int(eq),
                                 down_quant=int(dq), sgate_quant=int(sq), sup_quant=int(sq), sdown_quant=int(sdq))
        ref = oracle.moe_block_forward(host, x[:tokens].cpu().numpy(), logits_override=a[3], threads=8)
        assert np.array_equal(a[2], ref.topk_ids.astype(np.int32))
        tol = 2e-5 if max_tokens < 64 else 2e-3   # fp32 regimes / fp16 matrix-core regime
        assert rel_to_peak(a[1][:tokens], ref.l_out) <= tol
    f.close()


def test_model_geometry_shipped_layer_through_a_mapped_file(oracle, X, tmp_path):
    """One layer at the model's shapes (725 MB of expert bytes) in the shipped layout, read through the mapping."""
    import torch

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(3), 3)
    q = X.ExpertQuant
    t = _layer_tensors(X, g, 9500, q.Q6K, q.Q8_0, q.Q8_0, q.Q8_0, False)
    w = GgufWriter().kv("general.architecture", G.T_STRING, "qwen35moe")
    _add_moe_layer(w, X, g, 17, t, q.Q6K, q.Q8_0, q.Q8_0, q.Q8_0, False)
    path = tmp_path / "layer17.gguf"
    path.write_bytes(w.build())
    f = X.GgufFile.open(path)
    assert f.tensor("blk.17.ffn_down_exps.weight").n_bytes == 256 * 512 * 2048 // 32 * 34
    up = X.UploadedMoeLayer.upload(f, 17, g)
    f.close()   # the device copies do not depend on the mapping
    x = activations(9510, 3, 2048)
    a = _forward(X, g, up, x, 3)
    b = _forward(X, g, _direct(X, t, q.Q6K, q.Q8_0, q.Q8_0, q.Q8_0), x, 3)
    assert np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32)) and np.array_equal(a[2], b[2])
    assert torch.equal(torch.from_numpy(a[1]), torch.from_numpy(b[1]))


def test_upload_errors(X):
    g = X.MoeGeometry(8, 2, 512, 256, 32, 3)
    E, H, I = 8, 512, 256
    q = X.ExpertQuant
    t = _layer_tensors(X, g, 9700, q.Q8_0, q.Q8_0, q.Q8_0, q.Q8_0, False)

    def build(edit):
        w = GgufWriter()
        _add_moe_layer(w, X, g, 0, t, q.Q8_0, q.Q8_0, q.Q8_0, q.Q8_0, False)
        w.tensors = [e for e in (edit(x) for x in w.tensors) if e is not None]
        return X.GgufFile.from_bytes(w.build())

    def swap(name, **kw):
        def edit(e):
            if e[0] != "blk.0." + name:
                return e
            if kw.get("drop"):
                return None
            return (e[0], kw.get("dims", e[1]), kw.get("ty", e[2]), kw.get("data", e[3]), e[4])
        return edit

    X.UploadedMoeLayer.upload(build(lambda e: e), 0, g)
    with pytest.raises(X.gguf.MissingTensor, match="layer 0 has no `ffn_up_exps.weight`"):
        X.UploadedMoeLayer.upload(build(swap("ffn_up_exps.weight", drop=True)), 0, g)
    with pytest.raises(X.gguf.MissingTensor, match="layer 3 has no"):
        X.UploadedMoeLayer.upload(build(lambda e: e), 3, g)
    with pytest.raises(X.gguf.UnsupportedDenseType, match="ffn_gate_inp.weight` is f16"):
        X.UploadedMoeLayer.upload(build(swap("ffn_gate_inp.weight", ty=G.F16, data=bytes(E * H * 2))), 0, g)
    with pytest.raises(X.moe.UnsupportedExpertType, match="is f32"):
        X.UploadedMoeLayer.upload(build(swap("ffn_down_exps.weight", ty=G.F32, dims=[4], data=bytes(16))), 0, g)
    with pytest.raises(X.moe.UnsupportedExpertType, match="q4_K"):
        X.UploadedMoeLayer.upload(build(swap("ffn_gate_shexp.weight", ty=G.Q4K, data=bytes(I * H // 256 * 144))), 0, g)
    with pytest.raises(X.gguf.ShapeMismatch, match="holds 1024 elements, the geometry implies 512"):
        X.UploadedMoeLayer.upload(build(swap("post_attention_norm.weight", dims=[2 * H], data=bytes(8 * H))), 0, g)
    with pytest.raises(X.gguf.ShapeMismatch, match="ffn_gate_exps.weight"):
        X.UploadedMoeLayer.upload(build(swap("ffn_gate_exps.weight", dims=[H, I, E // 2], data=bytes(E // 2 * I * H // 32 * 34))), 0, g)
    # the right element count in the wrong arrangement is a shape mismatch too (the directory's check)
    with pytest.raises(X.gguf.ShapeMismatch, match=r"dimensions \[256, 512, 8\]"):
        X.UploadedMoeLayer.upload(build(swap("ffn_up_exps.weight", dims=[I, H, E])), 0, g)
    # a geometry that does not describe the file
    with pytest.raises(X.gguf.ShapeMismatch):
        X.UploadedMoeLayer.upload(build(lambda e: e), 0, X.MoeGeometry(16, 2, 512, 256, 32, 3))


def test_dense_layer_from_a_file(oracle, X, tmp_path):
    import torch

    H, I = 1024, 2048
    q = X.ExpertQuant
    for layer, (gq, dq) in enumerate(((q.Q6K, q.Q6K), (q.Q8_0, q.Q8_0), (q.Q6K, q.Q8_0))):
        gate, upw, down = (X.synth_quant(gq, 9800 + layer, H * I, 0.02), X.synth_quant(gq, 9810 + layer, H * I, 0.02),
                           X.synth_quant(dq, 9820 + layer, H * I, 0.02))
        pn = 1.0 + X.synth_normal_f32(9830 + layer, H, 0.1)
        torch.cuda.synchronize()
        p = f"blk.{layer}."
        w = (GgufWriter().tensor(p + "post_attention_norm.weight", [H], G.F32, _raw(pn))
             .tensor(p + "ffn_gate.weight", [H, I], GGML[int(gq)], _raw(gate)).tensor(p + "ffn_up.weight", [H, I], GGML[int(gq)], _raw(upw))
             .tensor(p + "ffn_down.weight", [I, H], GGML[int(dq)], _raw(down)))
        f = X.GgufFile.from_bytes(w.build())
        up = X.UploadedDenseFfnLayer.upload(f, layer, H, I)
        assert up.quants() == [gq, gq, dq] and up.bytes() == H * 4 + gate.numel() + upw.numel() + down.numel()
        direct = X.DenseFfnLayerWeights(pn, X.QuantTensor(gate, gq), X.QuantTensor(upw, gq), X.QuantTensor(down, dq))
        outs = []
        for weights in (up, direct):
            blk = X.DenseFfnBlock(H, I, 4)
            x = X.synth_normal_f32(9850, 4 * H, 1.0).view(4, H)
            ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
            blk.forward(weights, x, 4, ffn, lout)
            torch.cuda.synchronize()
            outs.append(lout.cpu().numpy())
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
        with pytest.raises(X.gguf.MissingTensor):
            X.UploadedDenseFfnLayer.upload(f, layer + 1, H, I)
        with pytest.raises(X.gguf.ShapeMismatch):
            X.UploadedDenseFfnLayer.upload(f, layer, H, 2 * I)

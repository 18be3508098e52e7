"""Each part alone against the plain implementation's function for it: norm, rotation + attention
over the paged cache, gated feed-forward, block arrangement, embedding and head, at sizes that
differ from the tiny models'."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def setup(dtype):
    from miniserve_amd.loading import runtime

    return runtime(dtype)


def tensor(shape, rt, seed, scale=1.0, offset=0.0):
    g = torch.Generator().manual_seed(seed)
    t = (torch.randn(shape, generator=g) * scale + offset).to(torch.bfloat16)
    return t.to(rt.dtype).to(rt.device)


def f64(t):
    return t.double().cpu().numpy()


def close(got, want, dtype, what):
    got = got.double().cpu().numpy() if isinstance(got, torch.Tensor) else got
    scale = np.abs(want).max()
    tol = 2e-5 if dtype == "float32" else 2e-2
    assert np.abs(got - want).max() <= tol * scale, f"{what}: {np.abs(got - want).max():.3e} > {tol * scale:.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_alone(dtype):
    from miniserve_amd.config import PartSpec
    from miniserve_amd.parts import part_class

    rt = setup(dtype)
    spec = PartSpec("rmsnorm", {"width": 200, "eps": 3e-4, "tensor": "w"})
    norm = part_class("norm", spec)(spec, rt)
    w = tensor((200,), rt, 1, 0.3, 1.0)
    norm.bind({"w": w})
    x = tensor((9, 200), rt, 2, 2.0).float().contiguous()
    close(norm.forward(x), P.rms_norm(f64(x), f64(w), 3e-4), dtype, "norm")
    rows = torch.tensor([8, 3], dtype=torch.int32, device=rt.device)
    close(norm.forward(x, rows=rows), P.rms_norm(f64(x), f64(w), 3e-4)[[8, 3]], dtype, "norm rows")


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_alone(dtype):
    from miniserve_amd.config import PartSpec
    from miniserve_amd.parts import part_class

    rt = setup(dtype)
    spec = PartSpec("gated_mlp", {"prefix": "m.", "hidden_size": 72, "intermediate_size": 200, "activation": "silu"})
    ffn = part_class("feed_forward", spec)(spec, rt)
    ws = {"m.gate_proj.weight": tensor((200, 72), rt, 3, 0.1), "m.up_proj.weight": tensor((200, 72), rt, 4, 0.1),
          "m.down_proj.weight": tensor((72, 200), rt, 5, 0.1)}
    assert set(type(ffn).tensors(spec)) == set(ws)
    ffn.bind(ws)
    for rows in (5, 100):  # the small-M and the tile product
        x = tensor((rows, 72), rt, 6)
        residual = tensor((rows, 72), rt, 7).float().contiguous()
        before = f64(residual)
        pending = ffn.forward(x, residual)
        rt.ops.add_pending(residual, pending)
        want = before + P.swiglu(f64(x), *(f64(ws[k]) for k in ("m.gate_proj.weight", "m.up_proj.weight", "m.down_proj.weight")))
        close(residual, want, dtype, f"feed-forward {rows} rows")
    with pytest.raises(NotImplementedError):
        bad = PartSpec("gated_mlp", {"hidden_size": 8, "intermediate_size": 8, "activation": "gelu"})
        part_class("feed_forward", bad)(bad, rt)
    # the activation is a parameter of the part, not of the architecture: the other one the kernels know
    other = PartSpec("gated_mlp", {"prefix": "m.", "hidden_size": 72, "intermediate_size": 200, "activation": "gelu_tanh"})
    gelu = part_class("feed_forward", other)(other, rt)
    gelu.bind(ws)
    x = tensor((9, 72), rt, 8)
    residual = torch.zeros((9, 72), dtype=torch.float32, device=x.device)
    rt.ops.add_pending(residual, gelu.forward(x, residual))
    g, u = f64(x) @ f64(ws["m.gate_proj.weight"]).T, f64(x) @ f64(ws["m.up_proj.weight"]).T
    tanh_gelu = 0.5 * g * (1 + np.tanh(np.sqrt(2 / np.pi) * (g + 0.044715 * g**3)))
    close(residual, (tanh_gelu * u) @ f64(ws["m.down_proj.weight"]).T, dtype, "feed-forward with the tanh form of GELU")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,d,window,qk_norm,rot", [(6, 2, 32, 0, True, 32), (4, 4, 64, 20, False, 16), (8, 2, 128, 0, True, 128)])
def test_attention_alone(dtype, heads, kv_heads, d, window, qk_norm, rot):
    """The mixer over the real pool, tables and batch: a whole sequence in one step, then the same in
    portions with the last tokens one by one; against the plain layer."""
    from miniserve_amd.cache.manager import CacheLayout, CacheManager
    from miniserve_amd.cache.pool import KVPool
    from miniserve_amd.config import PartSpec
    from miniserve_amd.engine.batch import BatchBuilder, StepRow
    from miniserve_amd.parts import part_class
    from miniserve_amd.parts.model import CacheSlotNeed

    rt = setup(dtype)
    hidden, theta, eps, scale = 96, 5000.0, 1e-5, 0.11
    spec = PartSpec("gqa_attention", {
        "prefix": "a.", "hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": d, "scale": scale,
        "qk_norm_eps": eps if qk_norm else None, "window": window,
        "position": PartSpec("rotary", {"dim": rot, "theta": theta})})
    mixer = part_class("mixer", spec)(spec, rt)
    ws = {"a.q_proj.weight": tensor((heads * d, hidden), rt, 1, 0.1), "a.k_proj.weight": tensor((kv_heads * d, hidden), rt, 2, 0.1),
          "a.v_proj.weight": tensor((kv_heads * d, hidden), rt, 3, 0.1), "a.o_proj.weight": tensor((hidden, heads * d), rt, 4, 0.1)}
    if qk_norm:
        ws["a.q_norm.weight"] = tensor((d,), rt, 5, 0.2, 1.0)
        ws["a.k_norm.weight"] = tensor((d,), rt, 6, 0.2, 1.0)
    assert set(type(mixer).tensors(spec)) == set(ws)
    mixer.bind(ws)
    T = 70
    x = tensor((T, hidden), rt, 7)

    # plain: the layer's formulas with this part's constants
    xd = f64(x)
    q = (xd @ f64(ws["a.q_proj.weight"]).T).reshape(T, heads, d)
    k = (xd @ f64(ws["a.k_proj.weight"]).T).reshape(T, kv_heads, d)
    v = (xd @ f64(ws["a.v_proj.weight"]).T).reshape(T, kv_heads, d)
    if qk_norm:
        q, k = P.rms_norm(q, f64(ws["a.q_norm.weight"]), eps), P.rms_norm(k, f64(ws["a.k_norm.weight"]), eps)
    ang = P.rotary_angles(np.arange(T), rot, theta)
    q = np.concatenate((P.apply_rotary(q[..., :rot], ang), q[..., rot:]), -1)
    k = np.concatenate((P.apply_rotary(k[..., :rot], ang), k[..., rot:]), -1)
    want = P.attention(q, k, v, scale, window).reshape(T, heads * d) @ f64(ws["a.o_proj.weight"]).T

    layout = CacheLayout.from_needs([CacheSlotNeed(0, mixer.kv_need(), None)])
    manager = CacheManager(layout, 16, [8], 2)
    pool = KVPool(layout, 16, [8], 2, rt.dtype, rt.device)
    builder = BatchBuilder(rt.device, 1)
    for cuts in ([T], [33, 30, 1, 1, 1, 1, 1, 1, 1]):
        rc = manager.acquire()
        residual = torch.zeros((T, hidden), dtype=torch.float32, device=rt.device)
        at = 0
        for n in cuts:
            start = rc.num_tokens
            manager.extend(rc, n)
            batch = builder.build([StepRow(rc, [0] * n, [])], [start])
            part = residual[at : at + n]
            pending = mixer.forward(x[at : at + n].contiguous(), batch, pool.view(0, batch, True), None, part)
            rt.ops.add_pending(part, pending)
            manager.advance(rc)
            at += n
        close(residual, want, dtype, f"attention cut {cuts[:3]}")
        manager.release(rc)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_alone(dtype):
    from miniserve_amd.config import PartSpec
    from miniserve_amd.parts import part_class

    rt = setup(dtype)
    e_spec = PartSpec("token_embedding", {"vocab_size": 301, "width": 40, "tensor": "E"})
    emb = part_class("embedding", e_spec)(e_spec, rt)
    table = tensor((301, 40), rt, 1)
    emb.bind({"E": table})
    ids = torch.tensor([300, 0, 7, 7], dtype=torch.int32, device=rt.device)
    out = emb.forward(ids)
    assert out.dtype == torch.float32 and torch.equal(out, table[ids.long()].float())
    for tied in (None, "E"):
        h_spec = PartSpec("linear_head", {"vocab_size": 301, "width": 40, "tensor": "lm", "tied_to": tied})
        head = part_class("head", h_spec)(h_spec, rt)
        w = tensor((301, 40), rt, 2)
        # a tied head declares no tensor of its own but an alias: it is handed the source under its own name
        assert type(head).aliases(h_spec) == ({"lm": "E"} if tied else {})
        assert type(head).tensors(h_spec) == ({} if tied else {"lm": type(head).tensors(h_spec)["lm"]})
        head.bind({"lm": table if tied else w})
        assert (head.weight is table) == (tied is not None)
        x = tensor((3, 40), rt, 3)
        logits = head.forward(x)
        assert logits.dtype == torch.float32
        close(logits, f64(x) @ f64(table if tied else w).T, dtype, "head")

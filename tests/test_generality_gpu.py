"""A toy architecture, defined entirely in this test, is registered, built and stepped without a
change to the framework's files: a mixer with fixed-size per-request state of its own, a run order
that names one layer's weights twice and lets an entry read another entry's cache, and a second
position-free attention layer. Whole prompts, portions, single tokens and captured decode graphs
must all agree with a plain implementation of the same toy, also defined here."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu

H, HEADS, KVH, D, INTER, VOCAB, DECAY = 64, 4, 2, 16, 96, 97, 0.75


@pytest.fixture(scope="module")
def toy():
    from miniserve_amd.config import LayerSpec, ModelSpec, PartSpec, RunEntry, register_architecture, unregister_architecture
    from miniserve_amd.parts import Mixer, StateNeed, TensorSpec, register, unregister

    @register("mixer", "toy_decay")
    class DecayMixer(Mixer):
        """s_t = decay * s_{t-1} + x_t per request (s starts at 0); output = s_t W^T."""

        def __init__(self, spec, rt):
            super().__init__(spec, rt)
            self.width, self.decay = int(spec["width"]), float(spec["decay"])

        @classmethod
        def tensors(cls, spec):
            return {"toy.weight": TensorSpec((int(spec["width"]), int(spec["width"])))}

        def bind(self, tensors):
            self.weight = tensors["toy.weight"]

        def state_need(self):
            return StateNeed((self.width,), "float32")

        def forward(self, x, batch, cache, state, residual):
            xf = x.float()
            slots = batch.state_slots.long()
            if batch.is_decode:  # one token per row: no host loop, capturable in a graph
                s = torch.where(batch.starts[:, None] == 0, torch.zeros_like(xf), state[slots]) * self.decay + xf
                state[slots] = s
                out = s
            else:
                out = torch.empty_like(xf)
                t = 0
                for i, (n, start) in enumerate(zip(batch.row_lens, batch.row_starts_host)):
                    slot = slots[i]
                    s = torch.zeros(self.width, device=xf.device) if start == 0 else state[slot].clone()
                    for j in range(n):
                        s = s * self.decay + xf[t + j]
                        out[t + j] = s
                    state[slot] = s
                    t += n
            return self.rt.ops.linear(out.to(x.dtype).contiguous(), self.weight, accumulate_into=residual, defer=True)

    @register_architecture("ToyForCausalLM")
    class ToyConfig:
        @classmethod
        def from_dict(cls, cfg):
            return cls()

        def to_dict(self):
            return {"architectures": ["ToyForCausalLM"]}

        def to_spec(self):
            def norm(t):
                return PartSpec("rmsnorm", {"width": H, "eps": 1e-5, "tensor": t})

            def block():
                return PartSpec("prenorm", {"mixer_norm": norm("n1.weight"), "ffn_norm": norm("n2.weight")})

            ffn = PartSpec("gated_mlp", {"prefix": "mlp.", "hidden_size": H, "intermediate_size": INTER, "activation": "silu"})
            attn = PartSpec("gqa_attention", {
                "prefix": "attn.", "hidden_size": H, "num_heads": HEADS, "num_kv_heads": KVH, "head_dim": D,
                "scale": 0.3, "qk_norm_eps": None, "window": 0, "position": PartSpec("rotary", {"dim": 8, "theta": 100.0})})
            layers = (
                LayerSpec("l0.", block(), PartSpec("toy_decay", {"width": H, "decay": DECAY}), ffn),
                LayerSpec("l1.", block(), attn, ffn),
            )
            order = (RunEntry(0, 0), RunEntry(1, 1), RunEntry(1, 2), RunEntry(1, 1, writes_cache=False))
            return ModelSpec(
                architecture="ToyForCausalLM", vocab_size=VOCAB, hidden_size=H,
                embedding=PartSpec("token_embedding", {"vocab_size": VOCAB, "width": H, "tensor": "emb.weight"}),
                layers=layers, run_order=order, final_norm=norm("out_norm.weight"),
                head=PartSpec("linear_head", {"vocab_size": VOCAB, "width": H, "tensor": "head.weight", "tied_to": None}))

    yield ToyConfig
    unregister_architecture("ToyForCausalLM")
    unregister("mixer", "toy_decay")


def plain_toy(w, ids):
    """The toy in float64: layer 0 (decay mixer), then layer 1's weights three times: with a cache of
    its own, with another cache of its own, and reading the keys and values of the first of these."""
    w = {k: v.double().cpu().numpy() for k, v in w.items()}
    T = len(ids)
    h = w["emb.weight"][np.asarray(ids)]

    def mlp(h, p):
        y = P.rms_norm(h, w[p + "n2.weight"], 1e-5)
        return h + P.swiglu(y, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    x = P.rms_norm(h, w["l0.n1.weight"], 1e-5)
    s, outs = np.zeros(H), []
    for t in range(T):
        s = DECAY * s + x[t]
        outs.append(s)
    h = mlp(h + np.stack(outs) @ w["l0.toy.weight"].T, "l0.")

    ang = P.rotary_angles(np.arange(T), 8, 100.0)

    def rot(v):  # partial rotation: the first 8 elements of each head
        return np.concatenate((P.apply_rotary(v[..., :8], ang), v[..., 8:]), axis=-1)

    def qkv(h):
        x = P.rms_norm(h, w["l1.n1.weight"], 1e-5)
        q = rot((x @ w["l1.attn.q_proj.weight"].T).reshape(T, HEADS, D))
        k = rot((x @ w["l1.attn.k_proj.weight"].T).reshape(T, KVH, D))
        v = (x @ w["l1.attn.v_proj.weight"].T).reshape(T, KVH, D)
        return q, k, v

    def attend(h, q, k, v):
        o = P.attention(q, k, v, 0.3).reshape(T, HEADS * D)
        return mlp(h + o @ w["l1.attn.o_proj.weight"].T, "l1.")

    q, k1, v1 = qkv(h)
    h = attend(h, q, k1, v1)
    q, k2, v2 = qkv(h)
    h = attend(h, q, k2, v2)
    q, _, _ = qkv(h)
    h = attend(h, q, k1, v1)  # reads what the first of the three stored
    return P.rms_norm(h, w["out_norm.weight"], 1e-5) @ w["head.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_runs_through_the_engine(toy, dtype):
    from miniserve_amd.config import config_from_dict
    from miniserve_amd.engine.batch import StepRow
    from miniserve_amd.engine.runner import ModelRunner
    from miniserve_amd.loading import runtime
    from miniserve_amd.parts import DecoderModel
    from miniserve_amd.weights import Init, random_tensors
    from tolerances import check_logits

    cfg = config_from_dict({"architectures": ["ToyForCausalLM"]})
    spec = cfg.to_spec()
    rt = runtime(dtype)
    weights = random_tensors(spec, 7, Init(0.08, (0.6, 1.4)), dtype=rt.dtype, device=rt.device)
    model = DecoderModel(spec, weights, rt)
    needs = model.cache_slots()
    assert [n.slot for n in needs] == [0, 1, 2] and needs[0].kv is None and needs[0].state.shape == (H,)
    assert needs[1].kv.head_dim == D and needs[1].state is None

    runner = ModelRunner(model, kv_pool_tokens=16 * 12, max_running=4, decode_graph=True)
    assert [g.slots for g in runner.layout.groups] == [(1, 2)] and [s.slot for s in runner.layout.states] == [0]
    rng = np.random.default_rng(3)
    seqs = [rng.integers(0, VOCAB, n).tolist() for n in (37, 50, 9)]
    want = [plain_toy(weights, ids) for ids in seqs]

    def feed(rc, ids, at, n, wanted):
        return StepRow(rc, ids[at : at + n], wanted)

    # whole
    for ids, ref in zip(seqs, want):
        rc = runner.acquire()
        got = runner.step([feed(rc, ids, 0, len(ids), range(len(ids)))]).cpu().numpy()
        check_logits(got, ref, dtype, "toy whole")
        runner.release(rc)
    # portions of some beside single tokens of others; the state must carry across steps
    handles = [runner.acquire() for _ in seqs]
    fed = [0] * len(seqs)
    portion = [5, 1, 1]  # once the first request is through, the steps are pure decode steps
    while any(f < len(s) for f, s in zip(fed, seqs)):
        rows, meta = [], []
        for i, (rc, ids) in enumerate(zip(handles, seqs)):
            n = min(portion[i], len(ids) - fed[i])
            if n:
                rows.append(feed(rc, ids, fed[i], n, range(n)))
                meta.append((i, fed[i], n))
                fed[i] += n
        got = runner.step(rows).cpu().numpy()
        at = 0
        for i, s, n in meta:
            check_logits(got[at : at + n], want[i][s : s + n], dtype, f"toy request {i} at {s}")
            at += n
    assert runner.graph_steps > 0, "pure decode steps were meant to replay a captured graph"
    slots = {rc.state_slot for rc in handles}
    assert len(slots) == 3
    for rc in handles:
        runner.release(rc)
    assert runner.cache.idle
    # a slot that held another request's state is handed out again and starts from zero
    rc = runner.acquire()
    assert rc.state_slot in slots
    got = runner.step([feed(rc, seqs[2], 0, len(seqs[2]), range(len(seqs[2])))]).cpu().numpy()
    check_logits(got, want[2], dtype, "toy after slot reuse")
    runner.release(rc)

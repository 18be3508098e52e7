"""A toy architecture, defined entirely in this test, is registered, built and stepped without a
change to the framework's files: a mixer with fixed-size per-request state of its own, a feed-forward
that routes each token to one of three experts and reads another part's tensor under a name of its own
(an alias), a position encoding of its own inside the stock attention mixer (once turning the halves of
a head, once adjacent elements), a block arrangement of its own (mixer and feed-forward side by side
behind one norm), a layer that attends within a window beside layers that keep every key (two cache
groups, the windowed one with fewer pages), the other activation of the stock gated feed-forward, and a
run order that names one layer's weights twice and lets an entry read another entry's cache. Whole
prompts, portions, single tokens and captured decode graphs must all agree with a plain implementation
of the same toy, also defined here."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu

H, HEADS, KVH, D, INTER, VOCAB, DECAY = 64, 4, 2, 16, 96, 97, 0.75
EXPERTS, EXPERT_WIDTH, ROUTER_SCALE = 3, 32, 60.0  # the scale keeps the winner clear of bfloat16 rounding
ROT_DIM, POS_STEP = 8, 0.5  # the toy position encoding turns pair j of the first 8 elements by (POS_STEP * position) / (j + 1)
WINDOW = 12  # of the last layer's attention


@pytest.fixture(scope="module")
def toy():
    from miniserve_amd.config import LayerSpec, ModelSpec, PartSpec, RunEntry, register_architecture, unregister_architecture
    from miniserve_amd.parts import (Block, FeedForward, Mixer, PositionEncoding, Rotation, StateNeed, StateTensor, TensorSpec, part_class,
                                     register, unregister)

    @register("mixer", "toy_decay")
    class DecayMixer(Mixer):
        """s_t = decay * s_{t-1} + x_t per request (s starts at 0), n_t = tokens seen so far (this one
        included); output = (s_t / (1 + n_t / 8) + bias) W^T. The state is two tensors of different
        dtypes (the float32 sum and the int32 count), the bias a one-dimensional tensor that is no norm weight."""

        def __init__(self, spec, rt):
            super().__init__(spec, rt)
            self.width, self.decay = int(spec["width"]), float(spec["decay"])

        @classmethod
        def tensors(cls, spec):
            w = int(spec["width"])
            return {"toy.weight": TensorSpec((w, w)), "toy.bias": TensorSpec((w,), init="uniform")}

        def bind(self, tensors):
            self.weight, self.bias = tensors["toy.weight"], tensors["toy.bias"]

        def state_need(self):
            return StateNeed((StateTensor("sum", (self.width,), "float32"), StateTensor("seen", (1,), "int32")))

        def forward(self, x, batch, cache, state, residual):
            xf = x.float()
            total, seen = state["sum"], state["seen"]
            slots = batch.state_slots.long()
            if batch.is_decode:  # one token per row: no host loop, capturable in a graph
                fresh = batch.starts[:, None] == 0
                s = torch.where(fresh, torch.zeros_like(xf), total[slots]) * self.decay + xf
                n = torch.where(fresh, torch.zeros_like(seen[slots]), seen[slots]) + 1
                total[slots], seen[slots] = s, n
                out = s / (1 + n.float() / 8)
            else:
                out = torch.empty_like(xf)
                t = 0
                for i, (n, start) in enumerate(zip(batch.row_lens, batch.row_starts_host)):
                    slot = slots[i]
                    s = torch.zeros(self.width, device=xf.device) if start == 0 else total[slot].clone()
                    for j in range(n):
                        s = s * self.decay + xf[t + j]
                        out[t + j] = s / (1 + (start + j + 1) / 8)
                    total[slot] = s
                    seen[slot] = start + n
                    t += n
            out = out + self.bias.float()
            return self.rt.ops.linear(out.to(x.dtype).contiguous(), self.weight, accumulate_into=residual, defer=True)

    @register("feed_forward", "toy_routed")
    class RoutedFeedForward(FeedForward):
        """Each token goes to the expert with the largest router logit (float32) and gets that expert's
        ``W2 relu(W1 x)`` times the router's softmax weight of it. All experts are run and the others'
        hidden units zeroed: no host decision, so a decode step can be captured."""

        def __init__(self, spec, rt):
            super().__init__(spec, rt)
            self.width, self.experts, self.inner = int(spec["width"]), int(spec["experts"]), int(spec["inner"])
            self.router_scale = float(spec["router_scale"])

        @classmethod
        def tensors(cls, spec):
            w, e, f = int(spec["width"]), int(spec["experts"]), int(spec["inner"])
            return {"moe.router.weight": TensorSpec((e, w)), "moe.w1.weight": TensorSpec((e * f, w)),
                    "moe.w2.weight": TensorSpec((w, e * f))}

        @classmethod
        def aliases(cls, spec):
            return {"moe.bias": spec["bias_from"]}  # nothing is stored under this name: it is another part's tensor

        def bind(self, tensors):
            self.router, self.w1, self.w2 = (tensors["moe." + n + ".weight"] for n in ("router", "w1", "w2"))
            self.out_bias = tensors["moe.bias"]
            self.expert_ids = torch.arange(self.experts, device=self.router.device)

        def forward(self, x, residual):
            ops = self.rt.ops
            logits = (x.float() @ self.router.float().T) * self.router_scale
            prob, choice = torch.softmax(logits, dim=-1).max(dim=-1)
            hidden = torch.relu(ops.linear(x, self.w1, out_dtype=self.rt.dtype)).view(-1, self.experts, self.inner)
            chosen = (choice[:, None] == self.expert_ids[None, :]).to(hidden.dtype)[:, :, None]
            y = ops.linear((hidden * chosen).view(-1, self.experts * self.inner).contiguous(), self.w2, out_dtype=torch.float32)
            residual += prob[:, None] * y + self.out_bias.float()
            return None

        def parameters_bytes(self):
            return sum(t.numel() * t.element_size() for t in (self.router, self.w1, self.w2))

    @register("position", "toy_slow_rotation")
    class SlowRotation(PositionEncoding):
        """Pair j of the first ``dim`` elements of a head is turned by ``step * position / (j + 1)``; which
        elements make a pair is a parameter."""

        def __init__(self, spec, rt):
            super().__init__(spec, rt)
            self.dim, self.step, self.pairing = int(spec["dim"]), float(spec["step"]), spec.get("pairing", "halves")

        def rotation(self, batch):
            key = ("toy_slow_rotation", self.dim, self.step)
            if key not in batch.memo:
                j = torch.arange(1, self.dim // 2 + 1, device=batch.positions.device, dtype=torch.float32)
                ang = (batch.positions.float() * self.step)[:, None] / j[None, :]
                batch.memo[key] = torch.cat((torch.cos(ang), torch.sin(ang)), dim=1).contiguous()
            return Rotation(self.dim, batch.memo[key], self.pairing)

    @register("block", "toy_side_by_side")
    class SideBySide(Block):
        """``h += mixer(norm(h)) + feed_forward(norm(h))``: one norm, both parts read its output."""

        def __init__(self, spec, rt, mixer, feed_forward):
            super().__init__(spec, rt, mixer, feed_forward)
            n = spec["norm"]
            self.norm = part_class("norm", n)(n, rt)

        @classmethod
        def tensors(cls, spec):
            return dict(part_class("norm", spec["norm"]).tensors(spec["norm"]))

        def bind(self, tensors):
            self.norm.bind(tensors)

        def forward(self, residual, batch, cache, state, pending=None):
            x = self.norm.forward(residual, add=pending)
            self.rt.ops.add_pending(residual, self.mixer.forward(x, batch, cache, state, residual))
            return self.feed_forward.forward(x, residual)

        def parameters_bytes(self):
            return self.norm.parameters_bytes()

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
                "scale": 0.3, "qk_norm_eps": None, "window": 0,
                "position": PartSpec("toy_slow_rotation", {"dim": ROT_DIM, "step": POS_STEP})})
            routed = PartSpec("toy_routed", {"width": H, "experts": EXPERTS, "inner": EXPERT_WIDTH, "router_scale": ROUTER_SCALE,
                                             "bias_from": "l0.toy.bias"})
            near = PartSpec("gqa_attention", {
                "prefix": "attn.", "hidden_size": H, "num_heads": HEADS, "num_kv_heads": KVH, "head_dim": D,
                "scale": 0.3, "qk_norm_eps": 1e-5, "window": WINDOW,
                "position": PartSpec("toy_slow_rotation", {"dim": ROT_DIM, "step": POS_STEP, "pairing": "adjacent"})})
            gelu = PartSpec("gated_mlp", {"prefix": "mlp.", "hidden_size": H, "intermediate_size": INTER, "activation": "gelu_tanh"})
            layers = (
                LayerSpec("l0.", PartSpec("toy_side_by_side", {"norm": norm("n1.weight")}), PartSpec("toy_decay", {"width": H, "decay": DECAY}), routed),
                LayerSpec("l1.", block(), attn, ffn),
                LayerSpec("l2.", block(), near, gelu),
            )
            order = (RunEntry(0, 0), RunEntry(1, 1), RunEntry(1, 2), RunEntry(1, 1, writes_cache=False), RunEntry(2, 3))
            return ModelSpec(
                architecture="ToyForCausalLM", vocab_size=VOCAB, hidden_size=H,
                embedding=PartSpec("token_embedding", {"vocab_size": VOCAB, "width": H, "tensor": "emb.weight"}),
                layers=layers, run_order=order, final_norm=norm("out_norm.weight"),
                head=PartSpec("linear_head", {"vocab_size": VOCAB, "width": H, "tensor": "head.weight", "tied_to": None}))

    yield ToyConfig
    unregister_architecture("ToyForCausalLM")
    unregister("mixer", "toy_decay")
    unregister("feed_forward", "toy_routed")
    unregister("position", "toy_slow_rotation")
    unregister("block", "toy_side_by_side")


margins: list[float] = []  # smallest gap between the two best router logits of each sequence the plain toy ran


def plain_toy(w, ids):
    """The toy in float64: layer 0 (decay mixer and routed feed-forward side by side behind one norm), then layer 1's weights three
    times: with a cache of its own, with another cache of its own, and reading the keys and values of
    the first of these."""
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
        outs.append(s / (1 + (t + 1) / 8) + w["l0.toy.bias"])
    mixed = np.stack(outs) @ w["l0.toy.weight"].T
    # routed feed-forward on the same normalised input: the expert with the largest router logit, weighted by its softmax weight
    y = x
    logits = (y @ w["l0.moe.router.weight"].T) * ROUTER_SCALE
    prob = np.exp(logits - logits.max(-1, keepdims=True))
    prob /= prob.sum(-1, keepdims=True)
    choice = logits.argmax(-1)
    ranked = np.sort(logits, axis=-1)
    margins.append(float((ranked[:, -1] - ranked[:, -2]).min()))
    w1 = w["l0.moe.w1.weight"].reshape(EXPERTS, EXPERT_WIDTH, H)
    w2 = w["l0.moe.w2.weight"].reshape(H, EXPERTS, EXPERT_WIDTH)
    out = np.stack([prob[t, e] * (w2[:, e, :] @ np.maximum(w1[e] @ y[t], 0.0)) for t, e in enumerate(choice)])
    h = h + mixed + out + w["l0.toy.bias"]  # the routed feed-forward reads the mixer's bias as its own output bias

    ang = ((np.arange(T) * POS_STEP)[:, None] / np.arange(1, ROT_DIM // 2 + 1)[None, :]).astype(np.float32)

    def rot(v):  # partial rotation: the first ROT_DIM elements of each head
        return np.concatenate((P.apply_rotary(v[..., :ROT_DIM], ang), v[..., ROT_DIM:]), axis=-1)

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

    # layer 2: per-head norms, adjacent elements (2j, 2j + 1) turned by angle j, a window, the tanh form of GELU
    def turn_adjacent(v):
        a, b = v[..., 0:ROT_DIM:2], v[..., 1:ROT_DIM:2]
        cos, sin = np.cos(ang.astype(np.float64))[:, None, :], np.sin(ang.astype(np.float64))[:, None, :]
        out = v.copy()
        out[..., 0:ROT_DIM:2], out[..., 1:ROT_DIM:2] = a * cos - b * sin, b * cos + a * sin
        return out

    x = P.rms_norm(h, w["l2.n1.weight"], 1e-5)
    q = P.rms_norm((x @ w["l2.attn.q_proj.weight"].T).reshape(T, HEADS, D), w["l2.attn.q_norm.weight"], 1e-5)
    k = P.rms_norm((x @ w["l2.attn.k_proj.weight"].T).reshape(T, KVH, D), w["l2.attn.k_norm.weight"], 1e-5)
    v = (x @ w["l2.attn.v_proj.weight"].T).reshape(T, KVH, D)
    o = P.attention(turn_adjacent(q), turn_adjacent(k), v, 0.3, WINDOW).reshape(T, HEADS * D)
    h = h + o @ w["l2.attn.o_proj.weight"].T
    y = P.rms_norm(h, w["l2.n2.weight"], 1e-5)
    g, u = y @ w["l2.mlp.gate_proj.weight"].T, y @ w["l2.mlp.up_proj.weight"].T
    h = h + (0.5 * g * (1 + np.tanh(np.sqrt(2 / np.pi) * (g + 0.044715 * g**3))) * u) @ w["l2.mlp.down_proj.weight"].T
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
    # The comparison below means something only where rounding cannot change an expert choice: the first
    # seed whose weights keep the router's two best logits apart at every position of the test's sequences.
    rng = np.random.default_rng(3)
    seqs = [rng.integers(0, VOCAB, n).tolist() for n in (37, 50, 9)]
    for seed in range(7, 47):
        weights = random_tensors(spec, seed, Init(0.08, (0.6, 1.4)), dtype=rt.dtype, device=rt.device)
        margins.clear()
        want = [plain_toy(weights, ids) for ids in seqs]
        if min(margins) > (0.5 if dtype == "bfloat16" else 1e-3):
            break
    else:
        pytest.fail(f"no seed keeps the router's choice clear of rounding (last margins {margins})")
    model = DecoderModel(spec, weights, rt)
    needs = model.cache_slots()
    assert [n.slot for n in needs] == [0, 1, 2, 3] and needs[0].kv is None and needs[3].kv.window == WINDOW
    assert [(t.name, t.shape, t.dtype) for t in needs[0].state.tensors] == [("sum", (H,), "float32"), ("seen", (1,), "int32")]
    assert [(p.name, p.heads, p.width) for p in needs[1].kv.planes] == [("k", KVH, D), ("v", KVH, D)] and needs[1].state is None
    assert weights["l0.toy.bias"].float().abs().max() > 0.01, "the bias was meant to be drawn, not taken for a norm weight"

    assert model.blocks[0].feed_forward.out_bias is model.blocks[0].mixer.bias, "an alias is the source's tensor, not a copy"
    assert "l0.moe.bias" not in weights, "nothing is drawn or stored under an alias"

    # steps carry at most 5 tokens of a request here: the windowed group never holds more than the window and a step
    # per request, and gets only those pages; whole prompts (below) need a runner that does not promise that
    runner = ModelRunner(model, kv_pool_tokens=16 * 12, max_running=4, decode_graph=True, request_step_tokens=5)
    assert [(g.slots, g.window) for g in runner.layout.groups] == [((1, 2), 0), ((3,), WINDOW)]
    assert [s.slot for s in runner.layout.states] == [0]
    assert runner.pages_per_group == [12, 4 * 2] and runner.cache.total_pages() == [12, 8]
    assert [b[n].shape[1] for b, n in zip(runner.pool.buffers, ("k", "k"))] == [13, 9]  # pages + the dummy page
    whole = ModelRunner(model, kv_pool_tokens=16 * 12, max_running=4)
    assert whole.pages_per_group == [12, 12]

    def feed(rc, ids, at, n, wanted):
        return StepRow(rc, ids[at : at + n], wanted)

    # whole
    for ids, ref in zip(seqs, want):
        rc = whole.acquire()
        got = whole.step([feed(rc, ids, 0, len(ids), range(len(ids)))]).cpu().numpy()
        check_logits(got, ref, dtype, "toy whole")
        whole.release(rc)
    del whole
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
    ids = seqs[2]
    got = np.concatenate([runner.step([feed(rc, ids, at, min(5, len(ids) - at), range(min(5, len(ids) - at)))]).cpu().numpy()
                          for at in range(0, len(ids), 5)])
    check_logits(got, want[2], dtype, "toy after slot reuse")
    runner.release(rc)
    # the parts say what a step costs: the model's figure is their sum, and a part that says nothing counts as nothing
    rows = [(5, 20), (1, 33)]
    stock = sum(b.mixer.flops(rows) + b.feed_forward.flops(rows) for b in (model.blocks[1], model.blocks[1], model.blocks[1], model.blocks[2]))
    assert model.step_flops(rows) == stock + model.head.flops(rows) and model.blocks[0].mixer.flops(rows) == 0
    near = model.blocks[2].mixer
    pairs = sum(min(p + 1, WINDOW) for p in range(20, 25)) + min(34, WINDOW)
    assert near.flops(rows) == 2 * 6 * H * (HEADS * D + 2 * KVH * D) + 2 * 6 * HEADS * D * H + 4 * pairs * HEADS * D

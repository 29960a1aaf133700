"""Toy parts for the tests of generality: a feed-forward that routes, a position encoding of
its own, a run order that names a layer twice.  Nothing here is a model of anyone's."""
from dataclasses import dataclass
from typing import ClassVar

import torch

import plain_qwen2 as plain


def run_toy_mix(dtype, device, tolerance):
    """Parts defined here -- a feed-forward that routes every token to one of three experts, and
    a rotary encoding that pairs neighbouring dimensions -- are registered and put into a model
    beside the framework's own parts; the first layer runs a second time at the end, reading the
    keys and values of its first run.  The model also uses what the model specification offers beyond
    the one architecture's needs: a factor on the embedding rows, a factor on the logits, a bias on the
    output head, and a score scale of its own in one layer's attention.  Whole requests and requests cut
    into portions beside other requests agree with each other and with a plain computation written out below."""
    from torchlet_amd.config import (AttentionSpec, BlockSpec, ModelConfig, ModelSpec, PartSpec, RMSNormSpec, RotarySpec,
                                     RunEntry, SwiGLUSpec)
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import build_model, make_runner
    from torchlet_amd.kernels import ops
    from torchlet_amd.parts import FEED_FORWARDS, POSITION_ENCODINGS, FeedForward, PositionEncoding, WeightSpec
    from torchlet_amd.registry import config_class, register_architecture, unregister_architecture
    from torchlet_amd.weights.random_init import random_tensors

    H, HEADS, KVH, HD, INTER, EXPERTS, VOCAB, THETA = 48, 4, 2, 16, 40, 3, 50, 100.0
    EMBED_SCALE, LOGIT_SCALE, SCORE_SCALE = 1.7, 0.6, 0.31

    @dataclass(frozen=True)
    class PairRotarySpec(PartSpec):
        kind: ClassVar[str] = "toy_rope_pairs"
        head_dim: int = 0
        theta: float = 10000.0

    @POSITION_ENCODINGS.register("toy_rope_pairs")
    class PairRotary(PositionEncoding):
        """Rotation of the pairs (2j, 2j + 1) by pos * theta**(-2j / head_dim), in 32-bit."""

        def apply(self, q, k, positions):
            hd = self.spec.head_dim
            inv = 1.0 / (self.spec.theta ** (torch.arange(0, hd, 2, dtype=torch.float32, device=q.device) / hd))
            ang = positions.float()[:, None] * inv
            c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
            for x in (q, k):
                if x is None:
                    continue
                a, b = x[..., 0::2].float(), x[..., 1::2].float()
                first, second = a * c - b * s, b * c + a * s       # both before either is stored: a and b may be views
                x[..., 0::2] = first.to(x.dtype)
                x[..., 1::2] = second.to(x.dtype)

    @dataclass(frozen=True)
    class Top1Spec(PartSpec):
        kind: ClassVar[str] = "toy_top1"
        hidden: int = 0
        intermediate: int = 0
        experts: int = 0

    @FEED_FORWARDS.register("toy_top1")
    class Top1Experts(FeedForward):
        """y = p_e * down_e(silu(gate_e x) * up_e x) for the expert e with the largest router
        logit, p = softmax of the router logits in 32-bit."""

        def weight_specs(self):
            s = self.spec
            specs = {"router.weight": WeightSpec((s.experts, s.hidden), keep="float32")}     # a matrix that stays 32-bit
            for e in range(s.experts):
                specs[f"experts.{e}.gate.weight"] = WeightSpec((s.intermediate, s.hidden))
                specs[f"experts.{e}.up.weight"] = WeightSpec((s.intermediate, s.hidden))
                specs[f"experts.{e}.down.weight"] = WeightSpec((s.hidden, s.intermediate))
            return specs

        def load_weights(self, tensors):
            self.router = self._place(tensors["router.weight"], "float32")
            self.w = {k: self._place(v, "compute") for k, v in tensors.items() if k.startswith("experts.")}

        def forward(self, h, ctx):
            s = self.spec
            p = torch.softmax(h.float() @ self.router.T, dim=-1)
            top = p.argmax(-1)
            y = torch.zeros_like(h)
            for e in range(s.experts):
                rows = (top == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                x = h[rows].contiguous()
                g = torch.empty((x.shape[0], s.intermediate), dtype=h.dtype, device=h.device)
                u = torch.empty_like(g)
                ops.linear(x, self.w[f"experts.{e}.gate.weight"], None, g)
                ops.linear(x, self.w[f"experts.{e}.up.weight"], None, u)
                z = (torch.nn.functional.silu(g.float()) * u.float()).to(h.dtype)
                d = torch.empty_like(x)
                ops.linear(z, self.w[f"experts.{e}.down.weight"], None, d)
                y[rows] = (d.float() * p[rows, e, None]).to(h.dtype)
            return y

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyMixForCausalLM"
        vocab_size: int

        def to_spec(self):
            norm = RMSNormSpec(dim=H, eps=1e-5)
            attn = lambda pos, scale=None: AttentionSpec(hidden=H, num_heads=HEADS, num_kv_heads=KVH, head_dim=HD, qkv_bias=False,
                                                         position=pos, scale=scale)
            first = BlockSpec(mixer=attn(PairRotarySpec(head_dim=HD, theta=THETA)), mixer_norm=norm, ffn_norm=norm,
                              ffn=SwiGLUSpec(hidden=H, intermediate=INTER))
            second = BlockSpec(mixer=attn(RotarySpec(head_dim=HD, theta=THETA, max_positions=4096), SCORE_SCALE), mixer_norm=norm,
                               ffn_norm=norm, ffn=Top1Spec(hidden=H, intermediate=INTER, experts=EXPERTS), ffn_name="moe")
            return ModelSpec(vocab_size=self.vocab_size, hidden=H, layers=(first, second),
                             order=(RunEntry(0), RunEntry(1), RunEntry(0, cache_of=0)), final_norm=norm,
                             tie_head=True, max_positions=4096, embed_scale=EMBED_SCALE, logit_scale=LOGIT_SCALE, head_bias=True)

    def pair_rope(x, positions):                      # x [heads, T, hd], float64
        inv = 1.0 / (THETA ** (torch.arange(0, HD, 2, dtype=torch.float32) / HD))
        ang = (positions.float()[:, None] * inv).double()
        a, b = x[..., 0::2], x[..., 1::2]
        y = torch.empty_like(x)
        y[..., 0::2] = a * ang.cos() - b * ang.sin()
        y[..., 1::2] = b * ang.cos() + a * ang.sin()
        return y

    def plain_attention(h, w, rope, kv=None, stored=lambda t: t, scale=None):
        """Returns the mixed heads' projection and the (k, v) it used; with ``kv`` given, only q is new.
        ``stored``: applied to what separate kernels hand each other through memory (see plain_qwen2)."""
        T = h.shape[0]
        pos = torch.arange(T)
        q = stored(rope(stored(h @ w["q_proj.weight"].T).view(T, HEADS, HD).transpose(0, 1), pos))
        if kv is None:
            k = stored(rope(stored(h @ w["k_proj.weight"].T).view(T, KVH, HD).transpose(0, 1), pos))
            v = stored(h @ w["v_proj.weight"].T).view(T, KVH, HD).transpose(0, 1)
            kv = (k, v)
        k, v = (t.repeat_interleave(HEADS // KVH, dim=0) for t in kv)
        if scale is not None:             # attention_weights divides the scores by sqrt(head size): undo that, put `scale` there
            q = q * (scale * HD ** 0.5)
        ctx = stored((plain.attention_weights(q, k) @ v).transpose(0, 1).reshape(T, HEADS * HD))
        return stored(ctx @ w["o_proj.weight"].T), kv

    def plain_forward(w, ids, stored=lambda t: t):
        sub = lambda p: {k[len(p):]: v for k, v in w.items() if k.startswith(p)}
        l0, l1 = sub("model.layers.0."), sub("model.layers.1.")
        x = w["model.embed_tokens.weight"][torch.tensor(ids)] * EMBED_SCALE
        norm = lambda t, weight: stored(plain.rms_norm(t, weight, 1e-5))
        a, kv0 = plain_attention(norm(x, l0["input_layernorm.weight"]), sub("model.layers.0.self_attn."), pair_rope, None, stored)
        x = x + a
        x = x + plain.swiglu_ffn(norm(x, l0["post_attention_layernorm.weight"]), sub("model.layers.0.mlp."), stored)
        a, _ = plain_attention(norm(x, l1["input_layernorm.weight"]), sub("model.layers.1.self_attn."),
                               lambda t, pos: plain.rope_apply(t, pos, THETA), None, stored, SCORE_SCALE)
        x = x + a
        h = norm(x, l1["post_attention_layernorm.weight"])
        p = torch.softmax(h @ l1["moe.router.weight"].T, dim=-1)
        top = p.argmax(-1)
        best2 = p.topk(2, dim=-1).values
        gaps.append(float((best2[:, 0] - best2[:, 1]).min()))
        rows = []
        for t in range(len(ids)):
            e = int(top[t])
            gate = stored(h[t] @ l1[f"moe.experts.{e}.gate.weight"].T)
            up = stored(h[t] @ l1[f"moe.experts.{e}.up.weight"].T)
            z = stored(torch.nn.functional.silu(gate) * up)
            rows.append(stored(p[t, e] * stored(z @ l1[f"moe.experts.{e}.down.weight"].T)))
        x = x + torch.stack(rows)
        a, _ = plain_attention(norm(x, l0["input_layernorm.weight"]), sub("model.layers.0.self_attn."), pair_rope, kv0, stored)
        x = x + a
        x = x + plain.swiglu_ffn(norm(x, l0["post_attention_layernorm.weight"]), sub("model.layers.0.mlp."), stored)
        last = stored(plain.rms_norm(x, w["model.norm.weight"], 1e-5) * LOGIT_SCALE)
        return last @ w["model.embed_tokens.weight"].T + w["lm_head.bias"]

    gaps = []
    register_architecture(ToyConfig)
    try:
        cfg = config_class("ToyMixForCausalLM").from_dict(dict(vocab_size=VOCAB))
        tensors = {k: (v * 5 if "proj" in k or "experts" in k or "router" in k else v)
                   for k, v in random_tensors(cfg, seed=4, dtype=torch.bfloat16).items()}
        assert "model.layers.1.moe.experts.2.down.weight" in tensors and "model.layers.1.moe.router.weight" in tensors
        assert tensors["lm_head.bias"].shape == (VOCAB,) and "lm_head.weight" not in tensors
        model = build_model(cfg, dtype, device=device, tensors=tensors)
        assert model.blocks[1].ffn.router.dtype == torch.float32 and model.blocks[1].ffn.router.shape == (EXPERTS, H)   # a matrix kept in 32-bit
        runner = make_runner(model, page_size=8, num_pages=24, max_requests=2)
        assert len(runner.caches) == 3 and runner.caches[2].planes[0].data_ptr() == runner.caches[0].planes[0].data_ptr() and not runner.caches[2].writable
        # token sequences for which no token's choice of expert hangs on the last bits of a
        # bfloat16 evaluation: the first seed whose smallest gap between the two best experts is wide
        w = {k: v.double() for k, v in tensors.items()}
        for seed in range(2, 60):
            g = torch.Generator().manual_seed(seed)
            seqs = {"a": torch.randint(0, VOCAB, (41,), generator=g).tolist(), "b": torch.randint(0, VOCAB, (19,), generator=g).tolist()}
            gaps.clear()
            refs = {k: plain_forward(w, v) for k, v in seqs.items()}
            if min(gaps) > 0.05:
                break
        else:
            raise AssertionError("no seed with a clear choice of expert for every token")
        whole = {k: runner.step([StepEntry(k, v, list(range(len(v))))]).cpu() for k, v in seqs.items()}
        for k in seqs:
            runner.release(k)
        got = {"a": [], "b": []}
        got["a"].append(runner.step([StepEntry("a", seqs["a"][:13], list(range(13)))]).cpu())
        out = runner.step([StepEntry("b", seqs["b"][:6], list(range(6))), StepEntry("a", seqs["a"][13:14], [0])]).cpu()
        got["b"].append(out[:6]); got["a"].append(out[6:])
        out = runner.step([StepEntry("a", seqs["a"][14:], list(range(27))), StepEntry("b", seqs["b"][6:], list(range(13)))]).cpu()
        got["a"].append(out[:27]); got["b"].append(out[27:])
        # The router reads which tokens chose which expert on the host (`.nonzero()`): it does not say it is safe to
        # record, neither does the toy position encoding, so the model is not, and a step function asked for graphs
        # runs every step of this model eagerly (a recorded step would replay the shapes of the step it recorded).
        assert not model.blocks[1].ffn.graph_safe and not model.blocks[0].mixer.position.graph_safe
        assert model.blocks[0].ffn.graph_safe and model.blocks[1].mixer.position.graph_safe and not model.graph_safe()
        for k in seqs:
            runner.release(k)
        eager = make_runner(model, page_size=8, num_pages=24, max_requests=2, use_graphs=True)
        assert not eager.use_graphs and eager.warm_up() == 0
        singles = {k: [] for k in seqs}
        for i in range(len(seqs["a"])):               # both requests token by token: decode-only steps, the router's shapes change
            live = [k for k in seqs if i < len(seqs[k])]
            out = eager.step([StepEntry(k, [seqs[k][i]], [0]) for k in live]).cpu()
            for j, k in enumerate(live):
                singles[k].append(out[j: j + 1])
        assert eager.graph_replays == 0 and not eager._graphs
        for k in seqs:
            tol = tolerance(dtype, refs[k])
            if dtype == torch.bfloat16:
                # what roundings to bfloat16 between the kernels alone do to the logits, in a 64-bit
                # evaluation: the engine rounds at the same places, so it may be off by as much, twice at most
                moved = plain_forward(w, seqs[k], stored=lambda t: t.to(torch.bfloat16).double()) - refs[k]
                tol = dict(atol=2 * float(moved.abs().max()), rtol=0.0)
            torch.testing.assert_close(whole[k].double(), refs[k], **tol)
            torch.testing.assert_close(torch.cat(got[k]).double(), refs[k], **tol)
            torch.testing.assert_close(torch.cat(singles[k]).double(), refs[k], **tol)
    finally:
        unregister_architecture("ToyMixForCausalLM")
        POSITION_ENCODINGS.unregister("toy_rope_pairs")
        FEED_FORWARDS.unregister("toy_top1")


def run_toy_qk_norm(dtype, device, tolerance):
    """A mixer that differs from the framework's attention in one stage only -- queries and keys are normalised per
    head before they are rotated and stored -- is a subclass that declares two more tensors and defines the
    ``transform_qk`` hook; projection, rotation, cache write, attention kernels and output projection are the
    framework's.  Whole requests, portions and single tokens agree with each other and with a plain computation."""
    from torchlet_amd.config import AttentionSpec, BlockSpec, ModelConfig, ModelSpec, RMSNormSpec, RotarySpec, RunEntry, SwiGLUSpec
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import build_model, make_runner
    from torchlet_amd.parts import MIXERS, WeightSpec
    from torchlet_amd.parts.attention import GQAttention
    from torchlet_amd.registry import config_class, register_architecture, unregister_architecture
    from torchlet_amd.weights.random_init import random_tensors

    H, HEADS, KVH, HD, INTER, VOCAB, THETA, EPS = 40, 6, 2, 32, 56, 60, 5000.0, 1e-6

    @dataclass(frozen=True)
    class QKNormAttentionSpec(AttentionSpec):
        kind: ClassVar[str] = "toy_qk_norm_attention"

    @MIXERS.register("toy_qk_norm_attention")
    class QKNormAttention(GQAttention):
        def weight_specs(self):
            specs = super().weight_specs()
            specs["q_norm.weight"] = WeightSpec((self.head_dim,), keep="stored", init="one_plus_normal")
            specs["k_norm.weight"] = WeightSpec((self.head_dim,), keep="stored", init="one_plus_normal")
            return specs

        def load_weights(self, tensors):
            super().load_weights(tensors)
            self.q_norm = self._place(tensors["q_norm.weight"], "stored").float()
            self.k_norm = self._place(tensors["k_norm.weight"], "stored").float()

        def transform_qk(self, q3, k3, ctx):
            for x, w in ((q3, self.q_norm), (k3, self.k_norm)):
                if x is not None:
                    f = x.float()
                    x.copy_((f * torch.rsqrt(f.pow(2).mean(-1, keepdim=True) + EPS) * w).to(x.dtype))

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyQKNormForCausalLM"
        vocab_size: int

        def to_spec(self):
            norm = RMSNormSpec(dim=H, eps=1e-5)
            block = BlockSpec(mixer=QKNormAttentionSpec(hidden=H, num_heads=HEADS, num_kv_heads=KVH, head_dim=HD, qkv_bias=True,
                                                        position=RotarySpec(head_dim=HD, theta=THETA, max_positions=512)),
                              mixer_norm=norm, ffn_norm=norm, ffn=SwiGLUSpec(hidden=H, intermediate=INTER))
            return ModelSpec(vocab_size=self.vocab_size, hidden=H, layers=(block, block), order=(RunEntry(0), RunEntry(1)),
                             final_norm=norm, tie_head=False, max_positions=512)

    def plain_forward(w, ids, stored=lambda t: t):
        sub = lambda p: {k[len(p):]: v for k, v in w.items() if k.startswith(p)}
        T = len(ids)
        pos = torch.arange(T)
        x = w["model.embed_tokens.weight"][torch.tensor(ids)]
        norm = lambda t, weight: stored(plain.rms_norm(t, weight, 1e-5))
        for layer in range(2):
            lw, a = sub(f"model.layers.{layer}."), sub(f"model.layers.{layer}.self_attn.")
            h = norm(x, lw["input_layernorm.weight"])
            q = stored(plain.linear(h, a["q_proj.weight"], a["q_proj.bias"])).view(T, HEADS, HD)
            k = stored(plain.linear(h, a["k_proj.weight"], a["k_proj.bias"])).view(T, KVH, HD)
            v = stored(plain.linear(h, a["v_proj.weight"], a["v_proj.bias"])).view(T, KVH, HD).transpose(0, 1)
            q = stored(plain.rms_norm(q, a["q_norm.weight"], EPS)).transpose(0, 1)
            k = stored(plain.rms_norm(k, a["k_norm.weight"], EPS)).transpose(0, 1)
            q, k = stored(plain.rope_apply(q, pos, THETA)), stored(plain.rope_apply(k, pos, THETA))
            k, v = (t.repeat_interleave(HEADS // KVH, dim=0) for t in (k, v))
            ctx = stored((plain.attention_weights(q, k) @ v).transpose(0, 1).reshape(T, HEADS * HD))
            x = x + stored(plain.linear(ctx, a["o_proj.weight"]))
            x = x + plain.swiglu_ffn(norm(x, lw["post_attention_layernorm.weight"]), sub(f"model.layers.{layer}.mlp."), stored)
        return plain.linear(norm(x, w["model.norm.weight"]), w["lm_head.weight"])

    register_architecture(ToyConfig)
    try:
        cfg = config_class("ToyQKNormForCausalLM").from_dict(dict(vocab_size=VOCAB))
        tensors = {k: (v * 4 if "proj" in k else v) for k, v in random_tensors(cfg, seed=6, dtype=torch.bfloat16).items()}
        assert tensors["model.layers.1.self_attn.q_norm.weight"].shape == (HD,)
        model = build_model(cfg, dtype, device=device, tensors=tensors)
        assert not model.blocks[0].mixer.pair_layout              # the hook sees the checkpoint's order of dimensions
        runner = make_runner(model, page_size=8, num_pages=20, max_requests=2)
        g = torch.Generator().manual_seed(3)
        seqs = {"a": torch.randint(0, VOCAB, (45,), generator=g).tolist(), "b": torch.randint(0, VOCAB, (21,), generator=g).tolist()}
        w = {k: v.double() for k, v in tensors.items()}
        refs = {k: plain_forward(w, v) for k, v in seqs.items()}
        whole = {k: runner.step([StepEntry(k, v, list(range(len(v))))]).cpu() for k, v in seqs.items()}
        for k in seqs:
            runner.release(k)
        got = {"a": [], "b": []}
        got["a"].append(runner.step([StepEntry("a", seqs["a"][:17], list(range(17)))]).cpu())
        out = runner.step([StepEntry("b", seqs["b"][:9], list(range(9))), StepEntry("a", seqs["a"][17:18], [0])]).cpu()
        got["b"].append(out[:9]); got["a"].append(out[9:])
        out = runner.step([StepEntry("a", seqs["a"][18:40], list(range(22))), StepEntry("b", seqs["b"][9:], list(range(12)))]).cpu()
        got["a"].append(out[:22]); got["b"].append(out[22:])
        for t in seqs["a"][40:]:
            got["a"].append(runner.step([StepEntry("a", [t], [0])]).cpu())
        for k in seqs:
            tol = tolerance(dtype, refs[k])
            if dtype == torch.bfloat16:
                moved = plain_forward(w, seqs[k], stored=lambda t: t.to(torch.bfloat16).double()) - refs[k]
                tol = dict(atol=2 * float(moved.abs().max()), rtol=0.0)
            torch.testing.assert_close(whole[k].double(), refs[k], **tol)
            torch.testing.assert_close(torch.cat(got[k]).double(), refs[k], **tol)
    finally:
        unregister_architecture("ToyQKNormForCausalLM")
        MIXERS.unregister("toy_qk_norm_attention")


def run_toy_latent(dtype, device):
    """A mixer whose per-token cache is not keys and values: two planes of different widths and of an element type of
    their own (a compressed latent of 12 numbers and 4 position features, both float32 whatever the model's dtype),
    declared as one ``PagedNeed`` and read back through the block table.  Requests in portions and token by token,
    interleaved and with pages used again, give what whole requests give."""
    from torchlet_amd.config import BlockSpec, ModelConfig, ModelSpec, PartSpec, RMSNormSpec, RunEntry, SwiGLUSpec
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import build_model, make_runner
    from torchlet_amd.parts import MIXERS, Mixer, PagedNeed, WeightSpec
    from torchlet_amd.registry import config_class, register_architecture, unregister_architecture
    from torchlet_amd.weights.random_init import random_tensors

    H, LATENT, POS, VOCAB = 32, 12, 4, 30

    @dataclass(frozen=True)
    class LatentSpec(PartSpec):
        kind: ClassVar[str] = "toy_latent"
        hidden: int = 0

    @MIXERS.register("toy_latent")
    class LatentMixer(Mixer):
        """c_t = h_t W_c, p_t = (sin, cos)(pos * f); y_t = (sum_s a_ts c_s) W_o with a_t = softmax_s<=t(c_t.c_s + p_t.p_s)."""

        def weight_specs(self):
            return {"down.weight": WeightSpec((LATENT, self.spec.hidden)), "up.weight": WeightSpec((self.spec.hidden, LATENT))}

        def load_weights(self, tensors):
            self.down = self._place(tensors["down.weight"], "compute")
            self.up = self._place(tensors["up.weight"], "compute")

        def paged_need(self):
            return PagedNeed(num_heads=1, head_dim=0, planes=((1, LATENT), (1, POS)), dtype=torch.float32)

        def forward(self, h, ctx, cache):
            latent_plane, pos_plane = cache.planes                       # [pages, 1, page, 12] and [pages, 1, page, 4], float32
            assert latent_plane.dtype == pos_plane.dtype == torch.float32 and latent_plane.shape[-1] == LATENT and pos_plane.shape[-1] == POS
            page = cache.page_size
            c = h.float() @ self.down.float().T
            pos = ctx.positions.float()[:, None] * torch.tensor([0.3, 0.05], device=h.device)
            feat = torch.cat((pos.sin(), pos.cos()), dim=-1)
            table = ctx.block_tables[cache.group].long()
            req = ctx.token_req.long()
            where = table[req, ctx.positions.long() // page]
            latent_plane[where, 0, ctx.positions.long() % page] = c
            pos_plane[where, 0, ctx.positions.long() % page] = feat
            out = torch.empty((h.shape[0], LATENT), dtype=torch.float32, device=h.device)
            indptr, ctx_lens = ctx.req_indptr.tolist(), ctx.ctx_lens.tolist()
            for r in range(len(ctx_lens)):
                total = ctx_lens[r] + indptr[r + 1] - indptr[r]
                blocks = table[r, : -(-total // page)]
                cs = latent_plane[blocks, 0].reshape(-1, LATENT)[:total]
                ps = pos_plane[blocks, 0].reshape(-1, POS)[:total]
                for t in range(indptr[r], indptr[r + 1]):
                    n = ctx_lens[r] + t - indptr[r] + 1
                    a = torch.softmax(cs[:n] @ c[t] + ps[:n] @ feat[t], dim=0)
                    out[t] = a @ cs[:n]
            return (out @ self.up.float().T).to(h.dtype)

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyLatentForCausalLM"
        vocab_size: int

        def to_spec(self):
            norm = RMSNormSpec(dim=H, eps=1e-6)
            block = BlockSpec(mixer=LatentSpec(hidden=H), mixer_norm=norm, ffn_norm=norm, ffn=SwiGLUSpec(hidden=H, intermediate=48), mixer_name="mix")
            return ModelSpec(vocab_size=self.vocab_size, hidden=H, layers=(block, block), order=(RunEntry(0), RunEntry(1)),
                             final_norm=norm, tie_head=True, max_positions=4096)

    register_architecture(ToyConfig)
    try:
        cfg = config_class("ToyLatentForCausalLM").from_dict(dict(vocab_size=VOCAB))
        tensors = {k: (v * 8 if ".mix." in k else v) for k, v in random_tensors(cfg, seed=2, dtype=torch.float32).items()}
        model = build_model(cfg, dtype, device=device, tensors=tensors)
        runner = make_runner(model, page_size=4, num_pages=26, max_requests=3)
        group = runner.cache.groups[0]
        assert len(runner.cache.groups) == 1 and [tuple(t.shape) for t in group.tensors] == [(2, 26, 1, 4, LATENT), (2, 26, 1, 4, POS)]
        assert {t.dtype for t in group.tensors} == {torch.float32}
        g = torch.Generator().manual_seed(1)
        seqs = {k: torch.randint(0, VOCAB, (n,), generator=g).tolist() for k, n in (("a", 37), ("b", 18), ("c", 29))}
        whole = {}
        for k, v in seqs.items():                                       # one at a time: the next one uses the same pages again
            whole[k] = runner.step([StepEntry(k, v, list(range(len(v))))]).cpu()
            runner.release(k)
        got = {k: [] for k in seqs}
        done = {k: 0 for k in seqs}
        plan = [{"a": 9}, {"a": 1, "b": 7}, {"b": 1, "a": 14, "c": 2}, {"c": 5, "a": 1, "b": 10}, {"a": 12, "c": 22}]
        for step in plan:
            entries = [StepEntry(k, seqs[k][done[k]: done[k] + n], list(range(n))) for k, n in step.items()]
            out = runner.step(entries).cpu()
            at = 0
            for k, n in step.items():
                got[k].append(out[at: at + n]); at += n; done[k] += n
                if done[k] == len(seqs[k]):
                    runner.release(k)
            runner.cache.check()
        assert done == {k: len(v) for k, v in seqs.items()} and runner.cache.live_requests() == []
        tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)
        for k in seqs:
            torch.testing.assert_close(torch.cat(got[k]), whole[k], **tol)
        assert float(whole["a"].std()) > 0.05
    finally:
        unregister_architecture("ToyLatentForCausalLM")
        MIXERS.unregister("toy_latent")


def run_toy_norm(dtype, device):
    """A norm of another kind than the framework's (it centres the row before it scales it, and has a bias) in every
    place a norm stands, beside the framework's attention and feed-forward.  For a step of one token it offers itself
    unrun, as the framework's norm does (``Norm.lazy``), naming its kind: the attention and the feed-forward, whose
    kernels can make a root-mean-square norm inside and no other, must run it the usual way.  Requests token by
    token, in portions and whole agree with each other and with the library's layer norm."""
    from torchlet_amd.config import AttentionSpec, BlockSpec, ModelConfig, ModelSpec, PartSpec, RotarySpec, RunEntry, SwiGLUSpec
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import build_model, make_runner
    from torchlet_amd.parts import NORMS, Norm, WeightSpec
    from torchlet_amd.parts.base import LazyNorm
    from torchlet_amd.registry import config_class, register_architecture, unregister_architecture
    from torchlet_amd.weights.random_init import random_tensors

    H, HEADS, KVH, HD, INTER, VOCAB, EPS = 64, 4, 2, 16, 96, 70, 1e-5
    counts = {"offered": 0, "run_from_offer": 0}

    @dataclass(frozen=True)
    class CentredNormSpec(PartSpec):
        kind: ClassVar[str] = "toy_centred_norm"
        dim: int = 0

    @NORMS.register("toy_centred_norm")
    class CentredNorm(Norm):
        graph_safe = True

        def weight_specs(self):
            return {"weight": WeightSpec((self.spec.dim,), keep="stored", init="one_plus_normal"),
                    "bias": WeightSpec((self.spec.dim,), keep="stored")}

        def load_weights(self, tensors):
            self.weight = self._place(tensors["weight"], "stored").float()
            self.bias = self._place(tensors["bias"], "stored").float()

        def forward(self, stream, rows=None, gain=1.0):
            r = stream.residual
            if stream.pending is not None:
                add = stream.pending.float()
                r = r + (add.sum(0) if add.dim() == 3 else add)         # slabs of partial sums, or one tensor
            if rows is None:
                stream.residual.copy_(r)
                stream.pending = None
            else:
                r = r[rows.long()]
            y = torch.nn.functional.layer_norm(r, (self.spec.dim,), self.weight, self.bias, EPS) * gain
            return y.to(self.dtype)

        def lazy(self, stream):
            if stream.residual.shape[0] == 1:
                counts["offered"] += 1
                return _Counted(self, stream, "toy_centred_norm", weight=self.weight, bias=self.bias, eps=EPS)
            return None

    class _Counted(LazyNorm):
        def value(self):
            if self._value is None:
                counts["run_from_offer"] += 1
            return super().value()

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyCentredNormForCausalLM"
        vocab_size: int

        def to_spec(self):
            norm = CentredNormSpec(dim=H)
            block = BlockSpec(mixer=AttentionSpec(hidden=H, num_heads=HEADS, num_kv_heads=KVH, head_dim=HD, qkv_bias=True,
                                                  position=RotarySpec(head_dim=HD, theta=10000.0, max_positions=256)),
                              mixer_norm=norm, ffn_norm=norm, ffn=SwiGLUSpec(hidden=H, intermediate=INTER))
            return ModelSpec(vocab_size=self.vocab_size, hidden=H, layers=(block, block), order=(RunEntry(0), RunEntry(1)),
                             final_norm=norm, tie_head=False, max_positions=256)

    def plain_forward(w, ids):
        sub = lambda p: {k[len(p):]: v for k, v in w.items() if k.startswith(p)}
        T = len(ids)
        x = w["model.embed_tokens.weight"][torch.tensor(ids)]
        norm = lambda t, n: torch.nn.functional.layer_norm(t, (H,), n["weight"], n["bias"], EPS)
        for layer in range(2):
            lw = sub(f"model.layers.{layer}.")
            x = x + plain.gqa_attention(norm(x, sub(f"model.layers.{layer}.input_layernorm.")), sub(f"model.layers.{layer}.self_attn."),
                                        num_heads=HEADS, num_kv_heads=KVH, head_dim=HD, theta=10000.0, positions=torch.arange(T))
            x = x + plain.swiglu_ffn(norm(x, sub(f"model.layers.{layer}.post_attention_layernorm.")), sub(f"model.layers.{layer}.mlp."))
        return plain.linear(norm(x, sub("model.norm.")), w["lm_head.weight"])

    register_architecture(ToyConfig)
    try:
        cfg = config_class("ToyCentredNormForCausalLM").from_dict(dict(vocab_size=VOCAB))
        tensors = {k: (v * 4 if "proj" in k else v) for k, v in random_tensors(cfg, seed=15, dtype=torch.bfloat16).items()}
        assert tensors["model.layers.1.post_attention_layernorm.bias"].shape == (H,)
        model = build_model(cfg, dtype, device=device, tensors=tensors)
        assert model.graph_safe()
        runner = make_runner(model, page_size=8, num_pages=20, max_requests=2)
        g = torch.Generator().manual_seed(4)
        seqs = {"a": torch.randint(0, VOCAB, (37,), generator=g).tolist(), "b": torch.randint(0, VOCAB, (18,), generator=g).tolist()}
        refs = {k: plain_forward({n: t.double() for n, t in tensors.items()}, v) for k, v in seqs.items()}
        whole = {k: runner.step([StepEntry(k, v, list(range(len(v))))]).cpu() for k, v in seqs.items()}
        for k in seqs:
            runner.release(k)
        assert counts["offered"] == 0                     # steps of many rows: nothing offered
        singles = {k: [] for k in seqs}
        singles["a"].append(runner.step([StepEntry("a", seqs["a"][:20], list(range(20)))]).cpu())
        for t in seqs["a"][20:]:                          # one request, one token a step: the norms offer themselves
            singles["a"].append(runner.step([StepEntry("a", [t], [0])]).cpu())
        assert counts["offered"] == 2 * 2 * 17 and counts["run_from_offer"] == counts["offered"], counts
        singles["b"].append(runner.step([StepEntry("b", seqs["b"][:9], list(range(9)))]).cpu())
        for i in range(9, 18):                            # two requests a step: rows of two, nothing offered
            out = runner.step([StepEntry("b", [seqs["b"][i]], [0])]).cpu()
            singles["b"].append(out)
        tol = dict(atol=3e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=6e-2, rtol=5e-2)
        for k in seqs:
            torch.testing.assert_close(whole[k].double(), refs[k], **tol)
            torch.testing.assert_close(torch.cat(singles[k]).double(), refs[k], **tol)
        assert float(refs["a"].std()) > 0.05
    finally:
        unregister_architecture("ToyCentredNormForCausalLM")
        NORMS.unregister("toy_centred_norm")

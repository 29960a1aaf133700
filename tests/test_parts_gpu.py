"""Each part alone on the GPU against its plain formula, at sizes of its own, and a toy
mixer with fixed-size state registered from outside the framework."""
from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch

import plain_qwen2 as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


# Bounds are relative to the root mean square of the result, because the parts are tested at
# weights large enough for scores and sums to be of order 1 to 10.
# 32-bit: 2^-18 of the rms (64 ulp: sums over up to a few hundred terms and exp of scores of
# size ~10, each of which multiplies the 2^-24 rounding by about its size).  bfloat16: every stage of a part rounds its output to 8 bits of mantissa
# (half an ulp = 2^-9 of the value); a part chains up to four such stages and sums over their
# outputs, so the bound is 2^-6 of the result's root mean square (absolute) and 2^-6 relative.
def _tol(dtype, ref):
    if dtype == torch.float32:
        return dict(atol=2 ** -18 * max(1.0, float(ref.double().pow(2).mean().sqrt())), rtol=2e-5)
    return dict(atol=2 ** -6 * float(ref.double().pow(2).mean().sqrt()), rtol=2 ** -6)


def _ctx(cache, req_lens, ctx_lens, tile_sizes, want=()):
    """A step context for requests "r0", "r1", ... that already hold ``ctx_lens`` tokens."""
    from torchlet_amd.engine.batch import StepContext
    ids = [f"r{i}" for i in range(len(req_lens))]
    for r, c, n in zip(ids, ctx_lens, req_lens):
        if not cache.has(r):
            cache.add_request(r)
        assert cache.reserve(r, c + n)
    blocks = -(-max(c + n for c, n in zip(ctx_lens, req_lens)) // cache.page_size)
    ctx = StepContext(new_lens=req_lens, ctx_lens=ctx_lens, slots=[cache.slot(r) for r in ids],
                      token_ids=[0] * sum(req_lens), want_rows=list(want),
                      block_tables=[cache.block_table(g, ids, blocks) for g in range(len(cache.groups))],
                      tile_sizes=tile_sizes, device="cuda")
    for r, c, n in zip(ids, ctx_lens, req_lens):
        cache.commit(r, c + n)
    return ctx


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part_adds_the_pending_branch_in_32_bit(dtype):
    from torchlet_amd.config import RMSNormSpec
    from torchlet_amd.parts import NORMS, Stream
    norm = NORMS.build(RMSNormSpec(dim=200, eps=1e-5), dtype, torch.device("cuda"))
    w = 1 + 0.1 * torch.randn(200)
    norm.load_weights({"weight": w.to(torch.bfloat16)})
    assert norm.weight.dtype == (torch.bfloat16 if dtype == torch.bfloat16 else torch.float32)
    res, pend = torch.randn(6, 200).cuda() * 100, torch.randn(6, 200).to(dtype).cuda()
    stream = Stream(res.clone(), pend)
    h = norm.forward(stream)
    total = res.double() + pend.double()
    assert stream.pending is None
    torch.testing.assert_close(stream.residual.double(), total, atol=1e-5, rtol=1e-7)   # a bfloat16 sum would be off by ~0.4
    ref = plain.rms_norm(total, w.to(torch.bfloat16).double().cuda(), 1e-5)
    torch.testing.assert_close(h.double(), ref, **_tol(dtype, ref))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotary_part_alone(dtype):
    from torchlet_amd.config import RotarySpec
    from torchlet_amd.parts import POSITION_ENCODINGS
    rope = POSITION_ENCODINGS.build(RotarySpec(head_dim=48, theta=12345.0, max_positions=4096), dtype, torch.device("cuda"))
    q, k = torch.randn(9, 5, 48).to(dtype), torch.randn(9, 2, 48).to(dtype)
    pos = torch.tensor([0, 1, 2, 3, 100, 101, 1000, 2047, 4095], dtype=torch.int32)
    dq, dk = q.cuda(), k.cuda()
    rope.apply(dq, dk, pos.cuda())
    for got, x in ((dq, q), (dk, k)):
        ref = plain.rope_apply(x.double().transpose(0, 1), pos, 12345.0).transpose(0, 1)
        torch.testing.assert_close(got.cpu().double(), ref, **_tol(dtype, ref))


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part_alone(dtype):
    from torchlet_amd.config import SwiGLUSpec
    from torchlet_amd.parts import FEED_FORWARDS
    ffn = FEED_FORWARDS.build(SwiGLUSpec(hidden=72, intermediate=200), dtype, torch.device("cuda"))
    w = {"gate_proj.weight": torch.randn(200, 72) * 0.2, "up_proj.weight": torch.randn(200, 72) * 0.2,
         "down_proj.weight": torch.randn(72, 200) * 0.2}
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    ffn.load_weights(w)
    h = torch.randn(11, 72).to(dtype)
    y = ffn.forward(h.cuda(), None)
    ref = plain.swiglu_ffn(h.double(), {k: v.double() for k, v in w.items()})
    torch.testing.assert_close(y.cpu().double(), ref, **_tol(dtype, ref))


def test_swiglu_part_with_a_long_intermediate_hands_partial_sums_to_the_next_norm():
    """17 rows up over a long intermediate size and a narrow output: the down product comes back as
    slabs of partial sums, which the next norm adds into the residual in 32-bit."""
    from torchlet_amd.config import RMSNormSpec, SwiGLUSpec
    from torchlet_amd.parts import FEED_FORWARDS, NORMS, Stream
    hidden, inter, rows = 72, 8192, 24
    dev = torch.device("cuda")
    ffn = FEED_FORWARDS.build(SwiGLUSpec(hidden=hidden, intermediate=inter), torch.bfloat16, dev)
    w = {"gate_proj.weight": torch.randn(inter, hidden) * 0.2, "up_proj.weight": torch.randn(inter, hidden) * 0.2,
         "down_proj.weight": torch.randn(hidden, inter) * 0.03}
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    ffn.load_weights(w)
    h = torch.randn(rows, hidden).to(torch.bfloat16)
    y = ffn.forward(h.cuda(), None)
    assert y.dim() == 3 and y.dtype == torch.float32 and y.shape[1:] == (rows, hidden)
    ref = plain.swiglu_ffn(h.double(), {k: v.double() for k, v in w.items()})
    torch.testing.assert_close(y.sum(0).cpu().double(), ref, **_tol(torch.bfloat16, ref))
    norm = NORMS.build(RMSNormSpec(dim=hidden, eps=1e-6), torch.bfloat16, dev)
    norm.load_weights({"weight": torch.ones(hidden, dtype=torch.bfloat16)})
    res = torch.randn(rows, hidden).cuda()
    stream = Stream(res.clone(), y)
    norm.forward(stream)
    torch.testing.assert_close(stream.residual.cpu().double(), res.cpu().double() + y.sum(0).cpu().double(), atol=1e-5, rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kvh,hd,window,bias", [(6, 2, 32, None, True), (4, 4, 16, 9, False), (7, 1, 64, None, True)])
def test_attention_part_alone_whole_and_in_two_portions(dtype, heads, kvh, hd, window, bias):
    from torchlet_amd.cache.manager import CacheManager
    from torchlet_amd.config import AttentionSpec, RotarySpec
    from torchlet_amd.parts import MIXERS
    hidden, T, page = 40, 45, 8
    spec = AttentionSpec(hidden=hidden, num_heads=heads, num_kv_heads=kvh, head_dim=hd, qkv_bias=bias, window=window,
                         position=RotarySpec(head_dim=hd, theta=1e4, max_positions=128))
    attn = MIXERS.build(spec, dtype, torch.device("cuda"))
    g = torch.Generator().manual_seed(1)
    # weights sized so that scores are of order one: larger scores multiply the rounding of q and k
    w = {n: (torch.randn(s.shape, generator=g) * (0.12 if n.endswith("weight") else 0.2)).to(torch.bfloat16)
         for n, s in attn.weight_specs().items()}
    attn.load_weights(w)
    h = torch.randn(T, hidden, generator=g).to(dtype)
    ref = plain.gqa_attention(h.double(), {k: v.double() for k, v in w.items()}, num_heads=heads, num_kv_heads=kvh,
                              head_dim=hd, theta=1e4, positions=torch.arange(T), window=window)
    for cuts in ([T], [29, 16]):
        cache = CacheManager([(attn.paged_need(), None, None)], page_size=page, num_pages=16, max_requests=2,
                             dtype=dtype, device="cuda")
        outs, done = [], 0
        for n in cuts:
            ctx = _ctx(cache, [n], [done], {attn.tile_tokens})
            outs.append(attn.forward(h[done:done + n].cuda(), ctx, cache.layer_cache(0)))
            done += n
        torch.testing.assert_close(torch.cat(outs).cpu().double(), ref, **_tol(dtype, ref))


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_part_alone(dtype):
    from torchlet_amd.cache.manager import CacheManager
    from torchlet_amd.config import Qwen2Config
    from torchlet_amd.parts import BLOCKS, Stream
    cfg = Qwen2Config.from_dict(dict(vocab_size=50, hidden_size=48, num_hidden_layers=1, num_attention_heads=3,
                                     num_key_value_heads=1, intermediate_size=100, max_position_embeddings=64,
                                     rms_norm_eps=1e-5, rope_theta=1e4))
    block = BLOCKS.build(cfg.to_spec().layers[0], dtype, torch.device("cuda"))
    g = torch.Generator().manual_seed(2)
    w = {n: ((1.0 if s.init == "one_plus_normal" else 0.0) + torch.randn(s.shape, generator=g) * 0.1).to(torch.bfloat16)
         for n, s in block.weight_specs().items()}
    block.load_weights(w)
    x = torch.randn(20, 48, generator=g)
    cache = CacheManager([(block.mixer.paged_need(), None, None)], page_size=16, num_pages=4, max_requests=1, dtype=dtype, device="cuda")
    ctx = _ctx(cache, [20], [0], {block.mixer.tile_tokens})
    stream = block.forward(Stream(x.cuda().clone()), ctx, cache.layer_cache(0))
    got = stream.residual.double() + stream.pending.double()
    pc = plain.PlainConfig(cfg.to_dict())
    ref = plain.block(x.double(), {k: v.double() for k, v in w.items()}, pc, 0, torch.arange(20))
    torch.testing.assert_close(got.cpu(), ref, **_tol(dtype, ref))


# ---------------------------------------------------------------- a toy mixer from outside

@pytest.mark.parametrize("graphs", [False, True])
def test_toy_mixer_with_state_of_its_own_registers_builds_and_steps(tmp_path, graphs):
    """A mixer defined here -- a per-channel running average whose only memory is a
    fixed-size state per request -- is registered, put into a model through a configuration
    of its own, and stepped in portions and token by token, without touching the framework's files.
    It says it is ``graph_safe`` (a step of one token per request works from the step's device-side
    numbers only), so with ``graphs`` its decode steps are captured and replayed: the state tensor is a
    static buffer, and the padding rows of a replayed step use the state row that belongs to no request."""
    from torchlet_amd.config import BlockSpec, ModelConfig, ModelSpec, PartSpec, RMSNormSpec, RunEntry, SwiGLUSpec
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import build_model, make_runner
    from torchlet_amd.parts import MIXERS, Mixer, StateNeed, WeightSpec
    from torchlet_amd.parts.base import INIT_LAWS, register_init_law
    from torchlet_amd.registry import config_class, register_architecture, unregister_architecture
    from torchlet_amd.weights.random_init import random_tensors

    @dataclass(frozen=True)
    class DecaySpec(PartSpec):
        kind: ClassVar[str] = "toy_decay"
        hidden: int = 0

    @MIXERS.register("toy_decay")
    class DecayMixer(Mixer):
        """y_t = s_t with s_t = a * s_{t-1} + x_t per channel, a = sigmoid(decay)."""
        graph_safe = True

        def weight_specs(self):
            return {"decay": WeightSpec((self.spec.hidden,), keep="float32", init="toy_decay_logit")}

        def load_weights(self, tensors):
            self.decay = self._place(tensors["decay"], "float32")

        def state_need(self):
            return StateNeed((self.spec.hidden,), torch.float32)

        def forward(self, h, ctx, cache):
            a = torch.sigmoid(self.decay.float())
            if ctx.decode_only:          # one token per request: nothing of the step is read on the host
                slots = ctx.slots.long()
                s = a * cache.state[slots] + h.float()
                cache.state.index_copy_(0, slots, s)
                return s.to(h.dtype)
            out = torch.empty_like(h)
            indptr, slots = ctx.req_indptr.tolist(), ctx.slots.tolist()
            for r, slot in enumerate(slots):
                s = cache.state[slot]
                for t in range(indptr[r], indptr[r + 1]):
                    s = a * s + h[t].float()
                    out[t] = s.to(h.dtype)
                cache.state[slot] = s
            return out

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyDecayForCausalLM"
        vocab_size: int
        hidden_size: int
        num_hidden_layers: int
        intermediate_size: int

        def to_spec(self):
            norm = RMSNormSpec(dim=self.hidden_size, eps=1e-6)
            block = BlockSpec(mixer=DecaySpec(hidden=self.hidden_size), mixer_norm=norm, ffn_norm=norm,
                              ffn=SwiGLUSpec(hidden=self.hidden_size, intermediate=self.intermediate_size), mixer_name="mix")
            return ModelSpec(vocab_size=self.vocab_size, hidden=self.hidden_size, layers=(block,) * self.num_hidden_layers,
                             order=tuple(RunEntry(i) for i in range(self.num_hidden_layers)), final_norm=norm,
                             tie_head=True, max_positions=1 << 20)

    # a law of the random-weights mode that the framework does not have, added by name from here
    register_init_law("toy_decay_logit")(lambda shape, gen, device, std: torch.rand(shape, generator=gen, device=device) * 4 - 2)
    register_architecture(ToyConfig)
    try:
        cfg = config_class("ToyDecayForCausalLM").from_dict(dict(vocab_size=40, hidden_size=24, num_hidden_layers=2, intermediate_size=56))
        tensors = random_tensors(cfg, seed=9, dtype=torch.float32)
        assert "model.layers.1.mix.decay" in tensors and float(tensors["model.layers.1.mix.decay"].abs().max()) > 1.0   # U(-2, 2), not N(0, 0.02)
        model = build_model(cfg, "float32", tensors=tensors)
        runner = make_runner(model, page_size=16, num_pages=2, max_requests=3, use_graphs=graphs)
        assert runner.cache.groups == [] and runner.caches[0].state.shape == (4, 24) and runner.use_graphs == graphs
        seqs = {"a": torch.randint(0, 40, (23,)).tolist(), "b": torch.randint(0, 40, (9,)).tolist(), "c": torch.randint(0, 40, (31,)).tolist()}
        whole = {k: runner.step([StepEntry(k, v, list(range(len(v))))]).cpu() for k, v in seqs.items()}
        for k in seqs:
            runner.release(k)
        # three requests token by token from their first token on: steps of one token per request, replayed as
        # graphs of width four (one padding row) when graphs are on; "b" ends first and the width drops to two
        singles = {k: [] for k in seqs}
        for i in range(31):
            live = [k for k in seqs if i < len(seqs[k])]
            out = runner.step([StepEntry(k, [seqs[k][i]], [0]) for k in live]).cpu()
            for j, k in enumerate(live):
                singles[k].append(out[j: j + 1])
            for k in live:
                if i == len(seqs[k]) - 1:
                    runner.release(k)
        for k in seqs:
            torch.testing.assert_close(torch.cat(singles[k]), whole[k], atol=1e-5, rtol=1e-5)
        assert (runner.graph_replays > 20) == graphs
        del seqs["c"]
        # the same two requests interleaved, in portions: the state carries over by slot
        got = {"a": [], "b": []}
        got["a"].append(runner.step([StepEntry("a", seqs["a"][:7], list(range(7)))]).cpu())
        out = runner.step([StepEntry("b", seqs["b"][:4], list(range(4))), StepEntry("a", seqs["a"][7:8], [0])]).cpu()
        got["b"].append(out[:4]); got["a"].append(out[4:])
        out = runner.step([StepEntry("a", seqs["a"][8:], list(range(15))), StepEntry("b", seqs["b"][4:], list(range(5)))]).cpu()
        got["a"].append(out[:15]); got["b"].append(out[15:])
        for k in seqs:
            torch.testing.assert_close(torch.cat(got[k]), whole[k], atol=1e-5, rtol=1e-5)
        # and the whole pass equals a plain computation of the recurrence
        w = {k: v.double() for k, v in tensors.items()}
        x = w["model.embed_tokens.weight"][torch.tensor(seqs["a"])]
        for i in range(2):
            p = f"model.layers.{i}."
            h = plain.rms_norm(x, w[p + "input_layernorm.weight"], 1e-6)
            a, s, ys = torch.sigmoid(w[p + "mix.decay"]), torch.zeros(24, dtype=torch.float64), []
            for t in range(len(seqs["a"])):
                s = a * s + h[t]
                ys.append(s)
            x = x + torch.stack(ys)
            x = x + plain.swiglu_ffn(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-6),
                                     {k[len(p) + 4:]: v for k, v in w.items() if k.startswith(p + "mlp.")})
        ref = plain.rms_norm(x, w["model.norm.weight"], 1e-6) @ w["model.embed_tokens.weight"].T
        torch.testing.assert_close(whole["a"].double(), ref, atol=1e-5, rtol=1e-4)
    finally:
        unregister_architecture("ToyDecayForCausalLM")
        MIXERS.unregister("toy_decay")
        INIT_LAWS.pop("toy_decay_logit", None)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_routed_feed_forward_and_toy_position_encoding_with_a_layer_run_twice(dtype):
    import toy_parts
    toy_parts.run_toy_mix(dtype, torch.device("cuda"), _tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_attention_that_differs_in_one_stage(dtype):
    import toy_parts
    toy_parts.run_toy_qk_norm(dtype, torch.device("cuda"), _tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_mixer_whose_cache_planes_differ_in_width_and_element_type(dtype):
    import toy_parts
    toy_parts.run_toy_latent(dtype, torch.device("cuda"))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_norm_of_another_kind_is_run_and_never_taken_for_the_frameworks_own(dtype):
    import toy_parts
    toy_parts.run_toy_norm(dtype, torch.device("cuda"))

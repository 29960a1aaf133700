"""Attention at the context lengths the benchmark runs (2048 to 16 400 tokens and beyond), where the
kernels split a request's keys over many work-groups and merge the parts.

Kernel level: the decode kernel at the head layouts of the 7B and 14B/32B checkpoints with the split
count the attention mixer itself picks for the step, at explicit split counts up to 64, with a window,
and with block tables wider than 2048 entries; the 128-row prompt kernel for whole prompts of 2048 and
4096 tokens and for a 512-token portion deep into a prompt (tiles split over their keys and merged).
Places of the cache that hold no key are NaN, and a few far keys are scaled up so that losing one
shows.  The reference is the float64 formula on the GPU.

Engine level: two narrow two-layer models with 8192 positions, requests of 2048 to 5000 tokens, cut
whole, with the last 32 tokens one by one, in 512-token portions, and with a portion beside decode
tokens of other long requests, in both dtypes, against the plain implementation in float64.  Their
query and key projections are scaled up so that single far keys carry weight.
"""
import math
from types import SimpleNamespace

import pytest
import torch

import plain_qwen2 as plain
import scenarios

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from torchlet_amd.kernels import ops
    return ops


# ------------------------------------------------------------------------ kernel level

def _reference(q, k, v, window, chunk=128):
    """One request in float64 on the GPU: q [n, heads, hd] at the last n positions of k/v [total, kvh, hd]."""
    n, heads, hd = q.shape
    total, kvh, _ = k.shape
    ctx, group = total - n, heads // kvh
    q, k, v = q.double(), k.double().transpose(0, 1), v.double().transpose(0, 1)      # k, v: [kvh, total, hd]
    out = torch.empty((n, heads, hd), dtype=torch.float64, device=q.device)
    kpos = torch.arange(total, device=q.device)[None, :]
    for a in range(0, n, chunk):
        c = min(chunk, n - a)
        qq = q[a:a + c].view(c, kvh, group, hd).permute(1, 2, 0, 3)                   # [kvh, group, c, hd]
        s = torch.einsum("kgcd,ktd->kgct", qq, k) / math.sqrt(hd)
        qpos = ctx + a + torch.arange(c, device=q.device)[:, None]
        hide = kpos > qpos
        if window:
            hide = hide | (kpos <= qpos - window)
        s = s.masked_fill(hide[None, None], -torch.inf)
        out[a:a + c] = torch.einsum("kgct,ktd->ckgd", torch.softmax(s, -1), v).reshape(c, heads, hd)
    return out


class _Paged:
    """Keys and values of some requests scattered over the pages of a pool whose other places are NaN."""

    def __init__(self, totals, nkv, hd, page, seed, table_width=0, dtype=torch.bfloat16):
        g = torch.Generator(device="cuda").manual_seed(seed)
        blocks = [-(-t // page) for t in totals]
        pages = sum(blocks) + 1
        order = torch.randperm(pages - 1, generator=g, device="cuda").int() + 1
        self.table = torch.zeros((len(totals), max(max(blocks), table_width)), dtype=torch.int32, device="cuda")
        self.kp = torch.full((pages, nkv, page, hd), float("nan"), dtype=dtype, device="cuda")
        self.vp = torch.full((pages, nkv, hd, page), float("nan"), dtype=dtype, device="cuda")
        self.k, self.v = [], []
        at = 0
        for r, t in enumerate(totals):
            self.table[r, : blocks[r]] = order[at: at + blocks[r]]
            at += blocks[r]
            k = torch.randn((t, nkv, hd), generator=g, device="cuda")
            v = torch.randn((t, nkv, hd), generator=g, device="cuda")
            for far in {min(5, t - 1), t // 2, max(0, t - 1000)}:      # keys that stand out among thousands
                k[far] *= 3.0
            k, v = k.to(dtype), v.to(dtype)
            pos = torch.arange(t, device="cuda")
            pg, off = self.table[r][pos // page].long(), pos % page
            self.kp[pg, :, off] = k
            self.vp[pg, :, :, off] = v
            self.k.append(k)
            self.v.append(v)


def _mixer_splits(nh, nkv, hd, window, longest, tiles):
    """The split count the attention mixer picks for a decode step."""
    from torchlet_amd.config.base import AttentionSpec
    from torchlet_amd.parts.attention import GQAttention
    mixer = GQAttention(AttentionSpec(hidden=nh * hd, num_heads=nh, num_kv_heads=nkv, head_dim=hd, window=window or None),
                        torch.bfloat16, torch.device("cuda"))
    return mixer._splits(SimpleNamespace(max_total_len=longest, max_new_tokens=1), tiles)


def _check_rows(got, ref, v, what):
    # one bfloat16 rounding of the result, accumulated input rounding, and the probabilities' rounding to
    # bfloat16 before the product with V (2^-9 of each weight)
    torch.testing.assert_close(got, ref, rtol=1.6e-2, atol=2e-3 + 2 ** -9 * float(v.abs().max()), msg=lambda m: f"{what}: {m}")


CONTEXTS = [2047, 2048, 4100, 16400]


@pytest.mark.parametrize("nh,nkv", [(28, 4), (40, 8)])
@pytest.mark.parametrize("batch", [1, 8, 64])
def test_decode_attention_at_benchmark_contexts_with_the_mixers_own_split_count(ops, nh, nkv, batch):
    hd, page = 128, 16
    totals = [CONTEXTS[(i + 3) % len(CONTEXTS)] + 1 for i in range(batch)]       # cached keys + the new token's
    if batch == 64:
        totals = [t if i % 4 == 0 else min(t, 2049) for i, t in enumerate(totals)]   # a quarter of them long
    cache = _Paged(totals, nkv, hd, page, seed=batch + nh)
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randn((batch, nh * hd), generator=g, device="cuda").to(torch.bfloat16)
    ctx_lens = torch.tensor([t - 1 for t in totals], dtype=torch.int32, device="cuda")
    splits, waves = _mixer_splits(nh, nkv, hd, 0, max(totals), batch)
    print(f"heads {nh}/{nkv}, batch {batch}: {splits} splits, {waves} waves, longest {max(totals)}", flush=True)
    # work-groups of eight waves, one to a compute unit, while one per request and head group would leave units idle;
    # 64 requests with 8 groups of heads fill them twice with work-groups of four
    assert (splits, waves) == {1: (64, 8) if nkv == 4 else (32, 8), 8: (8, 8) if nkv == 4 else (4, 8), 64: (1, 8) if nkv == 4 else (1, 4)}[batch]
    out = torch.full((batch, nh * hd), float("nan"), dtype=torch.bfloat16, device="cuda")
    tq = ops.attention_tile_tokens(nh, nkv)
    ops.paged_attention(q, out, cache.kp, cache.vp, cache.table, None, ctx_lens, None, None, batch, tq,
                        nh, nkv, hd, page, 0, 1.0 / math.sqrt(hd), splits, waves=waves)
    for r in range(batch):
        ref = _reference(q[r: r + 1].view(1, nh, hd), cache.k[r], cache.v[r], 0)
        _check_rows(out[r].double().view(1, nh, hd), ref, cache.v[r], f"request {r} of {totals[r]} keys")


@pytest.mark.parametrize("dtype,general,waves", [(torch.bfloat16, False, 4), (torch.bfloat16, False, 8), (torch.float32, False, 4)])
@pytest.mark.parametrize("nh,nkv,hd,page,window,splits,totals,width", [
    (28, 4, 128, 16, 0, 8, [2500, 4999, 3000], 0),
    (28, 4, 128, 16, 0, 9, [2500, 4999, 3000], 0),          # the merge's second pass over the parts
    (40, 8, 128, 16, 0, 16, [4100, 2048], 2100),            # a table wider than 2048 entries, mostly unused
    (14, 2, 64, 8, 0, 64, [5000, 1, 300], 0),               # more parts than some requests have steps of keys
    (6, 2, 128, 16, 3000, 12, [4999, 3001, 2999], 0),       # a window that cuts into the long ones
    (28, 4, 128, 16, 0, 33, [40000, 33000], 0),             # 2500 pages in use
])
def test_decode_attention_split_many_ways(ops, dtype, general, waves, nh, nkv, hd, page, window, splits, totals, width):
    if dtype == torch.float32 and max(totals) > 5000:
        totals = [t // 8 + 2048 for t in totals]             # the 32-bit kernel is slow; its tables stay narrow
    cache = _Paged(totals, nkv, hd, page, seed=splits, table_width=width, dtype=dtype)
    R = len(totals)
    g = torch.Generator(device="cuda").manual_seed(7)
    q = torch.randn((R, nh * hd), generator=g, device="cuda").to(dtype)
    ctx_lens = torch.tensor([t - 1 for t in totals], dtype=torch.int32, device="cuda")
    out = torch.full((R, nh * hd), float("nan"), dtype=dtype, device="cuda")
    tq = ops.attention_tile_tokens(nh, nkv)
    ops.paged_attention(q, out, cache.kp, cache.vp, cache.table, None, ctx_lens, None, None, R, tq,
                        nh, nkv, hd, page, window, 1.0 / math.sqrt(hd), splits, general=general, waves=waves)
    for r in range(R):
        ref = _reference(q[r: r + 1].view(1, nh, hd), cache.k[r], cache.v[r], window)
        got = out[r].double().view(1, nh, hd)
        if dtype == torch.float32:
            torch.testing.assert_close(got, ref, rtol=2e-5, atol=4e-6)
        else:
            _check_rows(got, ref, cache.v[r], f"request {r} of {totals[r]} keys, {splits} splits")


@pytest.mark.parametrize("nh,nkv,hd,page,window,new,ctx,parts", [
    (28, 4, 128, 16, 0, 2048, 0, 1),           # the benchmark's prefill
    (40, 8, 128, 16, 0, 4096, 0, 1),
    (28, 4, 128, 16, 0, 512, 15872, 4),        # a portion deep into a prompt: few tiles, each split over its keys
    (40, 8, 128, 8, 0, 512, 15872, 4),         # 2048 pages: the most the kernel keeps in shared memory
    (12, 4, 64, 16, 3000, 700, 4000, 4),       # heads of 64, a window
    (40, 8, 128, 16, 0, 2048, 6144, 3),        # 656 tiles of about equal length: two rounds of work-groups whole, four thirds in three parts
    (28, 4, 128, 16, 0, 2048, 6144, 1),        # 456 tiles: one round
])
def test_prompt_attention_at_benchmark_lengths(ops, nh, nkv, hd, page, window, new, ctx, parts):
    from torchlet_amd.parts.attention import _prompt_splits
    total = ctx + new
    cache = _Paged([total], nkv, hd, page, seed=new + ctx)
    g = torch.Generator(device="cuda").manual_seed(9)
    q = torch.randn((new, nh * hd), generator=g, device="cuda").to(torch.bfloat16)
    tq = ops.prompt_attention_tile_tokens(nh, nkv)
    tok0 = list(range(0, new, tq))
    tiles = len(tok0)
    groups = tiles * nkv
    splits = _prompt_splits(groups, total if not window else min(total, window + tq), uniform=total >= 2 * new)   # as the attention mixer decides
    print(f"{new} new tokens on {ctx}: {tiles} tiles, {splits} splits", flush=True)
    assert splits == parts
    out = torch.full((new, nh * hd), float("nan"), dtype=torch.bfloat16, device="cuda")
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    extra = dict(max_total_len=total, splits=splits)
    if splits > 1:
        extra["merge_tokens"] = (torch.arange(new, dtype=torch.int32, device="cuda"), new)
    ops.paged_attention_prompt(q, out, cache.kp, cache.vp, cache.table, i32([0, new]), i32([ctx]), i32([0] * tiles), i32(tok0),
                               tiles, tq, nh, nkv, hd, page, window, 1.0 / math.sqrt(hd), **extra)
    ref = _reference(q.view(new, nh, hd), cache.k[0], cache.v[0], window)
    _check_rows(out.double().view(new, nh, hd), ref, cache.v[0], f"{new} tokens on {ctx}")


@pytest.mark.parametrize("nh,nkv,hd,page,window,new,ctx", [
    (28, 4, 128, 8, 0, 512, 20000),            # 2564 pages: more than the 128-row kernel keeps in shared memory
    (8, 2, 96, 16, 0, 512, 5000),              # a head size the 128-row kernel is not built for
    (6, 3, 112, 4, 3000, 300, 9000),           # pages of 4 tokens, a window
])
def test_prompt_attention_in_tiles_of_64_rows_at_real_lengths(ops, nh, nkv, hd, page, window, new, ctx):
    """The 64-row kernel for prompt portions is what serves sequences of more than 2048 pages and head sizes other
    than 64 and 128 from contexts of 4096 tokens on (``parts/attention.py``): here at those lengths, against the
    float64 formula, with NaN in every place of the cache that holds no key."""
    assert not ops.prompt_attention_fits(torch.bfloat16, hd, page, -(-(ctx + new) // page))      # the case the mixer sends here
    total = ctx + new
    cache = _Paged([total], nkv, hd, page, seed=new + ctx)
    g = torch.Generator(device="cuda").manual_seed(10)
    q = torch.randn((new, nh * hd), generator=g, device="cuda").to(torch.bfloat16)
    tq = ops.prefill_attention_tile_tokens(nh, nkv)
    tok0 = list(range(0, new, tq))
    out = torch.full((new, nh * hd), float("nan"), dtype=torch.bfloat16, device="cuda")
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    print(f"{new} new tokens on {ctx}: {len(tok0)} tiles of {tq} tokens, {cache.table.shape[1]} pages", flush=True)
    ops.paged_attention_prefill(q, out, cache.kp, cache.vp, cache.table, i32([0, new]), i32([ctx]), i32([0] * len(tok0)), i32(tok0),
                                len(tok0), tq, nh, nkv, hd, page, window, 1.0 / math.sqrt(hd))
    ref = _reference(q.view(new, nh, hd), cache.k[0], cache.v[0], window)
    _check_rows(out.double().view(new, nh, hd), ref, cache.v[0], f"{new} tokens on {ctx}")


# ------------------------------------------------------------------------ engine level

LONG = {
    # heads of 128 in groups of three, pages of 16
    "L1": dict(architectures=["Qwen2ForCausalLM"], vocab_size=300, hidden_size=192, num_hidden_layers=2,
               num_attention_heads=6, num_key_value_heads=2, head_dim=128, intermediate_size=320,
               max_position_embeddings=8192, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False),
    # heads of 64 in one group of four, a window of 1000 keys on the second layer (a second group of pages)
    "L2": dict(architectures=["Qwen2ForCausalLM"], vocab_size=211, hidden_size=128, num_hidden_layers=2,
               num_attention_heads=4, num_key_value_heads=1, head_dim=64, intermediate_size=200,
               max_position_embeddings=8192, rope_theta=5e5, rms_norm_eps=1e-5, tie_word_embeddings=True,
               use_sliding_window=True, sliding_window=1000, max_window_layers=1),
}
LONG_PAGE = {"L1": 16, "L2": 8}
LONG_LENGTHS = [2048, 4100, 5000]
SHARPEN = 6.0       # factor on the query and key projections: single far keys carry a few percent of the weight


def _long_steps(requests):
    """Ways of cutting that reach the long-context paths: whole prompts; all but the last 32 tokens, then
    singles; 512-token portions; and a request fed in 512-token portions while two others, already
    thousands of tokens long, decode beside it."""
    want_all = lambda t: list(range(len(t)))
    modes = {"whole": scenarios.whole(requests), "tail_singles": scenarios.tail_singles(requests)}
    modes["portions_512"] = scenarios.portions(requests, sizes=(512, 512, 490, 534, 512))
    ids = list(requests)
    a, b, c = (requests[i] for i in ids)
    tail = 8
    steps = [dict(entries=[dict(id=ids[0], tokens=a[:-tail], want=want_all(a[:-tail]))], end=[]),
             dict(entries=[dict(id=ids[1], tokens=b[:-tail], want=want_all(b[:-tail]))], end=[])]
    done, i = 0, 0
    while done < len(c):
        n = min(512, len(c) - done)
        entries = [dict(id=ids[2], tokens=c[done:done + n], want=list(range(n)))]
        if i < tail:
            entries = [dict(id=ids[0], tokens=[a[len(a) - tail + i]], want=[0]), entries[0],
                       dict(id=ids[1], tokens=[b[len(b) - tail + i]], want=[0])]
        done += n
        end = ([ids[0], ids[1]] if i == tail - 1 else []) + ([ids[2]] if done == len(c) else [])
        steps.append(dict(entries=entries, end=end))
        i += 1
    assert i >= tail
    modes["portion_beside_decodes"] = steps
    return modes


@pytest.fixture(scope="module", params=list(LONG))
def long_model(request):
    from torchlet_amd.registry import ARCHITECTURES
    from torchlet_amd.weights.random_init import random_tensors
    d = LONG[request.param]
    config = ARCHITECTURES["Qwen2ForCausalLM"].from_dict(d)
    tensors = random_tensors(config, seed=21, dtype=torch.bfloat16, device="cuda")
    for k in tensors:
        if "q_proj" in k or "k_proj" in k:
            tensors[k] = (tensors[k].float() * SHARPEN).to(torch.bfloat16)
    requests = scenarios.make_requests(d["vocab_size"], LONG_LENGTHS, seed=6)
    cfg = plain.PlainConfig(d)
    expected, noise, noise16, rms16 = scenarios.bounds_from_plain(cfg, tensors, requests)
    print(f"{request.param}: 32-bit noise {noise:.3e}, bfloat16 roundings move the logits by {noise16:.3e} at most, {rms16:.3e} rms", flush=True)
    # the attention is peaked: late queries of the first layer give their heaviest key far more than 1/T
    w = {k: v.double() for k, v in tensors.items()}
    ids = torch.tensor(requests["r2"], device="cuda")
    h = plain.rms_norm(w["model.embed_tokens.weight"][ids], w["model.layers.0.input_layernorm.weight"], cfg.eps)
    q = plain.linear(h, w["model.layers.0.self_attn.q_proj.weight"], w["model.layers.0.self_attn.q_proj.bias"])
    k = plain.linear(h, w["model.layers.0.self_attn.k_proj.weight"], w["model.layers.0.self_attn.k_proj.bias"])
    pos = torch.arange(len(ids), device="cuda")
    q = plain.rope_apply(q.view(-1, cfg.num_heads, cfg.head_dim).transpose(0, 1)[:, -64:], pos[-64:], cfg.theta)
    k = plain.rope_apply(k.view(-1, cfg.num_kv_heads, cfg.head_dim).transpose(0, 1), pos, cfg.theta)
    s = (q @ k.repeat_interleave(cfg.num_heads // cfg.num_kv_heads, 0).transpose(-1, -2)) / cfg.head_dim ** 0.5
    heaviest = float(torch.softmax(s, -1).max(-1).values.mean())
    print(f"{request.param}: the heaviest key of a late query holds {heaviest:.3f} of the weight", flush=True)
    assert heaviest > 20 / len(ids)
    del w
    yield request.param, config, tensors, requests, expected, (noise, noise16, rms16)
    del tensors
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_split_at_long_contexts(long_model, dtype):
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import build_model, make_runner
    name, config, tensors, requests, expected, (noise, noise16, rms16) = long_model
    rms = float(torch.cat([e.flatten() for e in expected.values()]).pow(2).mean().sqrt())
    if dtype == "float32":
        tol = dict(atol=8.0 * noise, rtol=2e-5)
    else:
        assert noise16 < 0.2 * rms, f"bfloat16 roundings alone move the logits by {noise16:.2e} at a size of {rms:.2e}"
        tol = dict(atol=2 * noise16, rtol=0.0)
    model = build_model(config, dtype, tensors=tensors)
    page = LONG_PAGE[name]
    for mode, steps in _long_steps(requests).items():
        steps = scenarios.number(steps)
        need = scenarios.max_tokens_needed(steps, unit=page)
        runner = make_runner(model, page_size=page, num_pages=-(-need // page) + 1, max_requests=4)
        for g in runner.cache.groups:
            for plane in g.tensors:
                plane.fill_(float("nan"))           # whatever an earlier request left in a page must not matter
                plane[:, 0] = 0                     # but the sentinel page, which masked places may read
        print(f"{name} {dtype} {mode}: {len(steps)} steps, {need} tokens of cache", flush=True)
        out = {}
        for s in steps:
            logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
            if logits is not None:
                out[s["step"]] = logits.cpu().numpy()
            for r in s["end"]:
                runner.release(r)
        runner.cache.check()
        assert runner.cache.live_requests() == []
        scenarios.check(steps, out, expected, tol, what=f"{name} {dtype} {mode}")
        if dtype == "bfloat16":
            err = scenarios.rms_error(steps, out, expected)
            print(f"    rms error {err:.3e} (roundings alone: {rms16:.3e})", flush=True)
            assert err <= 1.25 * rms16
        del runner
    del model
    torch.cuda.empty_cache()


# A sequence of more pages than the 128-row prompt kernel holds: with pages of 8 tokens its 2048 pages are 16 384 tokens.
BEYOND = dict(architectures=["Qwen2ForCausalLM"], vocab_size=170, hidden_size=128, num_hidden_layers=2,
              num_attention_heads=4, num_key_value_heads=2, head_dim=64, intermediate_size=176,
              max_position_embeddings=40960, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_that_cross_the_edge_of_2048_pages(dtype):
    """One request of 16 884 tokens in pages of 8: portions of 2048 tokens while the sequence has at most 2048 pages
    (the 128-row kernel in bfloat16), then portions of 1500, 1000 and 32 tokens, the second of which takes the
    sequence past 16 384 tokens (from there on the 64-row kernel), then 16 tokens one by one.  Logits of the last 64
    tokens of every early portion and of every token from position 14 336 on, against the plain implementation."""
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import build_model, make_runner
    from torchlet_amd.kernels import ops
    from torchlet_amd.registry import ARCHITECTURES
    from torchlet_amd.weights.random_init import random_tensors
    page, sizes = 8, [2048] * 7 + [1500, 1000, 32] + [1] * 16
    config = ARCHITECTURES["Qwen2ForCausalLM"].from_dict(BEYOND)
    tensors = random_tensors(config, seed=23, dtype=torch.bfloat16, device="cuda")
    for k in tensors:
        if "q_proj" in k or "k_proj" in k:
            tensors[k] = (tensors[k].float() * SHARPEN).to(torch.bfloat16)
    requests = scenarios.make_requests(BEYOND["vocab_size"], [sum(sizes)], seed=8)
    tokens = requests["r0"]
    expected, noise, noise16, rms16 = scenarios.bounds_from_plain(plain.PlainConfig(BEYOND), tensors, requests)
    print(f"32-bit noise {noise:.3e}; bfloat16 roundings move the logits by {noise16:.3e} at most, {rms16:.3e} rms", flush=True)
    tol = dict(atol=8.0 * noise, rtol=2e-5) if dtype == "float32" else dict(atol=2 * noise16, rtol=0.0)
    steps, done, kernels = [], 0, []
    for n in sizes:
        want = list(range(n)) if done >= 14336 else list(range(n - 64, n))
        steps.append(dict(entries=[dict(id="r0", tokens=tokens[done:done + n], want=want)], end=["r0"] if done + n == len(tokens) else []))
        done += n
        kernels.append(ops.prompt_attention_fits(torch.bfloat16, 64, page, -(-done // page)))
    assert kernels[:8] == [True] * 8 and not any(kernels[8:])          # the step of 1000 tokens is the first past the edge
    steps = scenarios.number(steps)
    model = build_model(config, dtype, tensors=tensors)
    runner = make_runner(model, page_size=page, num_pages=-(-len(tokens) // page) + 2, max_requests=1)
    for g in runner.cache.groups:
        for plane in g.tensors:
            plane.fill_(float("nan"))
            plane[:, 0] = 0
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        out[s["step"]] = logits.cpu().numpy()
        for r in s["end"]:
            runner.release(r)
    runner.cache.check()
    scenarios.check(steps, out, expected, tol, what=f"{dtype}, past 2048 pages")
    del runner, model, tensors
    torch.cuda.empty_cache()

"""Generation through the Python entry point and the command line on the GPU; long decoding
and the first tokens of a sequence through the step function."""
import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import plain_qwen2
import scenarios
import tiny_models

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
TOL = {"float32": scenarios.FP32_TOL, "bfloat16": scenarios.BF16_TOL}


def _follows_the_plain_argmax(cfg, w, prompt, output, slack):
    """Every generated token is the plain implementation's arg max, up to ``slack`` in the logit
    (a reduced-precision engine may pick another token among near-ties; the check then goes
    on along the engine's own tokens)."""
    ids = list(prompt)
    for tok in output:
        logits = plain_qwen2.forward(cfg, w, ids)[-1]
        assert float(logits.max() - logits[tok]) <= slack, f"token {tok} after {len(ids)} tokens is not an arg max"
        ids.append(tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(model_folders, dtype):
    """On configuration B, whose head is not tied to the embedding: its greedy tokens change from step to step, so
    an engine that lost what it cached would generate something else (with a tied head and small random weights the
    arg max is the input token itself, whatever the cache holds)."""
    from torchlet_amd import LLM
    cfg, w = plain_qwen2.load_folder(model_folders["B"])
    prompts = list(scenarios.make_requests(cfg.vocab, [5, 17, 33], seed=2).values())
    llm = LLM(str(model_folders["B"]), max_decode_slots=4, kv_block_size=8, dtype=dtype, max_num_batched_tokens=24)
    outs = llm.generate(prompts, max_new_tokens=8)
    assert [len(o) for o in outs] == [8, 8, 8]
    assert all(len(set(o)) >= 3 for o in outs), f"tokens that do not vary cannot show a lost cache: {outs}"
    for p, o in zip(prompts, outs):
        if dtype == "float32":
            assert o == plain_qwen2.greedy(cfg, w, p, 8)
        _follows_the_plain_argmax(cfg, w, p, o, 2 * TOL[dtype]["atol"])
    assert llm.generate([], max_new_tokens=4) == [] and llm.generate([[1, 2]], max_new_tokens=0) == [[]]
    with pytest.raises(ValueError, match="tokenizer"):
        llm.generate(["hello"])
    assert llm.runner.cache.live_requests() == []


def test_a_folder_stored_in_32_bit_gives_a_32_bit_engine(tmp_path):
    """No dtype named: the engine runs in the dtype the folder is stored in, as the reference types its parameters
    and its cache after the checkpoint (/root/reference/src/torchlet/utils.py:18-38,
    v10_triton_paged_gqa/engine.py:58).  The folder's config.json has no ``torch_dtype``: what it stores decides."""
    from torchlet_amd import LLM
    from torchlet_amd.engine.batch import StepEntry
    folder = tiny_models.write("B", tmp_path, dtype=torch.float32)
    assert "torch_dtype" not in json.loads((folder / "config.json").read_text())
    cfg, w = plain_qwen2.load_folder(folder)
    llm = LLM(str(folder), max_decode_slots=2, kv_block_size=8, use_graphs=False)
    assert llm.engine_config.dtype == "float32" and llm.model.dtype == torch.float32
    assert llm.model.blocks[0].mixer.w_qkv.dtype == torch.float32 and llm.model.embed.dtype == torch.float32
    assert {t.dtype for g in llm.runner.cache.groups for t in g.tensors} == {torch.float32}
    prompt = list(scenarios.make_requests(cfg.vocab, [29], seed=3).values())[0]
    assert llm.generate([prompt], max_new_tokens=8)[0] == plain_qwen2.greedy(cfg, w, prompt, 8)
    logits = llm.runner.step([StepEntry("x", prompt, list(range(len(prompt))))]).cpu()
    llm.runner.release("x")
    torch.testing.assert_close(logits.double(), plain_qwen2.forward(cfg, w, prompt), **scenarios.FP32_TOL)
    # the same folder with bfloat16 named: converted at load
    llm16 = LLM(str(folder), max_decode_slots=2, kv_block_size=8, dtype="bfloat16", use_graphs=False)
    assert llm16.model.dtype == torch.bfloat16 and llm16.model.embed.dtype == torch.bfloat16


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graphs_are_captured_before_the_first_request(model_folders, dtype):
    """``LLM`` captures the graph of every (batch width, context bucket) its configuration can reach when it is built
    (the reference captures its one shape inside its first decode step,
    /root/reference/src/torchlet/v10_triton_paged_gqa/engine.py:137-176): every decode step, the first one
    included, is a replay; no step stops to capture; what is generated is what the eager engine generates."""
    from torchlet_amd import LLM
    cfg, w = plain_qwen2.load_folder(model_folders["B"])            # 256 positions in pages of 8: one bucket of 32 pages
    llm = LLM(str(model_folders["B"]), max_decode_slots=4, kv_block_size=8, dtype=dtype, use_graphs=True)
    assert llm.runner.use_graphs and llm.graphs_captured == 3 and sorted(llm.runner._graphs) == [(1, 32), (2, 32), (4, 32)]
    assert llm.runner.graph_replays == 0
    prompts = list(scenarios.make_requests(cfg.vocab, [21, 6, 40], seed=5).values())
    one = llm.generate([prompts[0]], max_new_tokens=9)[0]
    assert llm.runner.graph_replays >= 8                               # eight decode steps, the first of them too
    replays = llm.runner.graph_replays
    three = llm.generate(prompts, max_new_tokens=12)
    assert llm.runner.graph_replays >= replays + 11
    assert len(llm.runner._graphs) == 3 and all(g.graph is not None for g in llm.runner._graphs.values())   # nothing captured later
    eager = LLM(str(model_folders["B"]), max_decode_slots=4, kv_block_size=8, dtype=dtype, use_graphs=False)
    assert eager.graphs_captured == 0
    assert eager.generate([prompts[0]], max_new_tokens=9)[0] == one and eager.generate(prompts, max_new_tokens=12) == three
    if dtype == "float32":
        assert one == plain_qwen2.greedy(cfg, w, prompts[0], 9)
    # a longer model in more buckets, sized by max_model_len
    cfgd = json.loads((model_folders["D"] / "config.json").read_text())         # 400 positions, pages of 8
    llm = LLM(str(model_folders["D"]), max_decode_slots=2, kv_block_size=8, dtype=dtype, use_graphs=True)
    assert sorted(llm.runner._graphs) == [(w_, b) for w_ in (1, 2) for b in (32, 50)] and cfgd["max_position_embeddings"] == 400
    llm = LLM(str(model_folders["D"]), max_decode_slots=2, kv_block_size=8, dtype=dtype, use_graphs=True, max_model_len=200)
    assert sorted(llm.runner._graphs) == [(1, 25), (2, 25)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [False, True])
def test_decode_steps_enqueued_ahead_of_their_tokens_generate_the_same(model_folders, dtype, graphs):
    """Decode steps that take their tokens on the GPU from the sampling kernel's output, enqueued
    while the host still waits for those tokens (eagerly and as replayed graphs): the same tokens
    as step after step, with a temperature, with requests that end at different times, and with a
    stop token that ends one of them a step before the host finds out."""
    from torchlet_amd import LLM
    cfg = json.loads((model_folders["D"] / "config.json").read_text())
    prompts = list(scenarios.make_requests(cfg["vocab_size"], [3, 40, 21], seed=4).values())

    def run(lookahead, stop=None):
        llm = LLM(str(model_folders["D"]), max_decode_slots=4, kv_block_size=8, dtype=dtype, use_graphs=graphs,
                  lookahead=lookahead, seed=5)
        outs = [llm.generate([p], max_new_tokens=n, temperature=t, seed=i, stop_token_ids=stop)[0]
                for i, (p, n, t) in enumerate(zip(prompts, (30, 9, 17), (0.0, 0.8, 0.0)))]
        together = llm.generate(prompts, max_new_tokens=24, temperature=0.7, seed=11, stop_token_ids=stop)
        assert llm.runner.cache.live_requests() == [] and llm.engine._ahead is None
        return llm, outs, together

    plain_llm, alone, together = run(False)
    ahead_llm, alone2, together2 = run(True)
    assert alone2 == alone and together2 == together
    assert plain_llm.engine.steps_ahead == 0 and ahead_llm.engine.steps_ahead >= 40
    if graphs:
        assert ahead_llm.runner.graph_replays > 20
    stop = [alone[0][12]]                                  # the first request meets it after 12 tokens, or earlier
    _, alone_s, together_s = run(False, stop)
    _, alone_s2, together_s2 = run(True, stop)
    assert alone_s2 == alone_s and together_s2 == together_s and len(alone_s[0]) <= 12


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("A", "bfloat16"), ("C", "float32"), ("C", "bfloat16")])
@pytest.mark.parametrize("seed", range(4))
def test_steps_ahead_under_random_arrivals_stop_tokens_and_few_pages_as_replayed_graphs(model_folders, name, dtype, seed):
    """The random workloads of the host test (arrivals at random steps, stop tokens, temperatures, pools
    so small that requests are preempted; C has a window and two groups of pages) on the GPU with decode
    steps replayed as graphs: what only the GPU can get wrong -- a page given back and used again behind a
    step that counts for nothing, the static logits of a replay overwritten by the next, the tokens copied
    inside the graph -- would change a token.  Graph steps pad their batch with rows that own no page:
    the sentinel page must come out of it unwritten."""
    from torchlet_amd.engine.loading import load_model
    _, model = load_model(model_folders[name], dtype)
    engine = scenarios.check_steps_ahead_on_a_random_workload(model, tiny_models.PAGE_SIZES[name], seed, use_graphs=True)
    assert engine.runner.graph_replays > 0 and engine.steps_ahead > 0
    for group in engine.runner.cache.groups:
        assert not any(bool(plane[:, 0].any()) for plane in group.tensors), "the sentinel page was written"


def test_continuous_batching_with_temperature_and_few_pages(model_folders):
    """Configuration B's workload (temperature 0.8, fixed seed, 12 new tokens, arrivals at steps
    0, 0, 3, 5) with so few pages that requests are preempted: tokens equal each request alone."""
    from torchlet_amd.engine.engine import Engine
    from torchlet_amd.engine.loading import load_model, make_runner
    from torchlet_amd.engine.request import Request
    cfg = json.loads((model_folders["B"] / "config.json").read_text())
    prompts = list(scenarios.make_requests(cfg["vocab_size"], [1, 9, 40, 64], seed=3).values())
    _, model = load_model(model_folders["B"], "float32")
    kw = dict(max_new_tokens=12, temperature=0.8)

    def engine(pages, budget):
        return Engine(make_runner(model, page_size=8, num_pages=pages, max_requests=4), max_tokens_per_step=budget, seed=42)

    alone = []
    for i, p in enumerate(prompts):
        e = engine(64, 256)
        r = Request(prompt_tokens=p, seed=i, **kw)
        e.add_request(r)
        e.run_until_done()
        alone.append(r.output_tokens)
    e = engine(16, 32)
    reqs = [Request(prompt_tokens=p, seed=i, **kw) for i, p in enumerate(prompts)]
    arrivals, step = {0: [0, 1], 3: [2], 5: [3]}, 0
    while step < 6 or e.has_work():
        for i in arrivals.get(step, []):
            e.add_request(reqs[i])
        if e.has_work():
            e.step()
        step += 1
    assert e.scheduler.num_preemptions > 0
    assert [r.output_tokens for r in reqs] == alone
    e.runner.cache.check()
    assert e.runner.cache.free_pages() == [15]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(model_folders, dtype):
    """One token per step from the very first position, for 250 steps, across many pages."""
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import load_model, make_runner
    name = "B"
    cfg, w = plain_qwen2.load_folder(model_folders[name])
    ids = torch.randint(0, cfg.vocab, (250,), generator=torch.Generator().manual_seed(8)).tolist()
    ref = plain_qwen2.forward(cfg, w, ids)
    _, model = load_model(model_folders[name], dtype)
    runner = make_runner(model, page_size=8, num_pages=34, max_requests=2)
    for i, t in enumerate(ids):
        got = runner.step([StepEntry("x", [t], [0])])[0].double().cpu()
        assert torch.allclose(got, ref[i], **TOL[dtype]), f"position {i}: max abs error {float((got - ref[i]).abs().max()):.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_shows_a_dropped_or_misplaced_key(model_folders, tmp_path, dtype):
    """With N(0, 0.02) weights every key weighs about the same and one wrong key among hundreds
    changes little.  Here q and k projections are scaled so that the softmax is peaked on single,
    far keys, and the token sequence is one whose last query gives its very first key a large share
    of its weight: a key lost at a page edge or a portion's start moves the logits visibly, in
    bfloat16 too, where the bound is what roundings to bfloat16 between the kernels alone do."""
    from safetensors.torch import load_file, save_file
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import load_model, make_runner
    sharpen = 12 if dtype == "float32" else 8
    folder = tmp_path / "sharp"
    folder.mkdir()
    (folder / "config.json").write_text((model_folders["B"] / "config.json").read_text())
    t = load_file(str(model_folders["B"] / "model.safetensors"))
    for k in t:
        if "q_proj" in k or "k_proj" in k:
            t[k] = (t[k].float() * sharpen).to(torch.bfloat16)
    save_file(t, str(folder / "model.safetensors"))
    cfg, w = plain_qwen2.load_folder(folder)
    T = 200

    def first_layer_weights(ids):
        h = plain_qwen2.rms_norm(w["model.embed_tokens.weight"][torch.tensor(ids)], w["model.layers.0.input_layernorm.weight"], cfg.eps)
        q = plain_qwen2.linear(h, w["model.layers.0.self_attn.q_proj.weight"], w["model.layers.0.self_attn.q_proj.bias"])
        k = plain_qwen2.linear(h, w["model.layers.0.self_attn.k_proj.weight"], w["model.layers.0.self_attn.k_proj.bias"])
        pos = torch.arange(len(ids))
        q = plain_qwen2.rope_apply(q.view(T, 3, 32).transpose(0, 1), pos, cfg.theta)
        k = plain_qwen2.rope_apply(k.view(T, 1, 32).transpose(0, 1), pos, cfg.theta).repeat_interleave(3, 0)
        return plain_qwen2.attention_weights(q, k)

    # a sequence whose last query leans on its first key (the one a lost page or a wrong window edge would drop)
    for seed in range(200):
        ids = torch.randint(0, cfg.vocab, (T,), generator=torch.Generator().manual_seed(seed)).tolist()
        aw = first_layer_weights(ids)
        if float(aw[:, -1, 0].max()) > 0.25:
            break
    else:
        raise AssertionError("no sequence whose last query leans on its first key")
    assert float(aw[:, 150:].max(-1).values.mean()) > 5 / T        # the weights are peaked
    ref = plain_qwen2.forward(cfg, w, ids)
    if dtype == "float32":
        # Scores of this size amplify 32-bit rounding: the plain implementation itself, run in 32-bit, is
        # off by ~1e-5 here (4e-7 on the unscaled model).  The bound is four times that measured rounding.
        _, w32 = plain_qwen2.load_folder(folder, torch.float32)
        noise = float((plain_qwen2.forward(cfg, w32, ids).double() - ref).abs().max())
        assert 1e-6 < noise < 1e-4
        bound = 4 * noise
    else:
        # what roundings to bfloat16 of everything separate kernels hand each other do to the logits, in a
        # 64-bit evaluation: the engine rounds at these places or fewer; the bound is twice the largest move
        moved = plain_qwen2.forward(cfg, w, ids, stored=lambda x: x.to(torch.bfloat16).double()) - ref
        bound = 2 * float(moved.abs().max())
    # the bound does catch a single lost key: the plain model with the oldest key hidden from the last
    # query only (a window of T - 1) differs by far more, in the one row that lost it
    lost = plain_qwen2.forward(plain_qwen2.PlainConfig({**json.loads((folder / "config.json").read_text()),
                               "use_sliding_window": True, "sliding_window": T - 1, "max_window_layers": 0}), w, ids)
    effect = float((lost - ref)[-1].abs().max())
    print(f"{dtype}: bound {bound:.3e}, one lost key moves the last row by {effect:.3e}", flush=True)
    assert float((lost - ref)[:-1].abs().max()) == 0.0 and effect > 3 * bound
    _, model = load_model(folder, dtype)
    runner = make_runner(model, page_size=8, num_pages=30, max_requests=1)
    got, done = [], 0
    for n in (61, 2, 70, 1, 1, 33, 32):
        got.append(runner.step([StepEntry("s", ids[done:done + n], list(range(n)))]).cpu())
        done += n
    torch.testing.assert_close(torch.cat(got).double(), ref, atol=bound, rtol=0)
    runner.release("s")
    # the last 39 tokens one by one: the last query reads its first key from the first page through the decode kernel
    got = [runner.step([StepEntry("s", ids[:161], list(range(161)))]).cpu()]
    got += [runner.step([StepEntry("s", [tok], [0])]).cpu() for tok in ids[161:]]
    torch.testing.assert_close(torch.cat(got).double(), ref, atol=bound, rtol=0)


def test_command_line(model_folders, tmp_path):
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(tiny_models.CONFIGS["B"]))      # untied head: tokens that vary, so a lost cache would show
    out = subprocess.run([sys.executable, "-m", "torchlet_amd", "init", "--config", str(cfg_path), "--seed", "1", "--out", str(tmp_path / "m")],
                         cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    run = subprocess.run([sys.executable, "-m", "torchlet_amd", "--model", str(tmp_path / "m"), "--prompt-ids", "5,6,7", "--prompt-ids", "9",
                          "--max-new-tokens", "4", "--dtype", "float32", "--verbose"], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr
    assert "backend:" in run.stderr and "model.embed_tokens.weight" in run.stderr and "EngineConfig(" in run.stderr      # --verbose
    lines = [json.loads(l) for l in run.stdout.strip().splitlines()]
    cfg, w = plain_qwen2.load_folder(tmp_path / "m")
    assert [l["output"] for l in lines] == [plain_qwen2.greedy(cfg, w, [5, 6, 7], 4), plain_qwen2.greedy(cfg, w, [9], 4)]
    assert len(set(lines[0]["output"])) >= 3
    # the replay program as a sub-command: the same options and files as bin/trace_run
    step = json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [5, 6, 7, 72, 73], "want": [0, 4]}], "end": ["a"]})
    rep = subprocess.run([sys.executable, "-m", "torchlet_amd", "replay", "--model", str(tmp_path / "m"), "--dtype", "float32",
                          "--out", str(tmp_path / "logits"), "--max-tokens", "64"], input=step + "\n", cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert rep.returncode == 0 and rep.stdout.strip() == "done 0", rep.stderr
    import numpy as np
    got = torch.from_numpy(np.fromfile(tmp_path / "logits" / "0.f32", dtype="<f4").reshape(2, cfg.vocab))
    torch.testing.assert_close(got.double(), plain_qwen2.forward(cfg, w, [5, 6, 7, 72, 73])[[0, 4]], **scenarios.FP32_TOL)


def _write_tokenizer(folder, vocab_size):
    """A word-level tokenizer over made-up words and a chat template in the manner of the
    checkpoints this architecture ships with, written with the ``tokenizers`` library."""
    import json
    from tokenizers import Tokenizer, models, pre_tokenizers
    special = ["<|im_start|>", "<|im_end|>", "<|endoftext|>"]
    words = special + ["user", "assistant", "\n"] + [f"w{i}" for i in range(vocab_size - 6)]
    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.Split(" ", "removed")
    tok.add_special_tokens(special)
    tok.save(str(folder / "tokenizer.json"))
    template = ("{% for m in messages %}<|im_start|> {{ m['role'] }} \n {{ m['content'] }} <|im_end|> \n {% endfor %}"
                "{% if add_generation_prompt %}<|im_start|> assistant \n{% endif %}")
    (folder / "tokenizer_config.json").write_text(json.dumps({"chat_template": template, "eos_token": "<|endoftext|>"}))
    return words


def test_strings_in_strings_out_through_a_tokenizer_and_its_chat_template(model_folders, tmp_path):
    """Prompts given as strings are wrapped as one user turn by the folder's chat template
    (/root/reference/src/torchlet/v10_triton_paged_gqa/llm.py:87-95), generation stops at the
    template's end-of-turn token or the tokenizer's end token (llm.py:40-44), and the answer
    comes back as text without special tokens (engine.py:194-196)."""
    import shutil
    from torchlet_amd import LLM
    folder = tmp_path / "with_tokenizer"
    shutil.copytree(model_folders["A"], folder)
    cfg, w = plain_qwen2.load_folder(folder)
    words = _write_tokenizer(folder, cfg.vocab)
    llm = LLM(str(folder), max_decode_slots=2, dtype="float32")
    assert llm.stop_ids == frozenset({1, 2})
    text, ids = llm.tokenizer.encode_chat("w7 w8 w9")
    assert [words[i] for i in ids] == ["<|im_start|>", "user", "\n", "w7", "w8", "w9", "<|im_end|>", "\n", "<|im_start|>", "assistant", "\n"]
    outs = llm.generate(["w7 w8 w9", "w20"], max_new_tokens=12)
    for prompt, out in zip(["w7 w8 w9", "w20"], outs):
        _, ids = llm.tokenizer.encode_chat(prompt)
        expected = plain_qwen2.greedy(cfg, w, ids, 12, stop_ids=(1, 2))
        assert out == " ".join(words[t] for t in expected if t > 2) or out == llm.tokenizer.decode(expected)
        assert "<|" not in out


def test_concurrent_callers_share_the_engines_steps(model_folders):
    """Three callers of the coroutine form arrive one after the other, as in the reference's own
    demonstration (/root/reference/src/torchlet/v10_triton_paged_gqa/llm.py:113-140): their
    requests run in the same steps, and each gets what it would have got alone."""
    import asyncio
    from torchlet_amd import LLM
    cfg, w = plain_qwen2.load_folder(model_folders["B"])           # untied head: tokens that vary
    prompts = list(scenarios.make_requests(cfg.vocab, [9, 30, 4], seed=7).values())
    llm = LLM(str(model_folders["B"]), max_decode_slots=4, kv_block_size=8, dtype="float32", max_num_batched_tokens=16)

    async def caller(i):
        for _ in range(2 * i):
            await asyncio.sleep(0)          # arrive a few steps later than the caller before
        return (await llm.generate_async([prompts[i]], max_new_tokens=10))[0]

    async def main():
        return await asyncio.gather(*(caller(i) for i in range(3)))

    steps_before = llm.engine.steps
    outs = asyncio.run(main())
    for p, o in zip(prompts, outs):
        assert o == plain_qwen2.greedy(cfg, w, p, 10) and len(set(o)) >= 2
    alone = sum(-(-len(p) // 16) + 9 for p in prompts)
    assert llm.engine.steps - steps_before < alone, "the callers' requests did not share steps"
    assert llm.runner.cache.live_requests() == []

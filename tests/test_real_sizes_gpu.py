"""The engine at the layer widths of the 0.5B to 32B checkpoints (all heads, groups,
intermediate sizes and the whole vocabulary, one or two layers, random weights) against the
plain implementation, under every way of cutting the requests into steps.

The plain implementation runs on the GPU here, in 64-bit, through library routines only; it
shares no code with the engine.  The 32-bit bound is set from the plain implementation
itself: its own 32-bit evaluation differs from the 64-bit one by rounding that depends on
the order of summation only, and an engine that sums the same terms in another order may
differ by a small multiple of that and no more.  The bfloat16 bound comes from the plain
implementation as well: evaluated in 64-bit, but with every tensor that separate kernels hand
to each other through memory (normalised activations, projections, rotated heads, mixed heads,
branch outputs) rounded to bfloat16, it moves away from the unrounded result by what such
roundings alone do.  The engine rounds at these places or at fewer (the residual, the norms and
the softmax stay in 32-bit), in another order of summation, so its error has the same law; the
bound is twice the largest such move, over all logits of all requests, and the root mean
square of the engine's error, an average over tens of millions of logits and so a sharp
figure, may exceed that of the moves by a quarter at most."""
import pytest
import torch

import plain_qwen2 as plain
import scenarios

pytestmark = pytest.mark.gpu

SHAPES = {
    "0.5B": dict(num_hidden_layers=3, hidden_size=896, num_attention_heads=14, num_key_value_heads=2,
                 intermediate_size=4864, rms_norm_eps=1e-6, vocab_size=151936, tie_word_embeddings=True),
    "1.5B": dict(num_hidden_layers=2, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2,
                 intermediate_size=8960, rms_norm_eps=1e-6, vocab_size=151936, tie_word_embeddings=True),
    "3B": dict(num_hidden_layers=2, hidden_size=2048, num_attention_heads=16, num_key_value_heads=2,
               intermediate_size=11008, rms_norm_eps=1e-6, vocab_size=151936, tie_word_embeddings=True),
    "7B": dict(num_hidden_layers=2, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
               intermediate_size=18944, rms_norm_eps=1e-6),
    "14B": dict(num_hidden_layers=1, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                intermediate_size=13824, rms_norm_eps=1e-5),
    "32B": dict(num_hidden_layers=1, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                intermediate_size=27648, rms_norm_eps=1e-5),
}
COMMON = dict(architectures=["Qwen2ForCausalLM"], vocab_size=152064, max_position_embeddings=4096, rope_theta=1e6,
              attention_bias=True, tie_word_embeddings=False)
LENGTHS = [150, 70, 200, 40, 97]
PAGE = 16
NOISE_FACTOR = 8.0


@pytest.fixture(scope="module", params=list(SHAPES))
def sized(request):
    from torchlet_amd.registry import ARCHITECTURES
    from torchlet_amd.weights.random_init import random_tensors
    d = dict(COMMON, **SHAPES[request.param])
    config = ARCHITECTURES["Qwen2ForCausalLM"].from_dict(d)
    seed = 2 + list(SHAPES).index(request.param)
    tensors = random_tensors(config, seed=seed, dtype=torch.bfloat16, device="cuda")
    requests = scenarios.make_requests(d["vocab_size"], LENGTHS, seed=5)
    cfg = plain.PlainConfig(d)
    expected, noise, noise16, rms16 = scenarios.bounds_from_plain(cfg, tensors, requests)
    torch.cuda.empty_cache()
    print(f"{request.param}: 32-bit noise {noise:.3e}, bfloat16 roundings move the logits by {noise16:.3e} at most, {rms16:.3e} rms", flush=True)
    yield request.param, config, tensors, requests, expected, (noise, noise16, rms16)
    del tensors
    torch.cuda.empty_cache()


def _replay(model, steps, max_tokens):
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner
    runner = make_runner(model, page_size=PAGE, num_pages=-(-max_tokens // PAGE) + 1, max_requests=4)
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            out[s["step"]] = logits.cpu().numpy()
        for r in s["end"]:
            runner.release(r)
    runner.cache.check()
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_split_at_checkpoint_widths(sized, dtype):
    from torchlet_amd.engine.loading import build_model
    name, config, tensors, requests, expected, (noise, noise16, rms16) = sized
    rms = float(torch.cat([e.flatten() for e in expected.values()]).pow(2).mean().sqrt())
    assert 0 < noise < 1e-3 * rms, f"the plain implementation's own 32-bit rounding ({noise:.2e}) should be far below the logits' size ({rms:.2e})"
    if dtype == "float32":
        tol = dict(atol=NOISE_FACTOR * noise, rtol=2e-5)
    else:
        assert noise16 < 0.1 * rms, f"bfloat16 roundings alone move the logits by {noise16:.2e} at a size of {rms:.2e}: too coarse a yardstick"
        tol = dict(atol=2 * noise16, rtol=0.0)
    model = build_model(config, dtype, tensors=tensors)
    modes = {
        "whole": scenarios.whole(requests),
        "tail_singles": scenarios.tail_singles(requests),
        "portions": scenarios.portions(requests),
        "mixed": scenarios.mixed(requests, seed=3),
    }
    for mode, steps in modes.items():
        steps = scenarios.number(steps)
        print(f"{name} {dtype} {mode}: {len(steps)} steps", flush=True)
        out = _replay(model, steps, scenarios.max_tokens_needed(steps, unit=PAGE))
        scenarios.check(steps, out, expected, tol, what=f"{name} {dtype} {mode}")
        if dtype == "bfloat16":
            err = scenarios.rms_error(steps, out, expected)
            print(f"    rms error {err:.3e}", flush=True)
            assert err <= 1.25 * rms16, f"{name} {mode}: rms error {err:.3e}, bfloat16 roundings alone give {rms16:.3e}"
    del model
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape,batch", [("7B", 8), ("14B", 8), ("7B", 1), ("7B", 64)])
def test_the_benchmarks_own_steps_at_checkpoint_widths(shape, batch, dtype):
    """What the benchmark times, with its logits looked at: the widths of the 7B checkpoint (two layers, the whole
    vocabulary; and of the 14B one, 40 heads in 8 groups, one layer), 8 requests with 2048-token prompts, each prefilled whole in one step (the 128-row prompt kernel
    over 456 tiles, the large tiles of the products), then four decode steps of all 8 as replayed graphs (keys in
    16 parts and their merge, the few-rows products with rotation and cache write in their epilogue, products
    split over K whose slabs the norms add up); and the benchmark's other two points, one request (norms made
    inside the kernels that read them) and 64 (the tile kernels of 17 rows up, the rotation kernel that adds up
    the projection's slabs).  Every logit row of up to 8 of the requests against the plain implementation in
    64-bit, with the bounds derived from the plain implementation as above."""
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import build_model, make_runner
    from torchlet_amd.registry import ARCHITECTURES
    from torchlet_amd.weights.random_init import random_tensors
    prompt, new = 2048, 4
    d = dict(COMMON, **SHAPES[shape])
    config = ARCHITECTURES["Qwen2ForCausalLM"].from_dict(d)
    tensors = random_tensors(config, seed=21, dtype=torch.bfloat16, device="cuda")
    requests = scenarios.make_requests(d["vocab_size"], [prompt + new] * batch, seed=9)
    cfg = plain.PlainConfig(d)
    rows = new + 1                       # the prompt's last position and the four decoded ones
    checked = {r: requests[r] for r in list(requests)[:: max(1, batch // 8)]}
    w64 = {k: v.double() for k, v in tensors.items()}
    expected = {r: plain.forward(cfg, w64, t, last=rows).cpu() for r, t in checked.items()}
    rounded = lambda t: t.to(torch.bfloat16).double()
    moved = torch.stack([plain.forward(cfg, w64, t, stored=rounded, last=rows).cpu() - expected[r] for r, t in checked.items()])
    del w64
    w32 = {k: v.float() for k, v in tensors.items()}
    noise = max(float((plain.forward(cfg, w32, t, last=rows).cpu().double() - expected[r]).abs().max()) for r, t in checked.items())
    del w32
    torch.cuda.empty_cache()
    noise16, rms16 = float(moved.abs().max()), float(moved.pow(2).mean().sqrt())
    rms = float(torch.stack(list(expected.values())).pow(2).mean().sqrt())
    print(f"32-bit noise {noise:.3e}, bfloat16 roundings move the logits by {noise16:.3e} at most, {rms16:.3e} rms, logits {rms:.3e} rms", flush=True)
    assert 0 < noise < 1e-3 * rms and noise16 < 0.1 * rms
    tol = dict(atol=NOISE_FACTOR * noise, rtol=2e-5) if dtype == "float32" else dict(atol=2 * noise16, rtol=0.0)

    model = build_model(config, dtype, tensors=tensors)
    del tensors
    runner = make_runner(model, page_size=PAGE, num_pages=batch * (-(-(prompt + new) // PAGE)) + 1, max_requests=batch, use_graphs=True)
    errors = []

    def compare(logits, place, row_of):
        got = logits.double().cpu()
        for i, r in enumerate(requests):
            if r not in expected:
                continue
            ref = expected[r][row_of]
            if not torch.allclose(got[i], ref, **tol):
                raise AssertionError(f"{shape} {dtype}: request {r} {place}: max abs error {float((got[i] - ref).abs().max()):.3e}, allowed {tol['atol']:.3e}")
            errors.append(got[i] - ref)

    first = [runner.step([StepEntry(r, t[:prompt], [prompt - 1])]) for r, t in requests.items()]
    compare(torch.cat(first), "after its prompt", 0)
    for n in range(new):
        logits = runner.step([StepEntry(r, [t[prompt + n]], [0]) for r, t in requests.items()])
        compare(logits, f"decode step {n}", 1 + n)
    assert runner.graph_replays >= new - 1        # (the first of them may be the run that captures the graph)
    if dtype == "bfloat16":
        err = float(torch.stack(errors).pow(2).mean().sqrt())
        print(f"    rms error {err:.3e}", flush=True)
        assert err <= 1.25 * rms16, f"rms error {err:.3e}, bfloat16 roundings alone give {rms16:.3e}"

"""Random configurations of the architecture through the engine, against the plain model: a fixed
list of seeds, each of which draws every size and option (head counts and groups, head sizes, widths
that are no power of two, experts, top-k, renormalisation, shared expert, windows, dense layers, tied
head), the requests' lengths and the page size.  Three of the seeds are configurations that once
overshot the bfloat16 bound (outlier logits of a tied head; a router of 64 near-uniform experts)."""
import random

import pytest

import replay_util as ru

pytestmark = pytest.mark.gpu

TOL = (5e-6, 2e-5)      # float32: absolute, relative (see test_gpu_engine.TOL); bfloat16: the rounding model


def narrow_config(rng):
    hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
    nkv = rng.choice([1, 2, 3, 5])
    nh = nkv * rng.choice([1, 2, 3, 4, 7])
    hidden = rng.choice([64, 72, 100, 136, 192, 264])
    E = rng.choice([1, 2, 3, 7, 16, 33, 64])
    k = rng.randint(1, min(E, 8))
    L = rng.randint(1, 3)
    im = rng.choice([16, 24, 40, 72, 100])
    shared = rng.choice([0, im, 2 * im, 3 * im, 52])
    win = rng.choice([0, 5, 16, 37, 64])
    return {
        "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
        "num_hidden_layers": L, "hidden_size": hidden, "num_attention_heads": nh, "num_key_value_heads": nkv,
        "head_dim": hd, "num_experts": E, "num_experts_per_tok": k, "norm_topk_prob": rng.random() < 0.5,
        "moe_intermediate_size": im, "shared_expert_intermediate_size": shared,
        "intermediate_size": rng.choice([48, 100, 136]), "decoder_sparse_step": rng.choice([1, 1, 2]),
        "mlp_only_layers": [0] if rng.random() < 0.2 else [], "vocab_size": rng.choice([97, 256, 331, 1000, 1537]),
        "rope_theta": rng.choice([10000.0, 1e6]), "rms_norm_eps": rng.choice([1e-6, 1e-5]),
        "max_position_embeddings": 512, "use_sliding_window": win > 0, "sliding_window": win or 4096,
        "max_window_layers": rng.randint(0, L), "tie_word_embeddings": rng.random() < 0.5,
    }


def wide_config(rng):
    hd = rng.choice([64, 128])
    nkv = rng.choice([1, 2, 4, 8])
    nh = nkv * rng.choice([1, 2, 4, 7])
    hidden = rng.choice([512, 1024, 1536, 2048, 2560, 1096])
    E = rng.choice([4, 8, 24, 60])
    k = rng.randint(1, min(E, 8))
    im = rng.choice([256, 384, 704, 1408, 200])
    shared = rng.choice([0, 2 * im, 4 * im, 520])
    win = rng.choice([0, 0, 100, 257])
    return {
        "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
        "num_hidden_layers": 1, "hidden_size": hidden, "num_attention_heads": nh, "num_key_value_heads": nkv,
        "head_dim": hd, "num_experts": E, "num_experts_per_tok": k, "norm_topk_prob": rng.random() < 0.5,
        "moe_intermediate_size": im, "shared_expert_intermediate_size": shared, "intermediate_size": 1024,
        "decoder_sparse_step": 1, "mlp_only_layers": [], "vocab_size": rng.choice([500, 777, 1024]),
        "rope_theta": 1e6, "rms_norm_eps": 1e-6, "max_position_embeddings": 4096,
        "use_sliding_window": win > 0, "sliding_window": win or 4096, "max_window_layers": 0,
        "tie_word_embeddings": rng.random() < 0.5,
    }


def draw(seed: int, wide: bool):
    """(configuration, request lengths, page size): one stream of draws per seed"""
    rng = random.Random(seed)
    cfg = wide_config(rng) if wide else narrow_config(rng)
    lengths = [rng.randint(1, 150) for _ in range(rng.randint(2, 5))]
    if wide:
        lengths = [rng.randint(100, 700), rng.randint(20, 300)]
    bs = rng.choice([8, 16, 64])
    if wide:
        bs = rng.choice([16, 64])
    return cfg, lengths, bs


SEEDS = [(3, False), (23, False), (101, False), (222, False), (347, False), (556, False), (699, False),
         (812, False), (940, False), (1003, True), (1027, True), (2044, True)]


@pytest.mark.parametrize("seed,wide", SEEDS)
def test_random_configuration(seed, wide, tmp_path):
    from ferrox_amd.engine.loading import load_model, write_random_model
    from ferrox_amd.engine.runner import ModelRunner
    cfg, lengths, bs = draw(seed, wide)
    print(f"seed {seed}: page size {bs}, lengths {lengths}, {cfg}", flush=True)
    reqs = ru.make_requests(cfg["vocab_size"], lengths, seed)
    for dtype in ("float32", "bfloat16"):
        folder = str(tmp_path / dtype)
        write_random_model(dict(cfg), folder, seed, "bfloat16" if wide else dtype)
        model = load_model(folder, dtype, "cuda:0")
        kinds = {"whole": lambda: ru.trace_whole(reqs), "mixed": lambda: ru.trace_mixed(reqs, seed=seed),
                 "tail": lambda: ru.trace_tail_decode(reqs), "portions": lambda: ru.trace_portions(reqs)}
        for kind in (("whole", "mixed", "tail") if wide else ("mixed", "tail", "portions")):
            steps = kinds[kind]()
            pages = ru.max_live_tokens(steps, bs) // bs
            runner = ModelRunner(model, block_size=bs, num_pages=pages, max_seqs=4)
            routing = {} if dtype == "bfloat16" else None
            got = ru.run_trace(runner, steps, routing)
            assert runner.manager.n_free_pages() == pages
            if dtype == "bfloat16":
                ru.compare(got, folder, reqs, 0.0, 0.0, f"seed {seed} {dtype} {kind}", routing, storage="bfloat16")
            else:
                ru.compare(got, folder, reqs, TOL[0] * (max(cfg["hidden_size"], 64) / 64) ** 0.5, TOL[1],
                           f"seed {seed} {dtype} {kind}", routing)
        del model
        ru._plain_cache.clear()
        ru._stored_cache.clear()
        ru._plain_model.cache_clear()

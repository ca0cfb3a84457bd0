"""Every head size from 16 to 256 in steps of 16, with head counts, groups, widths, inner sizes and
vocabularies that change with it (most of them no power of two, some no multiple of 8): each
model is stepped through portions of prompts beside decoded tokens and compared with the plain
implementation, in float32 and in bfloat16.  A head size beyond what the kernels take is refused
when the model is built, with an error that says so."""

import pytest
import torch

import helpers
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu

KV_HEADS = [1, 2, 3, 4, 5, 8]
GROUPS = [1, 2, 3, 4, 5, 6, 7, 8]
WIDTHS = [72, 100, 136, 200, 264, 328, 520, 40]
INNER = [24, 40, 88, 176, 200, 344, 520, 1000]
VOCAB = [97, 256, 509, 1003, 2049]


def config_of(i: int, head_dim: int) -> dict:
    kv, group = KV_HEADS[i % 6], GROUPS[(3 * i) % 8]
    while kv * group * head_dim > 1536 and group > 1:
        group -= 1
    while kv * group * head_dim > 1536 and kv > 1:
        kv -= 1
    heads = kv * group
    cfg = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "hidden_size": heads * head_dim if i % 2 else WIDTHS[(i // 2) % 8], "head_dim": head_dim,
        "num_hidden_layers": 1 + i % 3, "num_attention_heads": heads, "num_key_value_heads": kv,
        "intermediate_size": INNER[i % 8] + (1 if i % 4 == 3 else 0), "vocab_size": VOCAB[i % 5],
        "rope_theta": [10000.0, 1000000.0, 500.0][i % 3], "rms_norm_eps": [1e-6, 1e-5, 1e-3][(i + 1) % 3],
        "tie_word_embeddings": i % 2 == 0, "max_position_embeddings": 256,
    }
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("i", range(16))
def test_head_sizes_in_steps_of_16(tmp_path, i, dtype):
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.context import StepEntry
    from from_scratch_inference_engine_amd.engine.model import Runner

    head_dim = 16 * (i + 1)
    cfg = config_of(i, head_dim)
    print(f"head_dim {head_dim}: {cfg['num_attention_heads']}/{cfg['num_key_value_heads']} heads, width "
          f"{cfg['hidden_size']}, inner {cfg['intermediate_size']}, vocabulary {cfg['vocab_size']}, "
          f"{cfg['num_hidden_layers']} layers, {dtype}", flush=True)
    d = helpers.make_model_dir(tmp_path / "m", cfg, seed=40 + i)
    ids = [helpers.token_ids(cfg["vocab_size"], n, 700 + 3 * i + j) for j, n in enumerate((91 + i, 37, 5))]
    ref = [plain.forward_dir(d, x).numpy() for x in ids]
    # 10 pages of 16: the third request gets pages that the second has given back
    runner = Runner(load_model(d, dtype=dtype), page_size=16, num_pages=10, max_requests=3)
    caches = [runner.manager.open(name) for name in "ab"]
    got = {0: [], 1: [], 2: []}
    fed = [0, 0, 0]
    # (request, tokens) of each step: a long portion beside a short one, single tokens beside a
    # portion, portions that end inside a page, the second request ends and the third starts
    plan = [[(0, 66), (1, 2)], [(0, 1), (1, 33)], [(0, 1), (1, 1)], [(0, 2), (1, 1)], "close b", [(0, 19 + i), (2, 3)],
            [(0, 1), (2, 1)], [(2, 1), (0, 1)]]
    for step in plan:
        if step == "close b":
            assert fed[1] == len(ids[1])
            runner.manager.close(caches[1])
            caches.append(runner.manager.open("c"))
            continue
        entries = [StepEntry(caches[r], ids[r][fed[r]:fed[r] + n], list(range(n))) for r, n in step]
        out = runner.step(entries).float().cpu()
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n])
            at += n
            fed[r] += n
    assert fed == [len(x) for x in ids]
    for r in range(3):
        helpers.assert_close_to_plain(torch.cat(got[r]).numpy(), ref[r], dtype, f"head_dim {head_dim} {dtype} request {r}")


def test_a_head_size_beyond_the_kernels_is_refused_when_the_model_is_built(tmp_path):
    from from_scratch_inference_engine_amd import load_model

    cfg = dict(config_of(0, 272), num_attention_heads=1, num_key_value_heads=1, hidden_size=32)
    d = helpers.make_model_dir(tmp_path / "m", cfg, seed=1)
    with pytest.raises(ValueError, match="head_dim 272 is larger than the kernels take"):
        load_model(d, dtype="bfloat16")

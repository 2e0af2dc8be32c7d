"""Random valid configurations (sizes, groups, windows, caps, scales drawn by a seeded generator), the engine in
float32 and bfloat16 against the plain implementation: unequal prompts in one step, then six tokens each.  Head sizes
are those whose attention library the build compiles, so nothing is compiled inside the test."""
import random

import pytest
import torch

from trapetum_amd.config import Gemma2Config
from trapetum_amd.weights import write_model_folder

from .plain import gemma2_plain as plain
from .tiny import random_tokens, rel_l2

pytestmark = pytest.mark.gpu
HEAD_SIZES = [16, 32, 48, 64, 80, 128, 256]


def draw(rng):
    hd = rng.choice(HEAD_SIZES)
    kv = rng.choice([1, 2, 3, 4])
    return dict(num_hidden_layers=rng.randint(1, 4), hidden_size=8 * rng.randint(4, 40) + rng.choice([0, 0, 4]),
                num_attention_heads=kv * rng.choice([1, 2, 3, 4, 8]), num_key_value_heads=kv, head_dim=hd,
                intermediate_size=rng.choice([16 * rng.randint(2, 30), rng.randint(20, 500)]), vocab_size=rng.randint(50, 3000),
                rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-3]), rope_theta=rng.choice([10000.0, 100.0, 1e6]),
                sliding_window=rng.choice([1, 3, 7, 16, 33, 64, 100, 4096]), query_pre_attn_scalar=rng.choice([hd, hd * 1.5, 24, 144]),
                attn_logit_softcapping=rng.choice([None, 50.0, 5.0]), final_logit_softcapping=rng.choice([None, 30.0, 8.0]),
                hidden_activation="gelu_pytorch_tanh", eos_token_id=1)


@pytest.mark.parametrize("case", range(8))
def test_random_configuration(case, tmp_path):
    from .gpu_engine import load_gpu_model
    rng = random.Random(1000 + case)
    kw = draw(rng)
    folder = str(tmp_path)
    write_model_folder(Gemma2Config.from_kwargs(**kw), folder, seed=case, sigma=rng.choice([0.02, 0.08]), sigma_norm=0.2)
    pcfg, pw = plain.read_folder(folder)
    lens = [rng.randint(1, 150) for _ in range(rng.randint(1, 4))]
    seqs = [random_tokens(n + 6, kw["vocab_size"], 100 * case + i) for i, n in enumerate(lens)]
    refs = [plain.forward(pcfg, pw, s) for s in seqs]
    for dtype, tol in (("float32", 1e-5), ("bfloat16", 2e-2)):
        model, _ = load_gpu_model(folder, dtype)
        cache = model.new_cache(max_tokens=2048)
        slots = [cache.acquire() for _ in lens]
        got = [[r] for r in model.step(cache, slots, [t for s, n in zip(seqs, lens) for t in s[:n]], counts=lens)]
        for step in range(6):
            out = model.step(cache, slots, [s[n + step] for s, n in zip(seqs, lens)])
            for i in range(len(lens)):
                got[i].append(out[i])
        for i, n in enumerate(lens):
            assert rel_l2(torch.stack(got[i]), refs[i][n - 1:n + 6]) < tol, (kw, lens, dtype, i)

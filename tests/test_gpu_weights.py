"""Random weights made on the GPU against the same made on the host: the generator is specified to the
bit, so a seed is one model wherever its tensors are made."""
import pytest
import torch

import util

pytestmark = pytest.mark.gpu


def test_deviates_made_on_the_gpu_equal_the_hosts(gpu):
    from tuff_amd.weights import random_init
    key = random_init.tensor_key(2, "model.embed_tokens.weight")
    for start, n in ((0, 300001), (2 ** 33 + 5, 4097)):
        host = random_init.normal_deviates(key, start, n, "cpu")
        dev = random_init.normal_deviates(key, start, n, gpu).cpu()
        assert torch.equal(host.view(torch.int64), dev.view(torch.int64)), (start, n)


@pytest.mark.parametrize("name", ["A", "B"])
def test_a_model_made_on_the_gpu_equals_the_folder_written_on_the_host(gpu, name, tmp_path):
    from tuff_amd.models import registry
    from tuff_amd.weights import loader, random_init
    raw, seed = util.CONFIGS[name]
    cfg = registry.config_from_dict(raw)
    decls = registry.build_model(cfg).weight_decls()
    folder = random_init.write_random_model(cfg, str(tmp_path / "host"), seed, device="cpu")
    read = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    made = random_init.random_weights(decls, seed, torch.bfloat16, gpu)
    for k in read:
        assert made[k].dtype == read[k].dtype and torch.equal(made[k].cpu(), read[k]), k
    # and a folder whose values were computed on the GPU holds the same bytes
    folder2 = random_init.write_random_model(cfg, str(tmp_path / "gpu"), seed, device=gpu)
    with open(folder + "/model.safetensors", "rb") as a, open(folder2 + "/model.safetensors", "rb") as b:
        assert a.read() == b.read()


def test_the_engine_from_a_configuration_is_the_engine_from_the_folder(gpu):
    """Engine.from_config (what `tuff --random` and the benchmark use) and Engine.from_folder on the folder that
    write_random_model wrote with the same seed: the same logits, bit for bit."""
    from tuff_amd.engine.batch import StepEntry
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models import registry
    raw, seed = util.CONFIGS["B"]
    toks = util.rand_tokens(40, raw["vocab_size"], 3)
    outs = []
    for eng in (Engine.from_folder(util.model_folder("B"), dtype="float32", max_tokens=256),
                Engine.from_config(registry.config_from_dict(raw), seed, dtype="float32", max_tokens=256)):
        eng.begin("r")
        outs.append(eng.step([StepEntry("r", toks, list(range(len(toks))))]).clone())
        eng.end("r")
    assert torch.equal(outs[0], outs[1])

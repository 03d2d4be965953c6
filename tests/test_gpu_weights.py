"""Random weights on the GPU: a model filled on the device from (configuration, seed) holds the numbers of
the folder that the host writes from the same configuration and seed."""
import pytest
import torch

import tiny_models as TM

pytestmark = pytest.mark.gpu


def _tensors_of(model):
    out = {}
    for i, (prefix, part) in enumerate(model._parts):
        for attr, value in vars(part).items():
            if isinstance(value, torch.Tensor):
                out[f"{i}:{prefix}{attr}"] = value
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_one_seed_one_model_on_the_device_and_in_a_folder(tmp_path, name, dtype):
    from infernum_amd import CacheConfig, Engine
    from infernum_amd.weights import write_random_model
    cfg = TM.tiny_config(name)
    tdt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    d = write_random_model(cfg, str(tmp_path / "m"), 9, dtype=tdt, **TM.SPEC_KW[name])
    cc = CacheConfig(page_size=16, num_pages=8, num_state_slots=2)
    a = Engine.from_config(cfg, seed=9, dtype=dtype, cache_config=cc, spec_kw=TM.SPEC_KW[name])
    b = Engine.from_pretrained(d, dtype=dtype, cache_config=cc)
    ta, tb = _tensors_of(a.model), _tensors_of(b.model)
    assert ta.keys() == tb.keys() and len(ta) >= 4 * cfg.num_hidden_layers + 2
    for k in ta:
        assert ta[k].dtype == tb[k].dtype and torch.equal(ta[k], tb[k]), k
    other = Engine.from_config(cfg, seed=10, dtype=dtype, cache_config=cc, spec_kw=TM.SPEC_KW[name])
    assert not torch.equal(_tensors_of(other.model)["0:model.embed_tokens.table"], ta["0:model.embed_tokens.table"])
    # and so the same logits
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    la = a.step([("r", toks, [7])])
    lb = b.step([("r", toks, [7])])
    assert torch.equal(la, lb)


def test_a_large_tensor_made_in_pieces_on_the_device_is_the_hosts():
    from infernum_amd.parts.base import WeightSpec
    from infernum_amd.weights import random_init as R
    spec = WeightSpec((3, (1 << 24) // 3 + 11), ("normal", 0.02))        # crosses a piece's end
    g = R.draw(spec, 5, "big", torch.device("cuda:0"))
    c = R.draw(spec, 5, "big", torch.device("cpu"))
    assert torch.equal(g.cpu(), c)

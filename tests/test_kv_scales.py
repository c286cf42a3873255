"""The fp8 KV-cache scale loader on the reference's own scale files (tests/fp8_kv/*/kv_cache_scales.json, kept as
data under tests/golden/fp8_kv/) and on files it must refuse (weight_utils.py:296-333, schema.py:19-84)."""
import json
import os

import pytest

from glake_amd.worker.kv_scales import kv_cache_scales_loader, layer_scales

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_kv")
F7B = os.path.join(GOLDEN, "llama2-7b_kv_cache_scales.json")
F70B = os.path.join(GOLDEN, "llama2-70b_kv_cache_scales.json")


def test_reads_the_reference_files():
    s = dict(kv_cache_scales_loader(F7B, 0, 1, 32, "llama"))
    assert len(s) == 32 and s[0] == 0.0152239128947258 and s[31] == 0.0482352152466774
    s = layer_scales(F70B, 80, model_type="llama")
    assert len(s) == 80 and all(0.019 < x < 0.086 for x in s)
    assert dict(kv_cache_scales_loader(F7B, 0, 1, 32, None))[13] == 0.040771484375  # model type not checked


@pytest.mark.parametrize("kwargs", [
    dict(num_hidden_layers=31), dict(tp_size=2), dict(model_type="opt"), dict(filename="/nonexistent.json")])
def test_a_file_that_does_not_fit_gives_no_scales(kwargs):
    args = dict(filename=F7B, tp_rank=0, tp_size=1, num_hidden_layers=32, model_type="llama")
    args.update(kwargs)
    assert list(kv_cache_scales_loader(**args)) == []
    args.pop("tp_rank")
    assert layer_scales(**args) == [1.0] * args["num_hidden_layers"]


def test_wrong_dtype_and_broken_json(tmp_path):
    doc = json.load(open(F7B))
    doc["kv_cache"]["dtype"] = "float8_e5m2"
    p = tmp_path / "a.json"
    p.write_text(json.dumps(doc))
    assert list(kv_cache_scales_loader(str(p), 0, 1, 32, "llama")) == []
    p.write_text("{ not json")
    assert list(kv_cache_scales_loader(str(p), 0, 1, 32, "llama")) == []
    doc = json.load(open(F7B))
    del doc["kv_cache"]["scaling_factor"]["0"]["5"]
    doc["kv_cache"]["scaling_factor"]["0"]["40"] = 0.1
    p.write_text(json.dumps(doc))
    assert list(kv_cache_scales_loader(str(p), 0, 1, 32, "llama")) == []

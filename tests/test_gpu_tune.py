"""The tile-table tuner (python -m lightop_amd.tune) end to end on a small layer: it times every block
size through the public entry point and writes the per-device JSON in the layout the reference's
reader expects (vllm_compat/w8a8_get_cache_json.py:133-174: file name by form and shape, keys
"N1_N2_K" -> M -> config1 / config2, flattened by the reader to "M_N1_N2_K")."""
import json
import os

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("workload,prefix", [("tiny-e8", "MOE_BLOCKINT8[128,128]"), ("tiny-e8-w4a8", "MOE_W4A8INT8[1,128]")])
def test_tuner_writes_the_reference_layout(tmp_path, capsys, workload, prefix):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lightop_amd import tune, workloads as wl

    print(f"[case] tuner {workload}", flush=True)
    layer = wl.LAYERS[workload]
    assert tune.main(["--workload", workload, "--tokens", "4,96", "--steps", "2", "--out", str(tmp_path)]) == 0
    text = capsys.readouterr().out
    assert "largest loss of the compiled-in table" in text
    files = os.listdir(tmp_path)
    assert len(files) == 1
    name = files[0]
    assert name.startswith(f"{prefix}_E={layer.E}_N1={2 * layer.I}_N2={layer.H}_K={layer.I}_TOPK{layer.top_k}_gfx950_")
    data = json.load(open(tmp_path / name))
    # the reader's flattening (w8a8_get_cache_json.py:166-171)
    flat = {f"{m}_{shape}": cfg for shape, per_m in data.items() for m, cfg in per_m.items()}
    for m in (4, 96):
        cfg = flat[f"{m}_{2 * layer.I}_{layer.H}_{layer.I}"]
        for part in ("config1", "config2"):
            assert cfg[part]["BLOCK_SIZE_M"] in (16, 32, 64, 128, 160)  # whichever was fastest in this run
            assert {"BLOCK_SIZE_N", "BLOCK_SIZE_K", "GROUP_SIZE_M", "num_warps", "num_stages"} <= set(cfg[part])

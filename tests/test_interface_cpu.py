"""Error contract of the Python API on a machine without a GPU (intra_attn/interface.py:17-23,
41-42, 60-63 of the reference): the checks fire before anything is launched."""
import pytest
import torch

import intra_amd
import intra_attn
from intra_amd import interface


def _cpu(S=128, H=4, Hkv=4, dtype=torch.bfloat16, D=128):
    return (torch.zeros(1, S, H, D, dtype=dtype), torch.zeros(1, S, Hkv, D, dtype=dtype),
            torch.zeros(1, S, Hkv, D, dtype=dtype))


def test_names_and_constants():
    assert intra_attn.intra_llm_attn is intra_amd.intra_llm_attn
    assert intra_attn.intra_image_attn is intra_amd.intra_image_attn
    assert interface.LLM_PATTERNS == {"scatter": 0, "gather1": 1, "window": 4}
    assert interface.IMAGE_PATTERNS == {"scatter": 0, "gather0": 4}
    assert interface.TEXT_LEN == 512 and intra_amd.__version__


def test_signatures_match_reference():
    import inspect
    llm = inspect.signature(intra_amd.intra_llm_attn)
    # the reference's parameters, in its order and with its defaults, come first; what this
    # package adds follows them and defaults to the reference's behaviour
    assert list(llm.parameters)[:7] == ["q", "k", "v", "pattern", "group_num", "window", "softmax_scale"]
    assert [p.default for p in llm.parameters.values()][3:7] == ["scatter", 8, 576, None]
    assert {n: p.default for n, p in list(llm.parameters.items())[7:]} == {
        "return_lse": False, "block": 256, "offset": 0, "n_sink": 0, "softmax": None}
    img = inspect.signature(intra_amd.intra_image_attn)
    assert list(img.parameters)[:6] == ["q", "k", "v", "pattern", "width", "softmax_scale"]
    assert [p.default for p in img.parameters.values()][3:6] == ["scatter", 64, None]
    assert {n: p.default for n, p in list(img.parameters.items())[6:]} == {"return_lse": False, "softmax": None}


@pytest.mark.parametrize("make", [lambda: _cpu(), lambda: _cpu(dtype=torch.float16), lambda: _cpu(D=64)])
def test_rejects_non_cuda_bf16_128(make):
    q, k, v = make()
    with pytest.raises(ValueError, match="CUDA bfloat16 tensors with head_dim 128"):
        intra_amd.intra_llm_attn(q, k, v)
    with pytest.raises(ValueError, match="CUDA bfloat16 tensors with head_dim 128"):
        intra_amd.intra_image_attn(q, k, v)


def test_missing_library_fails_loudly_and_nothing_falls_back(tmp_path):
    """Without the native library the package still imports (as the reference's does), but every
    call raises ImportError: there is no CPU or PyTorch fallback path."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("import torch, intra_amd\n"
            "q = torch.zeros(1, 64, 4, 128, dtype=torch.bfloat16)\n"
            "for fn in (intra_amd.intra_llm_attn, intra_amd.intra_image_attn):\n"
            "    try:\n"
            "        fn(q, q, q)\n"
            "    except ImportError as e:\n"
            "        assert 'not built' in str(e)\n"
            "    else:\n"
            "        raise SystemExit('call succeeded without the library')\n"
            "print('ok')\n")
    env = dict(os.environ, INTRA_HIP_LIB=str(tmp_path / "nowhere.so"), PYTHONPATH=root)
    res = subprocess.run([sys.executable, "-c", code], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0 and res.stdout.strip().endswith("ok"), res.stdout


def test_product_never_imports_the_oracle():
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for pkg in ("intra_amd", "intra_attn"):
        for name in os.listdir(os.path.join(root, pkg)):
            if name.endswith(".py"):
                text = open(os.path.join(root, pkg, name)).read()
                assert "import oracle" not in text and "from oracle" not in text, f"{pkg}/{name}"


def test_llama_caller_helper_plans_layers_on_cpu():
    """The test helper's layer planning is host logic: schedule, blocks and stripe offsets per layer,
    and which kernel call a layer makes."""
    from llama_caller import LayerPlan, plan_layers
    plans = plan_layers(32, "SWWWWWWW", group_num=2, window=575, n_sink=64, blocks=(256,), stripe_offsets=2)
    scatter = [(i, p) for i, p in enumerate(plans) if p.kind == "scatter"]
    assert [i for i, _ in scatter] == [0, 8, 16, 24]
    assert [p.offset for _, p in scatter] == [0, 1, 0, 1] and all(p.block == 256 for _, p in scatter)
    assert sum(p.kind == "window" for p in plans) == 28 and all(p.n_sink == 64 for p in plans if p.kind != "dense")
    assert plans[0].kernel_call() == ("block_scatter", dict(group_num=2, block=256, offset=0, n_sink=64))
    assert plans[1].kernel_call() == ("window_sink", dict(window=575, n_sink=64))
    # without stripes every Scatter layer has offset 0; blocks cycle over the Scatter layers
    plans = plan_layers(32, "sdw", group_num=8, window=512, blocks=(64, 128))
    assert [p.kind for p in plans[:4]] == ["scatter", "dense", "window", "scatter"]
    s_plans = [p for p in plans if p.kind == "scatter"]
    assert [p.block for p in s_plans[:4]] == [64, 128, 64, 128] and all(p.offset == 0 for p in s_plans)
    assert LayerPlan("dense").kernel_call() is None
    assert LayerPlan("scatter", group_num=8).kernel_call() == ("scatter", dict(group_num=8))  # token-level Scatter
    with pytest.raises(ValueError):
        plan_layers(2, "S", group_num=2, window=0, blocks=(128,), stripe_offsets=2)
    with pytest.raises(ValueError):
        LayerPlan("scatter", group_num=2, block=100).kernel_call()


def test_extension_stand_in_has_the_reference_signatures():
    """intra_attn_cuda.fwd / fwd_llm take the 16 positional arguments of mha_fwd / mha_fwd_llm
    (csrc/flash_attn/flash_api.cpp:356-371, 557-574) under the names the pybind module exports
    (flash_api.cpp:1766-1770)."""
    import inspect

    import intra_attn_cuda
    llm = list(inspect.signature(intra_attn_cuda.fwd_llm).parameters)
    img = list(inspect.signature(intra_attn_cuda.fwd).parameters)
    assert len(llm) == len(img) == 16
    assert llm[:3] == img[:3] == ["q", "k", "v"]
    assert llm[-3:] == ["mask", "group_num", "window"] and img[-3:] == ["mask", "width", "length"]
    assert llm[5:7] == ["p_dropout", "softmax_scale"]
    cpu = torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        intra_attn_cuda.fwd_llm(cpu, cpu, cpu, None, None, 0.0, 0.1, True, -1, -1, 0.0, False, None, 0, 8, 576)

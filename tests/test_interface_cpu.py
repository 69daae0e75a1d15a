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


def test_llama_caller_module_configuration_on_cpu():
    """install_intra_llama / set_dense_debug are host logic: schedule, block and stripe offsets per layer."""
    import types

    from intra_amd.llama_attention import install_intra_llama, set_dense_debug
    model = types.SimpleNamespace(model=types.SimpleNamespace(
        layers=[types.SimpleNamespace(self_attn=types.SimpleNamespace()) for _ in range(32)]))
    counts = install_intra_llama(model, num_groups=2, window=575, n_sink=64, scatter_blocks=(256,),
                                 layer_pattern="SWWWWWWW", scatter_stripe=True, scatter_n_offsets=2)
    assert counts == (4, 28, 0)
    cfgs = [l.self_attn._intra for l in model.model.layers]
    assert [c["layer_idx"] for c in cfgs if c["kind"] == "S"] == [0, 8, 16, 24]
    assert [c["scatter_offset"] for c in cfgs if c["kind"] == "S"] == [0, 1, 0, 1]
    assert all(c["scatter_block"] == 256 for c in cfgs if c["kind"] == "S")
    assert all(c["window"] == 575 and c["n_sink"] == 64 for c in cfgs)
    set_dense_debug(model, True)
    assert all(c["dense_debug"] for c in cfgs)
    # without stripes every Scatter layer has offset 0; blocks cycle over the Scatter layers
    counts = install_intra_llama(model, num_groups=8, scatter_blocks=(64, 128), layer_pattern="sd?w")
    assert counts == (11, 10, 11)
    s_cfgs = [l.self_attn._intra for l in model.model.layers if l.self_attn._intra["kind"] == "S"]
    assert [c["scatter_block"] for c in s_cfgs[:4]] == [64, 128, 64, 128]
    assert all(c["scatter_offset"] == 0 for c in s_cfgs)
    with pytest.raises(ValueError):
        install_intra_llama(model, num_groups=2, scatter_blocks=(128,), layer_pattern="S", scatter_stripe=True)


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

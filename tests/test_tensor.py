"""The library's tensor type: element type, shape, layout and ownership (no GPU needed for most of it)."""
import pytest
import torch

import llm_infer_amd
from llm_infer_amd.tensor import Tensor
from llm_infer_amd.weights import SafetensorsFile, write_safetensors
from llm_infer_amd.weights.loader import place_tensor


def test_ownership_is_read_off_the_memory_or_said():
    t = Tensor.wrap(torch.arange(6, dtype=torch.float32).view(2, 3))
    assert (t.owner, t.layout, t.logical, t.keeps) == ("host", "rows", (2, 3), None)
    assert t.describe() == "float32[2, 3] rows, host" and t.nbytes_stored == 24
    e = Tensor.empty((4, 2), torch.int32, "cpu")
    assert e.owner == "host" and e.dtype == torch.int32 and tuple(e.shape) == (4, 2)
    with pytest.raises(ValueError, match="owner 'device'"):
        Tensor.wrap(torch.zeros(2), owner="device")                 # memory on the host is not device-owned
    with pytest.raises(ValueError, match="contiguous"):
        Tensor.wrap(torch.zeros(4, 4).t())
    with pytest.raises(ValueError, match="element type"):
        Tensor.wrap(torch.zeros(2, dtype=torch.complex64))
    with pytest.raises(ValueError, match="layout"):
        Tensor.wrap(torch.zeros(2), layout="columns")


def test_torch_operations_work_and_give_plain_tensors_back():
    t = Tensor.wrap(torch.ones(2, 3))
    s = t * 2 + 1
    assert type(s) is torch.Tensor and torch.equal(s, torch.full((2, 3), 3.0))
    assert type(t[0]) is torch.Tensor and type(t.double()) is torch.Tensor
    assert torch.equal(t, torch.ones(2, 3)) and type(t.plain()) is torch.Tensor
    t += 1                                                           # in place: the same memory, still a Tensor
    assert isinstance(t, Tensor) and t.owner == "host" and t[1, 2].item() == 2.0


def test_a_checkpoint_s_tensors_are_borrowed_views_of_its_mapping(tmp_path):
    path = str(tmp_path / "m.safetensors")
    w = torch.randn(5, 7).to(torch.bfloat16)
    write_safetensors(path, {"w": w, "n": torch.ones(7)})
    f = SafetensorsFile(path)
    t = f.tensor("w")
    assert isinstance(t, Tensor) and t.owner == "borrowed" and t.keeps is not None and t.dtype == torch.bfloat16
    assert torch.equal(t, w) and f.tensor("n").owner == "borrowed"
    first = t.prefix(2)                                              # shares the mapping, and keeps it alive
    assert first.owner == "borrowed" and first.keeps is not None and torch.equal(first, w[:2])
    # what the engine keeps is a copy of its own, in the kept dtype (here on the CPU, as no GPU is asked for)
    kept = place_tensor(t, "matrix", torch.float32, "cpu")
    assert isinstance(kept, Tensor) and kept.owner == "host" and kept.dtype == torch.float32
    assert torch.equal(kept, w.float()) and kept.data_ptr() != t.data_ptr()
    assert place_tensor(f.tensor("n"), "vector", torch.bfloat16, "cpu").dtype == torch.float32


def test_tiled_layout_is_checked():
    flat = torch.zeros(32 * 64, dtype=torch.float16)
    t = Tensor.wrap(flat, "tiled", (20, 64))                         # 20 rows are stored as 32
    assert t.layout == "tiled" and t.logical == (20, 64) and t.describe() == "float16[20, 64] tiled, host"
    assert t.prefix(16).logical == (16, 64) and t.prefix(16).numel() == 16 * 64
    with pytest.raises(ValueError, match="multiples of 16"):
        t.prefix(8)
    with pytest.raises(ValueError, match="no torch view"):
        t.plain()
    with pytest.raises(ValueError, match="does not hold"):
        Tensor.wrap(flat, "tiled", (40, 64))
    with pytest.raises(ValueError, match="flat 16-bit storage"):
        Tensor.wrap(torch.zeros(32 * 64), "tiled", (20, 64))         # float32 is never tiled
    with pytest.raises(ValueError, match="does not hold|flat 16-bit"):
        Tensor.wrap(flat, "tiled", (20, 48))                         # k must be a multiple of 32


@pytest.mark.gpu
def test_device_and_pinned_memory_and_what_the_engine_holds():
    from llm_infer_amd.kernels import ops
    from tiny_configs import TINY_B
    d = Tensor.zeros((3, 64), torch.float16, "cuda")
    p = Tensor.pinned((8,), torch.int32)
    assert d.owner == "device" and p.owner == "pinned" and p.is_pinned()
    w = (torch.randn(40, 64) * 0.1).to(torch.float16)
    kept = place_tensor(Tensor.wrap(w), "matrix", torch.float16, "cuda")
    tiled = ops.prepare_weight(kept)
    assert kept.owner == "device" and ops.is_tiled(tiled) and tiled.owner == "device" and tiled.logical == (40, 64)
    assert torch.equal(ops.untile(tiled).cpu(), w)
    x = (torch.randn(3, 64) * 0.5).to(torch.float16).cuda()
    assert torch.allclose(ops.linear(x, tiled, out_dtype=torch.float32).cpu(), x.float().cpu() @ w.float().t(), atol=1e-2)
    # an engine's weights, cache pools and staging buffers are all of this type
    eng = llm_infer_amd.random_model(llm_infer_amd.config_from_dict(TINY_B), seed=0, dtype="bfloat16", max_tokens=256)
    mixer = eng.model.layers[0].mixer
    assert ops.is_tiled(mixer.wqkv) and mixer.wqkv.owner == "device" and eng.model.final_norm.weight.owner == "device"
    assert all(g.storage.owner == "device" for g in eng.cache.groups) and eng.cache.lens_dev.owner == "device"
    eng.generate([[1, 2, 3]], max_new_tokens=3, temperature=0.0)
    assert all(b.owner == "pinned" for b in eng._graph_bufs["host"])

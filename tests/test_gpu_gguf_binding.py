"""A Gemma-3-shaped model written as a GGUF file image, read back by the library's reader and bound
to the device: the forward pass equals the one of the same weights bound directly, bit for bit.
Tensor and metadata names follow the reference (src/engine/gemma_model.cpp:36-116,
src/engine/model.cpp:330-390)."""
from dataclasses import replace

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from gguf_image import write_gguf


@pytest.mark.parametrize("kind", ["target", "drafter"])
def test_model_bound_from_a_gguf_image_runs_like_the_direct_binding(kind):
    import torch
    from guffin_amd import gguf, hip, model
    hip.init(0)
    base = model.GEMMA3_12B if kind == "target" else model.GEMMA3_270M
    shape = replace(base, layers=7, vocab=2048, ring_global=1024, ring_local=base.ring_local)
    host = model.HostModel(shape, seed=5, position=0)
    image = write_gguf(host)
    reader = gguf.Reader(image)
    assert reader.info.alignment == 64 and reader.metadata()["general.architecture"] == "gemma3"
    assert len(reader.tensors()) == 2 + 13 * shape.layers
    bound = model.DeviceModel.from_gguf(reader, ring_local=shape.ring_local, ring_global=shape.ring_global, role=kind)
    direct = model.DeviceModel.from_host(host)
    assert replace(bound.shape, eps=shape.eps) == shape and abs(bound.shape.eps - shape.eps) < 1e-12
    tokens = torch.tensor([17, 1999], dtype=torch.int32, device="cuda")
    got = bound.forward(tokens, 0)
    want = direct.forward(tokens, 0)
    torch.cuda.synchronize()
    assert int(got[4].item()) == 0 and int(want[4].item()) == 0
    for g, w in zip(got[:4], want[:4]):
        assert torch.equal(g.view(torch.uint8), w.view(torch.uint8))


def test_blocks_of_mixed_formats_bind_matrix_by_matrix(gfo):
    """A Q4_K_M file keeps attn_v and ffn_down in Q6_K in some blocks and in Q4_K in others; each matrix is
    bound in its own format (src/engine/gemma_model.cpp:140-148) and the pass agrees with the oracle on the
    same canonical weights."""
    import torch
    from guffin_amd import gguf, hip, model
    hip.init(0)
    Q4, Q6 = model.Q4_K, model.Q6_K
    per_layer = ((Q4, Q4, Q6, Q4, Q4, Q4, Q6), (Q4, Q4, Q4, Q4, Q4, Q4, Q4), (Q4, Q4, Q6, Q4, Q4, Q4, Q4),
                 (Q4, Q4, Q4, Q4, Q4, Q4, Q6), (Q4, Q4, Q4, Q4, Q6, Q4, Q6), (Q4, Q4, Q6, Q4, Q4, Q4, Q6))
    shape = replace(model.GEMMA3_12B, layers=6, vocab=2048, ring_global=1024, layer_dtypes=per_layer)
    host = model.HostModel(shape, seed=8, position=0)
    bound = model.DeviceModel.from_gguf(gguf.Reader(write_gguf(host)), ring_local=shape.ring_local,
                                        ring_global=shape.ring_global)
    assert bound.shape.layer_dtypes == per_layer
    assert [[bound.layers[l].dtype[i] for i in range(7)] for l in range(6)] == [list(r) for r in per_layer]
    assert bound.shape.body_weight_bytes() == sum(host.w[l][i].size for l in range(6) for i in range(7))
    tokens = torch.tensor([17, 1999], dtype=torch.int32, device="cuda")
    got = bound.forward(tokens, 0)
    torch.cuda.synchronize()
    assert int(got[4].item()) == 0
    want, wk, wv = gfo.forward(host, [17, 1999], 0, threads=8)
    hidden = got[0].cpu().numpy().astype(np.float64)
    scale = np.sqrt((want.astype(np.float64) ** 2).mean(-1, keepdims=True))
    assert np.max(np.abs(hidden - want) / scale) <= 1e-3
    direct = model.DeviceModel.from_host(host).forward(tokens, 0)
    torch.cuda.synchronize()
    assert torch.equal(got[0].view(torch.uint8), direct[0].view(torch.uint8))


def test_binding_refuses_files_that_do_not_fit_the_model():
    from guffin_amd import gguf, hip, model
    hip.init(0)
    shape = replace(model.GEMMA3_270M, layers=2, vocab=512, ring_global=512)
    host = model.HostModel(shape, seed=6, position=0)
    host.norm[1][0] = host.norm[1][0][:-1].copy()          # a norm of the wrong width
    with pytest.raises(ValueError):
        model.DeviceModel.from_gguf(gguf.Reader(write_gguf(host)), ring_global=512, role="drafter")


def test_a_file_bound_as_target_must_have_the_targets_geometry():
    """The caller says what the file is; a drafter-shaped file (4 query heads on 1 KV head, Q8_0) given as the
    target is refused by the geometry rule (src/engine/gemma_model.cpp:120-124), not bound under other rules."""
    from guffin_amd import gguf, hip, model
    hip.init(0)
    shape = replace(model.GEMMA3_270M, layers=2, vocab=512, ring_global=512)
    image = write_gguf(model.HostModel(shape, seed=6, position=0))
    with pytest.raises(gguf.BindError) as refusal:
        model.DeviceModel.from_gguf(gguf.Reader(image), ring_global=512, role="target")
    assert "Gemma 3 target requires 256-wide paired GQA heads" in str(refusal.value)
    model.DeviceModel.from_gguf(gguf.Reader(image), ring_global=512, role="drafter")

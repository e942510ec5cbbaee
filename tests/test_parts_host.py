"""What the parts do on the host, without a GPU."""
import gc

import torch

import llama_cu_amd  # noqa: F401
from llama_cu_amd.parts import BuildContext, PartSpec, make_part
from llama_cu_amd.parts import position


def test_the_layers_of_a_model_share_one_pair_of_rotation_tables():
    """The tables depend on theta, the rotated dims, the positions and the device alone: 32 layers at 131,072
    positions hold one pair of 33.5 MB each, not 32 (2.1 GB), and build it once; another theta has its own; the
    pair is gone with the last part that holds it."""
    build = BuildContext(torch.float32, torch.device("cpu"), 131072, 16)
    spec = PartSpec("rotary", {"head_dim": 128, "theta": 500000.0, "max_positions": 131072})
    parts = [make_part("position", spec) for _ in range(32)]
    for p in parts:
        p.load({}, build)
    cos, sin, rot_dim, pairing = parts[0].rotary_tables()
    assert cos.shape == (131072, 64) and rot_dim == 128 and pairing == 0
    assert all(p.rotary_tables()[0].data_ptr() == cos.data_ptr() and p.rotary_tables()[1].data_ptr() == sin.data_ptr() for p in parts)
    assert len(position._tables) == 1
    other = make_part("position", PartSpec("rotary", {"head_dim": 128, "theta": 10000.0, "max_positions": 64}))
    other.load({}, build)
    assert other.rotary_tables()[0].data_ptr() != cos.data_ptr() and len(position._tables) == 2
    # the values are those of the formula (llama.cu/src/model/mod.rs:200-209), whoever built the pair
    want_cos, want_sin = parts[5].host_tables()
    assert torch.equal(cos, torch.from_numpy(want_cos)) and torch.equal(sin, torch.from_numpy(want_sin))
    del parts, p, other, cos, sin
    gc.collect()
    assert len(position._tables) == 0


def test_the_rows_of_zeros_for_the_library_can_be_fixed_instead_of_timed(monkeypatch):
    """``Tuning.library_rows``: 0 never fills the halves of a gate/up matrix up, n fills them up to a multiple of n;
    neither times anything (the default, -1, times the library on the GPU once per shape)."""
    import dataclasses
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts import linear
    monkeypatch.setattr(ops, "TUNING", dataclasses.replace(ops.TUNING, library_rows=0))
    assert linear.library_friendly_rows(11008, 4096, "cpu") == 11008
    monkeypatch.setattr(ops, "TUNING", dataclasses.replace(ops.TUNING, library_rows=2048))
    assert linear.library_friendly_rows(11008, 4096, "cpu") == 12288
    assert linear.library_friendly_rows(14336, 4096, "cpu") == 14336
    assert linear.library_friendly_rows(176, 64, "cpu") == 176            # small matrices stay as they are

"""The step's scratch buffers: named, reused, and kept apart by width."""

import pytest
import torch

from mini_gpt_inference_amd.parts.base import Workspace, WorkspaceFrozen


def test_buffers_are_reused_and_grow_by_rows_only():
    ws = Workspace(torch.device("cpu"))
    a = ws.get("qkv", 4, 160, torch.float32)
    assert ws.get("qkv", 3, 160, torch.float32) is a and ws.generation == 1
    b = ws.get("qkv", 9, 160, torch.float32)
    assert b.shape == (9, 160) and ws.generation == 2
    assert ws.get("qkv", 4, 160, torch.float32) is b


def test_layers_of_different_widths_do_not_take_each_others_buffer():
    """Two layers that ask for the same name at different widths each keep a buffer: otherwise every
    layer of a mixed model would allocate anew at every step, and no step of it could be captured."""
    ws = Workspace(torch.device("cpu"))
    narrow = ws.get("qkv", 4, 160, torch.float32)
    wide = ws.get("qkv", 4, 288, torch.float32)
    other = ws.get("qkv", 4, 288, torch.bfloat16)
    gen = ws.generation
    assert ws.get("qkv", 4, 160, torch.float32) is narrow
    assert ws.get("qkv", 4, 288, torch.float32) is wide
    assert ws.get("qkv", 4, 288, torch.bfloat16) is other
    assert ws.generation == gen
    ws.frozen = True
    assert ws.get("qkv", 2, 288, torch.float32) is wide
    with pytest.raises(WorkspaceFrozen, match="would have to grow"):
        ws.get("qkv", 5, 288, torch.float32)
    with pytest.raises(WorkspaceFrozen):
        ws.get("attn_out", 1, 96, torch.float32)

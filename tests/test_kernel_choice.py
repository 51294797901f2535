"""Which kernel family a call takes is decided on the host from the plan's sizes and the dtype (graphop._tiles,
_tiles_backward, _tile_seg_len) and where a plan is built from its size and the caller's preference
(plan._build_on_device, PlanCache.get(prefer_device=...)).  CPU only: the rules are plain functions of sizes."""
from types import SimpleNamespace

import torch

from bpt_amd import graphop, plan


def fake_plan(n_rows, n_edges):
    return SimpleNamespace(n_rows=n_rows, n_edges=n_edges, n_items=n_rows)


def test_tiles_need_64_columns_and_at_most_16_heads():
    cfg = graphop._SETTINGS
    for dtype in (torch.float32, torch.bfloat16):
        q = torch.empty(4, 8, 64, dtype=dtype)
        assert graphop._tiles(q, 8, 64, fake_plan(10, 100), 0.0, None, cfg)
        assert graphop._tiles(q, 16, 64, fake_plan(10, 100), 0.1, object(), cfg)        # dropout and score term included
        assert not graphop._tiles(q, 8, 32, fake_plan(10, 100), 0.0, None, cfg)
        assert not graphop._tiles(q, 32, 64, fake_plan(10, 100), 0.0, None, cfg)
    assert not graphop._tiles(torch.empty(4, 8, 64, dtype=torch.float64), 8, 64, fake_plan(10, 100), 0.0, None, cfg)
    old = graphop.set_group_rows(8)                                                       # a caller fixing the rows per group
    try:
        assert not graphop._tiles(torch.empty(4, 8, 64), 8, 64, fake_plan(10, 100), 0.0, None, graphop._SETTINGS)
    finally:
        graphop.set_group_rows(old)
    old = graphop.set_tiles(False)
    try:
        assert not graphop._tiles(torch.empty(4, 8, 64), 8, 64, fake_plan(10, 100), 0.0, None, graphop._SETTINGS)
    finally:
        graphop.set_tiles(old)


def test_backward_rule():
    f32, bf16 = torch.float32, torch.bfloat16
    term = torch.empty(1)                                                  # (any tensor: a score term is given)
    for plan in (fake_plan(8191, 98305), fake_plan(65535, 3293955), fake_plan(16383, 430237), fake_plan(33598, 573520)):
        for dtype in (f32, bf16):                                          # wherever the forward runs on tiles
            assert graphop._tiles_backward(plan, dtype) and graphop._tiles_backward(plan, dtype, term)
    old = graphop.TILE_BACKWARD
    try:
        graphop.TILE_BACKWARD = False
        assert not graphop._tiles_backward(fake_plan(10, 10), bf16)
    finally:
        graphop.TILE_BACKWARD = old


def test_segment_length_of_the_tile_plans_follows_the_mean_degree():
    assert graphop._tile_seg_len(fake_plan(16383, 430237)) == 64           # 26 edges per row
    assert graphop._tile_seg_len(fake_plan(65535, 3293955)) == 128         # 50
    assert graphop._tile_seg_len(fake_plan(4097, 524224)) == 256           # 128


def test_where_a_plan_is_built():
    cpu_eid = torch.zeros(1 << 18, dtype=torch.int64)
    assert not plan._build_on_device(cpu_eid, 1 << 20)                     # host tensors: on the host, whatever the size
    fake = SimpleNamespace(is_cuda=True, numel=lambda: 430237)
    assert not plan._build_on_device(fake, 16383)                          # below 24576 rows, mean degree 26
    assert plan._build_on_device(fake, 24576)
    dense = SimpleNamespace(is_cuda=True, numel=lambda: 524224)
    assert plan._build_on_device(dense, 4097)                              # 2^17 edges and more at a mean degree of 32 and more
    assert not plan._build_on_device(dense, 1000)                          # but not the CSR of a few hundred edge types
    old = plan.set_device_build(True)
    try:
        assert plan._build_on_device(fake, 10)
        plan.set_device_build(False)
        assert not plan._build_on_device(fake, 1 << 20)
    finally:
        plan.set_device_build(old)

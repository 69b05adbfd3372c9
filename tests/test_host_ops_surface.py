"""CPU-only: the torch.ops.glq schemas exist, their fakes agree with the schema arity and
give the shapes/dtypes the call sites rely on (reference tests/test_glq_vllm.py:94-140)."""
import inspect

import pytest
import torch

from glq_amd import custom_ops


@pytest.fixture(scope="module", autouse=True)
def _registered():
    custom_ops.register()
    custom_ops.register()            # idempotent


def _n_schema_args(schema):
    inside = schema[schema.index("(") + 1:schema.rindex(") ->")]
    return len([a for a in inside.split(",") if a.strip()])


def test_every_schema_has_fake_with_same_arity():
    for name, schema in custom_ops.SCHEMAS.items():
        assert hasattr(torch.ops.glq, name), name
        fake = custom_ops.FAKES[name]
        if fake is custom_ops._none_fake:
            continue
        assert len(inspect.signature(fake).parameters) == _n_schema_args(schema), name


def test_fakes_on_meta_tensors():
    m, n, B = 64, 128, 3
    mt = lambda *s, dt=torch.float16: torch.empty(*s, dtype=dt, device="meta")  # noqa: E731
    x = mt(B, n)
    i64 = torch.empty(1, dtype=torch.int64, device="meta")
    i32 = torch.empty(1, 4, dtype=torch.int32, device="meta")
    packed = mt(32, 64, dt=torch.int16)
    y = torch.ops.glq.fused_linear_trellis_3inst(x, mt(n), mt(m), packed, i64, i64, i32, i32, 0.02,
                                                 n, m, n, m)
    assert y.shape == (B, m) and y.dtype == torch.float16 and y.device.type == "meta"
    y = torch.ops.glq.fused_linear_trellis_3inst_rvq2(mt(B, n, dt=torch.bfloat16), mt(n), mt(m), packed,
                                                      packed, i64, i64, i32, i32, 0.02, 0.3, n, m, n, m)
    assert y.shape == (B, m) and y.dtype == torch.bfloat16
    q = mt(m, n // 8, dt=torch.int16)
    cb = mt(65536, 8)
    e = mt(0, dt=torch.int16)
    ef = mt(0)
    y = torch.ops.glq.fused_linear_block_diag(x, mt(n), mt(m), q, cb, 0.02, n, m, n, m, i64, i64, i32,
                                              i32, e, ef, 0.0, e, ef, 0.0, e, ef, 0.0)
    assert y.shape == (B, m) and y.dtype == torch.float16
    y = torch.ops.glq.dequant_matmul(x, q, cb, 0.02, e, ef, 0.0, ef, e, ef, 0.0, e, ef, 0.0)
    assert y.shape == (B, m) and y.dtype == torch.float32
    cbp = mt(65536, dt=torch.int32)
    y = torch.ops.glq.dequant_matmul_packed(x, q, cbp, 0.02)
    assert y.shape == (B, m) and y.dtype == torch.float32
    y = torch.ops.glq.dequant_matvec_packed(mt(n), q, cbp, 0.02)
    assert y.shape == (m,) and y.dtype == torch.float32
    assert torch.ops.glq.input_rht_triton(x, mt(n), mt(B, n, dt=torch.float32), n, n, 0.1, n, 7) is None
    assert torch.ops.glq.output_rht_triton(mt(B, m, dt=torch.float32), mt(m), mt(B, m), m, m, 6, 0.1) is None
    yr = mt(B, 2 * m, dt=torch.float32)
    assert torch.ops.glq.fused_linear_trellis_3inst_yrht(x, mt(n), packed, i64, i32, 0.02, n, n, m,
                                                         yr, m) is None


def test_module_buffers_match_the_checkpoint_contract():
    from glq_amd.quantized_linear import E8RHTLinear
    lin = E8RHTLinear(960, 960, block_diagonal=True)
    sd = lin.state_dict()
    assert sd["Qidxs"].shape == (960, 120) and sd["Qidxs"].dtype == torch.int16
    assert sd["SU"].dtype == torch.float16 and sd["Wscale"].shape == ()
    assert {"Qidxs2", "Qidxs3", "Qidxs4", "inv_resid_scale", "inv_resid_scale2",
            "inv_resid_scale3", "SV"} <= set(sd)
    assert lin.blocks_n == [512, 256, 128, 64]
    legacy = E8RHTLinear(100, 48)
    assert (legacy.m_pad, legacy.n_pad) == (64, 128) and not legacy.block_diagonal
    tr = E8RHTLinear(2048, 11008, codebook_type="trellis")
    assert tr.block_diagonal and tr.blocks_m == [8192, 2048, 512, 256]
    assert tr.trellis_packed.numel() == 0 and tr.tlut.numel() == 0
    # a single-stage trellis checkpoint loads without the optional keys
    tr2 = E8RHTLinear(128, 64, codebook_type="trellis")
    tr2.load_state_dict({"trellis_packed": torch.zeros(32, 64, dtype=torch.int16),
                         "SU": torch.ones(64, dtype=torch.float16),
                         "SV": torch.ones(128, dtype=torch.float16),
                         "Wscale": torch.tensor(0.5)})
    assert tr2.trellis_packed.shape == (32, 64) and tr2.trellis_packed2.numel() == 0
    # a block-diagonal shell checkpoint re-shapes a module built with the legacy default
    adapt = E8RHTLinear(160, 96)
    adapt.load_state_dict({"Qidxs": torch.zeros(96, 20, dtype=torch.int16),
                           "SU": torch.ones(96, dtype=torch.float16),
                           "SV": torch.ones(160, dtype=torch.float16), "Wscale": torch.tensor(1.0)})
    assert adapt.block_diagonal and adapt.blocks_n == [128, 32] and adapt.blocks_m == [64, 32]
    with pytest.raises(RuntimeError, match="GPU only"):
        tr2(torch.zeros(1, 128))
    with pytest.raises(NotImplementedError):
        E8RHTLinear(64, 64, codebook_type="e8p")


def test_derived_cache_is_keyed_by_memory_not_by_object():
    """The cache behind the packed tables and the folded index streams (ext._DerivedCache): a fresh view
    of the same memory hits, an in-place write or another tensor misses, and an entry goes with the
    storage it was derived from.  (Plain CPU tensors: the cache itself touches no device.)"""
    import gc
    from glq_amd import ext
    c = ext._DerivedCache()
    base = torch.arange(64, dtype=torch.int16).reshape(8, 8)
    c.put(base, "folded")
    assert c.get(base) == "folded" and c.get(base.view(8, 8)) == "folded" and c.get(base[:]) == "folded"
    assert c.get(base.view(64)) is None                       # another shape: another layer
    assert c.get(base[2:]) is None and c.get(base.clone()) is None
    assert c.get(base, ("table-2",)) is None                  # the same indices against another table
    stacked = torch.zeros(2, 8, 8, dtype=torch.int16)
    c.put(stacked[1], "shard")
    assert c.get(stacked[1]) == "shard" and c.get(stacked.view(16, 8)[8:]) == "shard" and c.get(stacked[0]) is None
    base.add_(1)                                              # written in place: the derived data is stale
    assert c.get(base) is None
    c.put(base, "again")
    assert c.get(base) == "again" and len(c) == 2             # the older version of the same tensor is gone
    assert c.holds(base) and c.holds(stacked[1]) and not c.holds(stacked[0].clone())
    del base
    gc.collect()
    assert len(c) == 1                                        # dropped with its storage
    keep = stacked[1]
    del stacked
    gc.collect()
    assert c.get(keep) == "shard"                             # a view keeps the storage, and the entry, alive
    del keep
    gc.collect()
    assert len(c) == 0


def test_merged_trellis_linear_host_side():
    """Shard bookkeeping and refusals of the merged-linear holder that need no GPU."""
    from glq_amd.linear_method import GLQShards, MergedTrellisLinear, trellis_rvq_recipe
    assert [trellis_rvq_recipe(b) for b in range(2, 9)] == [[2], [3], [4], [4, 1], [4, 2], [4, 3], [4, 4]]
    layer = MergedTrellisLinear(2048, [2048, 512, 512], bpw=4)
    assert layer.glq_is_fused and layer.glq_num_shards == 3 and layer.glq_n_pad == 2048
    assert len(layer.SU) == 3 and layer.SU.get_shard(1).shape == (512,) and layer.SV.get_shard(2).shape == (2048,)
    assert layer.trellis_packed.get_shard(0).numel() == 0     # nothing loaded yet
    single = MergedTrellisLinear(512, [256])
    assert not single.glq_is_fused
    import pytest
    with pytest.raises(RuntimeError, match="process_weights_after_loading"):
        layer.apply(torch.zeros(1, 2048))
    with pytest.raises(RuntimeError, match="trellis layers"):
        MergedTrellisLinear.from_linears([])
    sh = GLQShards([torch.zeros(1), torch.ones(2)])
    assert len(sh) == 2 and sh.get_shard(1).numel() == 2


def test_merged_shell_linear_host_side():
    """Shard bookkeeping and refusals of the E8-shell merged-linear holder that need no GPU."""
    import pytest
    from glq_amd.linear_method import MergedShellLinear
    table = torch.zeros(65536, 8, dtype=torch.float16)
    layer = MergedShellLinear(960, [960, 320, 320], table)
    assert layer.glq_is_fused and layer.glq_num_shards == 3 and not layer.glq_is_trellis
    assert len(layer.Qidxs) == 3 and layer.Qidxs2.get_shard(1).numel() == 0 and layer.SU.get_shard(2).shape == (320,)
    assert float(layer.inv_resid_scale3.get_shard(0)) == 0.0
    assert not MergedShellLinear(512, [256], table).glq_is_fused
    with pytest.raises(RuntimeError, match="process_weights_after_loading"):
        layer.apply(torch.zeros(1, 960))
    with pytest.raises(RuntimeError, match="E8-shell layers"):
        MergedShellLinear.from_linears([])

"""The GEMM tile descriptor (the GPU counterpart of the reference's MatmulConfig,
include/gc/Analysis/MatmulConfigAnalysis.h:25-34) and the per-op attribute override
(lib/gc/Analysis/MatmulConfigAnalysis.cpp:368-422: all nine attributes or none; an invalid config is dropped).
Host-side: no GPU needed."""
import re

import pytest


def _cfg(MThreads=1, NThreads=1, KThreads=1, MBlock=256, NBlock=256, KBlock=64, iM=128, iN=128, iK=32):
    return [MThreads, NThreads, KThreads, MBlock, NBlock, KBlock, iM, iN, iK]


def test_defaults_per_shape(gc):
    c, note = gc.tile_config(4096, 4096, 4096)
    assert (c.kernel, c.bm, c.bn, c.waves_m * c.waves_n, c.wave_m, c.wave_n, c.split_k) == (2, 256, 256, 4, 128, 128, 1)
    assert (c.mfma_m, c.mfma_n, c.mfma_k, c.kbytes, c.stages, c.workgroups, c.from_attrs) == (16, 16, 32, 64, 4, 256, 0)
    assert note == ""
    c, _ = gc.tile_config(4096, 11008, 4096, a_dtype=gc.U8)             # config 3: 688 tiles
    assert (c.kernel, c.mfma_k, c.workgroups) == (2, 64, 688)
    for odt in (gc.S32, gc.F32):                                        # raw accumulators / f32: the same 4-wave kernel
        c, _ = gc.tile_config(4096, 11008, 4096, a_dtype=gc.U8, out_dtype=odt)
        assert (c.kernel, c.waves_m * c.waves_n, c.wave_n, c.mfma_k, c.workgroups) == (2, 4, 128, 64, 688)
    c, _ = gc.tile_config(4096, 11008, 4096, a_dtype=gc.U8, out_dtype=gc.S32,   # 8 waves of 128 x 64 by name
                          matmul_config=_cfg(iN=64))
    assert (c.kernel, c.waves_m * c.waves_n, c.wave_n, c.from_attrs) == (1, 8, 64, 1)
    c, _ = gc.tile_config(300, 200, 100)                                # ragged: bounds-checked tile
    assert c.kernel == 0
    c, _ = gc.tile_config(32, 4096, 4096)                               # a short A: the weights are streamed, K slices fill the GPU
    assert c.kernel == 4 and (c.bm, c.bn) == (32, 64) and c.split_k == 4 and c.workgroups == 64 * 4
    c, _ = gc.tile_config(16, 11008, 4096)                              # 172 panels: no slices, one launch
    assert c.kernel == 4 and (c.bm, c.bn) == (32, 64) and c.split_k == 1 and c.workgroups == 172
    c, _ = gc.tile_config(32, 4096, 4096, matmul_config=_cfg(KThreads=8))   # the 256 x 256 tile by name: K slices of it
    assert c.kernel == 3 and (c.bm, c.bn) == (256, 256) and c.split_k == 8 and c.workgroups == 16 * 8
    c, _ = gc.tile_config(2048, 2048, 2048)                             # 64 large tiles: small tiles instead
    assert (c.kernel, c.bm, c.wave_m, c.wave_n, c.split_k, c.workgroups) == (5, 128, 64, 64, 1, 256)
    c, _ = gc.tile_config(1024, 1024, 8192)                             # and a deep K: slices of small tiles
    assert (c.kernel, c.bm, c.split_k, c.workgroups) == (3, 128, 4, 256)
    c, _ = gc.tile_config(128, 4096, 11008)                             # up to 128 rows the weights are streamed
    assert (c.kernel, c.bm, c.bn, c.split_k, c.workgroups) == (4, 128, 64, 4, 256)
    c, _ = gc.tile_config(192, 4096, 11008)                             # past that: slices of small tiles, of unequal length (86 ring groups)
    assert (c.kernel, c.bm, c.split_k) == (3, 128, 4)
    c, _ = gc.tile_config(2048, 11008, 4096)                            # 344 large tiles: more than a round, they stay
    assert (c.kernel, c.bm, c.split_k, c.workgroups) == (2, 256, 1, 344)
    c, _ = gc.tile_config(1024, 4096, 4096, a_dtype=gc.U8)              # 8-bit, 64 large tiles: small tiles, never K slices
    assert (c.kernel, c.bm, c.mfma_k, c.split_k, c.workgroups) == (5, 128, 64, 1, 256)
    c, _ = gc.tile_config(1024, 1024, 8192, a_dtype=gc.U8)
    assert (c.kernel, c.bm, c.split_k) == (5, 128, 1)
    c, _ = gc.tile_config(4096, 5120, 4096)                             # 320 large tiles: a round, and 64 tiles as 256 small ones
    assert (c.kernel, c.bm, c.workgroups) == (2, 256, 256 + 4 * 64)
    c, _ = gc.tile_config(4096, 11008, 4096)                            # 176 tiles in the last round: too many for that
    assert (c.kernel, c.workgroups) == (2, 688)
    c, _ = gc.tile_config(64, 4096, 4096, trans_b=True)                 # [N,K] weights, 64 rows: streamed, A tile of 64 rows
    assert (c.kernel, c.bm, c.bn, c.split_k) == (4, 64, 64, 4)
    c, _ = gc.tile_config(128, 4096, 4096, trans_b=True)                # up to 128 rows likewise
    assert (c.kernel, c.bm, c.bn, c.split_k) == (4, 128, 64, 4)
    c, _ = gc.tile_config(129, 4096, 4096, trans_b=True)                # one row more: slices of small tiles
    assert (c.kernel, c.bm, c.split_k) == (3, 128, 4)
    c, _ = gc.tile_config(32, 4096, 4096, trans_b=True)                 # [N,K] weights, short A: streamed
    assert c.kernel == 4 and c.split_k >= 4


def test_attributes_name_the_small_tile(gc):
    c, note = gc.tile_config(4096, 4096, 4096, matmul_config=_cfg(MBlock=128, NBlock=128, iM=64, iN=64))
    assert (c.kernel, c.bm, c.bn, c.workgroups, c.from_attrs, note) == (5, 128, 128, 1024, 1, "")
    c, note = gc.tile_config(4096, 4096, 4096, matmul_config=_cfg(MBlock=128, NBlock=128, iM=64, iN=64, KThreads=2))
    assert c.from_attrs == 0 and c.kernel == 2 and "no K slices" in note
    c, note = gc.tile_config(2048, 2048, 2048, matmul_config=_cfg())   # the large tile by name: no small tiles, no slices
    assert (c.kernel, c.bm, c.split_k, c.from_attrs) == (2, 256, 1, 1)


def test_all_nine_attributes_steer_waves_and_k_slices(gc):
    c, note = gc.tile_config(4096, 4096, 4096, matmul_config=_cfg(iN=64))
    assert (c.kernel, c.waves_m * c.waves_n, c.wave_n, c.from_attrs, note) == (1, 8, 64, 1, "")
    c, note = gc.tile_config(4096, 4096, 4096, matmul_config=_cfg(iN=128))
    assert (c.kernel, c.from_attrs) == (2, 1)
    c, note = gc.tile_config(32, 4096, 4096, matmul_config=_cfg(KThreads=4))
    assert (c.kernel, c.split_k, c.workgroups, c.from_attrs) == (3, 4, 64, 1)
    c, note = gc.tile_config(32, 4096, 4096, matmul_config=_cfg(KThreads=1))   # no slices: whole-K tiles
    assert c.split_k == 1 and c.kernel in (0, 1, 2)


@pytest.mark.parametrize("bad,why", [(dict(MBlock=128), "workgroup tile"), (dict(iM=32, iN=32), "wave's tile"),
                                     (dict(KThreads=0), "not positive"), (dict(MBlock=256, iM=96), "multiple"),
                                     (dict(KThreads=128, KBlock=64), "fewer K blocks")])
def test_invalid_or_unbuilt_configs_are_ignored_with_a_reason(gc, bad, why):
    c, note = gc.tile_config(4096, 4096, 4096, matmul_config=_cfg(**bad))
    d, _ = gc.tile_config(4096, 4096, 4096)
    assert c.from_attrs == 0 and why in note and note.startswith("MatmulConfig attributes ignored")
    assert [getattr(c, f) for f, _ in c._fields_] == [getattr(d, f) for f, _ in d._fields_]


def _matmul_json(ga, M, K, N, attrs):
    op = {"kind": "MatMul", "inputs": [ga._t(0, "bf16", [M, K]), ga._t(1, "bf16", [K, N])], "outputs": [ga._t(2, "bf16", [M, N])]}
    if attrs:
        op["attrs"] = {k: {"type": "s64", "value": v} for k, v in attrs.items()}
    return ga._graph([op], [0, 1], [2])


def test_explain_prints_the_descriptor_and_the_override(ga, gc):
    st, plan = ga.explain(_matmul_json(ga, 4096, 4096, 4096, None))
    assert st == 0 and re.search(r"tile: whole tiles, 4 waves \(one per SIMD\), 256x256 per workgroup, 64 B of K per stage x 4 "
                                 r"stages, waves 2x2 of 128x128, mfma 16x16x32, split_k 1, 256 workgroups\n", plan), plan
    nine = dict(zip(gc.MATMUL_CONFIG_NAMES, _cfg(iN=64)))
    st, plan = ga.explain(_matmul_json(ga, 4096, 4096, 4096, nine))
    assert st == 0 and "8 waves" in plan and "[MatmulConfig attributes applied]" in plan, plan
    eight = dict(nine)
    del eight["KBlock"]                      # incomplete: the reference ignores it, so does this
    st, plan = ga.explain(_matmul_json(ga, 4096, 4096, 4096, eight))
    assert st == 0 and "4 waves" in plan and "MatmulConfig" not in plan, plan
    st, plan = ga.explain(_matmul_json(ga, 4096, 4096, 4096, dict(nine, MBlock=64, innermostMBlock=32)))
    assert st == 0 and "MatmulConfig attributes ignored" in plan and "4 waves" in plan, plan


def test_mlir_attribute_dictionary_is_read(ga):
    attrs = "{MThreads = 4 : i32, NThreads = 2 : i32,  KThreads = 1 : i32, MBlock = 256 : i32, NBlock = 256 : i32, " \
            "KBlock = 256 : i32,innermostMBlock = 128 : i32, innermostNBlock = 64 : i32,  innermostKBlock = 32 : i32 }"
    mod = """func.func @entry(%a: tensor<4096x4096xbf16>, %b: tensor<4096x4096xbf16>) -> tensor<4096x4096xbf16> {
  %c0 = arith.constant 0.0 : bf16
  %e = tensor.empty() : tensor<4096x4096xbf16>
  %z = linalg.fill ins(%c0 : bf16) outs(%e : tensor<4096x4096xbf16>) -> tensor<4096x4096xbf16>
  %r = linalg.matmul """ + attrs + """ ins(%a, %b : tensor<4096x4096xbf16>, tensor<4096x4096xbf16>) outs(%z : tensor<4096x4096xbf16>) -> tensor<4096x4096xbf16>
  return %r : tensor<4096x4096xbf16>
}"""
    st, plan = ga.explain_mlir(mod)
    assert st == 0 and "8 waves" in plan and "[MatmulConfig attributes applied]" in plan, plan
    st, plan = ga.explain_mlir(mod.replace(attrs, ""))
    assert st == 0 and "4 waves" in plan, plan

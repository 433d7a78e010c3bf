"""The benchmark workloads at their FULL shapes, as parity tests: the very launches bench.py times (same builders, same
planner, through the C-ABI), each checked on sampled sequences against the oracle.

  configs[0]  INT4 key-only pages (konly), B=1, L=2048, uniform calibration: writer bytes and attention against the oracle
  configs[1]  INT4 key-only pages (konlya), B=32, 32q/8kv, L=8192: nsplit 1, chunk 8192, 16-wavefront workgroups; with
              the split plan of this build's planner and with the one the reference's cost model makes
  configs[2]  INT2 key-only pages (konlya2) + static key centring + 4 sink / 128 window BF16 rows, B=64, L=16384
  configs[3]  KIVI-style pages, B=16, 64q/8kv, L=32768, 128-token BF16 residual; FP16 and FP8 meta
  configs[4]  multi-query prefill, 4 requests x 512 new tokens over 16384 cached, 64q/8kv; static and key-only pages

Bars (the worst element-wise ratio |err| / (2e-3 + 1e-2 |ref|) is printed for every case):
  FlagRot decode   element-wise: |out - ref| <= 2e-3 + 1e-2 |ref| on every element of the sampled sequences;
  KIVI decode      element-wise as well (the score operands carry value + remainder, 22 bits; with single fp16
                   products the rounding of q' * scale * code and q' * min moved the weight of whole 32-token groups
                   by up to ~1 % and the worst ratio was 6.7); the reference's own bar is max |err| <= 1e-2 max |ref|
                   (integrations/vllm_flagrot/tests/test_kivi.py:243);
  MQ prefill       relative L2 <= 3e-3, the error of BF16 FlashAttention, which is what the reference measures its
                   kernel against (scripts/bench_mq_prefill.py:221-235); the bf16 rounding of the output alone is 1.1e-3.
"""
import sys
import types
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
import bench  # noqa: E402

pytestmark = pytest.mark.gpu


def _args(**kw):
    return types.SimpleNamespace(**{"nsplit": 0, "f8": False, "mq_fmt": "konlya", **kw})


def _report(name, r):
    print(f"\n{name}: {r['check']}  [{r['bar']}]", flush=True)


def test_configs0_b1_l2048_konly_uniform_calibration(dev):
    """configs[0] -- the reference's own CPU-runnable case (one decode step of the Llama-3.1-8B layer shape, batch 1,
    context 2048, INT4 key-only pages, C_q = I, c_o = 1; kernels/codebook_ref.py:191-236 for the writer,
    integrations/vllm_flagrot/tests/test_kernels.py:37-56 for the attention) through the HIP writer and decode: the pool
    must be byte-equal to the oracle's packed pool and the attention inside the element-wise bar"""
    from flagrot_releaser_amd import kernels as K
    r = bench.configs0(torch, K, dev, timed_legs=False)
    print("\n" + r["check"], flush=True)
    assert r["pool_bytes_equal"], r["check"]
    assert r["checked"] and r["errors"]["elementwise"] <= 1.0, r["check"]


def test_int2_at_the_headline_shape_b32_l8192(dev):
    """the metric names INT4 and INT2 at batch 32 x 8K: the INT2 key-only pages at configs[1]'s shape"""
    r = bench.run_flagrot(_args(), torch, dev, "int2_b32", 3, 2)["own"]
    _report("INT2 konlya2, B=32 L=8192", r)
    assert r["checked"] and r["errors"]["elementwise"] <= 1.0, r["check"]


def test_configs1_int4_b32_l8192_both_planners(dev):
    rr = bench.run_flagrot(_args(), torch, dev, "int4", 3, 2, plans=("own", "reference"))
    for plan, r in rr.items():
        _report(f"configs[1] ({plan} plan: nsplit {r['nsplit']}, chunk {r['chunk']})", r)
        assert r["checked"] and r["errors"]["elementwise"] <= 1.0, r["check"]
    assert (rr["own"]["nsplit"], rr["own"]["chunk"]) == (1, 8192)


def test_configs1_forced_splits(dev):
    """the same cache through the split-K path (4 splits of 2048 tokens: small workgroups that share page ranges)"""
    r = bench.run_flagrot(_args(nsplit=4), torch, dev, "int4", 3, 2)["own"]
    _report("configs[1] with nsplit 4", r)
    assert r["nsplit"] == 4 and r["checked"], r["check"]


def test_configs2_int2_centred_sink_window_b64_l16384(dev):
    r = bench.run_flagrot(_args(), torch, dev, "int2", 3, 2)["own"]
    _report("configs[2]", r)
    assert r["checked"] and r["sink"] == 4 and r["window"] == 128, r["check"]


@pytest.mark.parametrize("f8", [False, True], ids=["f16meta", "f8meta"])
def test_configs3_kivi_b16_l32768(dev, f8):
    r = bench.run_kivi(_args(f8=f8), torch, dev, 3, 2)
    _report("configs[3]" + (" FP8 meta" if f8 else ""), r)
    assert r["checked"] and r["errors"]["elementwise"] <= 1.0, r["check"]
    assert r["errors"]["max_over_max"] <= 1e-2 and r["errors"]["rel_l2"] <= 3e-3, r["check"]


@pytest.mark.parametrize("fmt", ["int4a", "konlya"])
def test_configs4_mq_prefill_4x512_over_16384(dev, fmt):
    r = bench.run_mq(_args(), torch, dev, 2, 1, fmt)
    _report(f"configs[4] {fmt}", r)
    assert r["checked"] and r["errors"]["rel_l2"] <= 3e-3, r["check"]
    assert r["rows_per_tile"] == 256


def test_head_dim_256_bench_shapes(dev):
    """the head dim 256 workloads of bench.py (--head-dim 256; GQA 24q/4kv, no configuration of the baseline): FlagRot
    INT4 decode, KIVI decode and the multi-query prefill at their record shapes, same bars as their 128-d workloads"""
    r = bench.run_flagrot(_args(head_dim=256), torch, dev, "int4", 3, 2)["own"]
    _report("INT4 decode, head dim 256", r)
    assert r["checked"] and r["errors"]["elementwise"] <= 1.0, r["check"]
    r = bench.run_kivi(_args(head_dim=256), torch, dev, 3, 2)
    _report("KIVI decode, head dim 256", r)
    assert r["checked"] and r["errors"]["elementwise"] <= 1.0, r["check"]
    r = bench.run_mq(_args(head_dim=256), torch, dev, 2, 1, "konlya")
    _report("MQ prefill, head dim 256", r)
    assert r["checked"] and r["errors"]["rel_l2"] <= 3e-3 and r["rows_per_tile"] == 128, r["check"]

"""Tuning entry points on the device: the exhaustive tracea_tune_* of the
reference's FFI (src/interface/ffi.rs), and the cache-first AutoTuner adapters.
The winner must be a compiled variant, be recorded under the reference's cache
key, and be the variant the operator then runs."""
import json

import numpy as np
import pytest

import oracle
from helpers import round_f16, tol_half, assert_close_scaled

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture
def cache_file(tmp_path, monkeypatch):
    from tracea_amd import tuner as T
    path = tmp_path / "tuning_cache_v2.json"
    monkeypatch.setenv("TRACEA_TUNING_CACHE", str(path))
    monkeypatch.setenv("TRACEA_TUNING_HISTORY", str(tmp_path / "tuning_history.json"))
    T.cache_reload()
    T.history_reload()
    yield path
    monkeypatch.delenv("TRACEA_TUNING_CACHE")
    monkeypatch.delenv("TRACEA_TUNING_HISTORY")
    T.cache_reload()
    T.history_reload()


def _device_name():
    return torch.cuda.get_device_properties(0).name


def test_tune_gemm_records_a_runnable_winner(tracea_gpu, cache_file):
    from tracea_amd import capi, tuner as T
    ok, score, cfg, err = capi.take_result(capi.lib().tracea_tune_gemm(1024, 1024, 512))
    assert ok, err
    cfg = json.loads(cfg)
    assert score > 1.0  # TFLOP/s; any MFMA variant clears this on 1024x1024x512
    assert T.validate(cfg) is None and T.variant_for_config(cfg) >= 0
    disk = json.loads(cache_file.read_text())
    keys = [k for k in disk if k.startswith("gemm_1024_1024_512_")]
    assert len(keys) == 1
    assert disk[keys[0]]["config"] == cfg and disk[keys[0]]["score"] == pytest.approx(score)
    # the same winner in the tuning history (src/optimizer/history.rs), key "HardwareId:OpFingerprint:Precision"
    hist = json.loads((cache_file.parent / "tuning_history.json").read_text())
    entry = hist["%s:%s:F16" % (_device_name(), keys[0])]
    assert entry["backend"] == "Rocm" and entry["config"] == cfg and entry["tflops"] == pytest.approx(score)
    assert entry["explanation"].startswith("Selected Rocm because it achieved %.2f TFLOPS." % score)
    # the operator still computes the right product afterwards (forced variant restored)
    rng = np.random.default_rng(5)
    a = round_f16(rng.standard_normal((1024, 512)).astype(np.float32) / np.sqrt(512))
    b = round_f16(rng.standard_normal((512, 1024)).astype(np.float32))
    c = tracea_gpu.gemm(torch.from_numpy(a).cuda().half(), torch.from_numpy(b).cuda().half())
    assert_close_scaled(c.float().cpu().numpy(), oracle.gemm_f64(a, b), tol_half(512, "f16"), "after tune")


def test_cache_records_for_another_operand_type_or_layout_are_ignored(tracea_gpu, cache_file):
    """A record carries the operand type and the B layout it was measured on; a launch with other operands
    does not take its variant (a record without the tags counts as f16, k-contiguous B)."""
    from tracea_amd import capi, tuner as T
    a = torch.randn(1024, 512, device="cuda")
    b = torch.randn(512, 1024, device="cuda")             # [K, N] row-major: N-contiguous B
    tracea_gpu.gemm(a.half(), b.half())
    default = capi.last_variant("gemm")
    names = capi.variants("gemm")
    planted = [c for c in T.propose_gemm_configs(1024, 1024, 512)
               if names[T.variant_for_config(c)] not in (default, default + "_m16") and c["m_tile"] == 64][0]
    planted_name = names[T.variant_for_config(planted)]
    key = "gemm_1024_1024_512_%s" % _device_name()

    def plant(**tags):
        cache_file.write_text(json.dumps({key: dict(config=planted, score=1.0, timestamp=1, **tags)}))
        T.cache_reload()

    def ran(dtype, bt):
        bb = b.to(dtype)
        tracea_gpu.gemm(a.to(dtype), bb.t().contiguous().t() if bt else bb)
        return capi.last_variant("gemm")

    plant(operand_dtype="bf16", b_layout="n_contiguous")
    assert ran(torch.float16, False) == default and ran(torch.bfloat16, False) == planted_name
    assert ran(torch.bfloat16, True) != planted_name      # same type, B stored [N, K]
    plant(operand_dtype="f16", b_layout="k_contiguous")
    assert ran(torch.float16, True) == planted_name and ran(torch.float16, False) == default
    plant()                                                # no tags: f16, k-contiguous
    assert ran(torch.float16, True) == planted_name and ran(torch.bfloat16, True) != planted_name


def test_autotune_gemm_is_cache_first_and_budgeted(tracea_gpu, cache_file):
    from tracea_amd import tuner as T
    best, score = T.autotune_gemm(512, 512, 256, iterations=4)
    assert score > 0.2 and T.variant_for_config(best) >= 0
    disk = json.loads(cache_file.read_text())
    key = [k for k in disk if k.startswith("gemm_512_512_256_")][0]
    # a planted entry under the same key is what the next call returns, unmeasured
    planted = T.propose_gemm_configs(512, 512, 256)[-1]
    T.cache_put(key, planted, 123.0, 1)
    again, score2 = T.autotune_gemm(512, 512, 256, iterations=0)
    assert again == planted and score2 == 123.0


def test_autotune_conv2d_and_tune_conv2d_agree_on_the_key(tracea_gpu, cache_file):
    from tracea_amd import capi, tuner as T
    best, score = T.autotune_conv2d(2, 32, 16, 16, 32, 3, 3, stride=1, pad=1, iterations=0)
    assert score > 0.01 and best["layout_policy"] == "NHWC"
    ok, score2, cfg, err = capi.take_result(capi.lib().tracea_tune_conv2d(2, 32, 16, 16, 32, 3, 3, 1, 1, 1))
    assert ok, err
    disk = json.loads(cache_file.read_text())
    keys = [k for k in disk if k.startswith("conv_2_16_16_32_32_3_3_1_1_")]
    assert len(keys) == 1  # both wrote the reference's key conv_B_H_W_C_K_R_S_stride_pad_device
    assert T.variant_for_config(json.loads(cfg)) >= 0


def test_tune_fa2_returns_a_flash_variant(tracea_gpu, cache_file):
    from tracea_amd import capi
    ok, score, cfg, err = capi.take_result(capi.lib().tracea_tune_fa2(1, 2, 256, 64, True))
    assert ok, err
    cfg = json.loads(cfg)
    assert cfg["attention_variant"] == "FlashV2" and score > 0.0
    ok, _, _, err = capi.take_result(capi.lib().tracea_tune_fa2(1, 2, 256, 96, True))
    assert not ok and "D 64 or 128" in err
    # the record decides which member of the family later calls on this problem run
    q, k, v = [torch.randn(1, 2, 256, 64, device="cuda").bfloat16() for _ in range(3)]
    tracea_gpu.attention(q, k, v, causal=True)
    ran = capi.last_variant("attention")
    shape = "M16N16K4" if ran.endswith("_m16") else "M32N32K2"
    assert ("q%d_" % cfg["m_tile"]) in ran and cfg["intrinsic_shape"] == shape
    assert cfg["fusion_count"] == (2 if ran.endswith("_x2") else 1)  # query blocks per workgroup
    # without a record: dense attention over a long sequence takes 256 queries on eight waves, one block per
    # workgroup; under a causal mask, with a pair of query blocks per CU or more, 128 on four, two blocks each
    q, k, v = [torch.randn(4, 32, 2048, 128, device="cuda").bfloat16() for _ in range(3)]
    tracea_gpu.attention(q, k, v, causal=False)
    assert capi.last_variant("attention") == "fa2_q256_kv64_d128_s2_pipe2"
    tracea_gpu.attention(q, k, v, causal=True)
    assert capi.last_variant("attention") == "fa2_q128_kv64_d128_pipe2_x2"
    # an odd number of blocks has no pairs; few pairs leave CUs idle
    q, k, v = [torch.randn(4, 32, 2048 + 256, 128, device="cuda").bfloat16() for _ in range(3)]
    tracea_gpu.attention(q, k, v, causal=False)
    assert capi.last_variant("attention") == "fa2_q256_kv64_d128_s2_pipe2"
    q, k, v = [torch.randn(1, 32, 1024, 128, device="cuda").bfloat16() for _ in range(3)]
    tracea_gpu.attention(q, k, v, causal=True)
    assert capi.last_variant("attention") == "fa2_q128_kv64_d128_pipe2"


def test_tuner_cli_writes_the_reference_record(tracea_gpu, cache_file, tmp_path):
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tracea_amd", "bin", "tracea-tuner")
    out = tmp_path / "bench_results.json"
    r = subprocess.run([exe, "gemm", "512", "512", "256", "--out", str(out)], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stderr
    assert "Starting Tuner for GEMM 512x512x256" in r.stdout and "Results saved to" in r.stdout
    rec = json.loads(out.read_text())
    assert list(rec)[:4] == ["timestamp", "kernel", "problem", "best_config"]  # src/bin/tuner.rs:93-102
    assert rec["kernel"] == "gemm" and rec["problem"] == {"m": 512, "n": 512, "k": 256}
    from tracea_amd import tuner as T
    assert T.variant_for_config(rec["best_config"]) >= 0 and rec["score_tflops"] > 0
    # the child process wrote the cache file this process points at
    assert any(k.startswith("gemm_512_512_256_") for k in json.loads(cache_file.read_text()))
    r = subprocess.run([exe, "attention", "1", "2", "256", "64", "--causal", "--out", str(out)], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    rec = json.loads(out.read_text())
    assert rec["kernel"] == "attention" and rec["problem"]["causal"] is True

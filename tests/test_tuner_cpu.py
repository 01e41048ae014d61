"""Host tuner through the C ABI of include/tracea_tuner.h, no GPU needed.

Pins, in order: PipelineConfig (the reference's own unit tests,
src/core/config.rs:481-535, and the record shape of its .tracea/tuning_cache.json),
HardwareProfile (src/optimizer/mod.rs:840-865 golden-config test plus hand
arithmetic), the Gaussian process (tests/gp_interpolation.rs values, then an
independent numpy posterior / likelihood on correlated points), the tuning
cache file format, and the AutoTuner loops on a synthetic benchmark."""
import json
import math
import os

import numpy as np
import pytest

from tracea_amd import tuner as T


# ---- PipelineConfig -----------------------------------------------------------------
def test_pipeline_config_validation_cases_of_the_reference():
    assert T.validate(T.pipeline_config(2, 64, 64, 16)) is None
    assert "m_tile" in T.validate(T.pipeline_config(2, 63, 64, 16))
    assert "n_tile" in T.validate(T.pipeline_config(2, 64, 63, 16))
    assert T.validate(T.pipeline_config(1, 64, 64, 16)) is not None
    assert T.validate(T.pipeline_config(2, 64, 64, 15)) is not None
    c = T.pipeline_config(2, 64, 64, 16)
    for bad in (0, 33):
        c["force_num_warps"] = bad
        assert T.validate(c) is not None
    c["force_num_warps"] = 32
    assert T.validate(c) is None


def test_pipeline_config_json_roundtrip():
    c = T.pipeline_config(3, 128, 64, 32)
    c["double_buffer"] = True
    c["bank_conflict_padding"] = 16
    c["vectorize_epilogue"] = False
    back = T.normalize(json.dumps(c))
    assert back == c
    assert list(back) == list(c)  # field order is the reference's declaration order
    assert len(T.to_vector(c)) > 0


def test_older_record_without_newer_fields_gets_defaults():
    # shape of the records in the reference's .tracea/tuning_cache.json: the four
    # fields added later (double_buffer .. fusion_count) are absent
    old = {"num_stages": 2, "m_tile": 64, "n_tile": 64, "k_tile": 32, "instruction": "CudaMMA",
           "swizzle_mode": "None", "quantization": "None", "layout_policy": "RowMajor", "epilogue": [],
           "force_num_warps": 4, "micro_m": 32, "micro_n": 1, "k_unroll": 1, "prefetch_distance": 0,
           "cp_async_distance": 0, "barrier_mode": "None", "softmax_granularity": "PerTile",
           "intrinsic_shape": "None", "vectorize_epilogue": True, "ttg_enabled": False,
           "attention_variant": "Naive", "gemm_variant": "Naive"}
    full = T.normalize(old)
    for k, v in old.items():
        assert full[k] == v
    assert full["double_buffer"] is False and full["register_strategy"] == "Array"
    assert full["bank_conflict_padding"] == 8 and full["fusion_count"] == 1


def test_to_vector_is_the_key_sorted_flattening():
    c = T.pipeline_config(3, 128, 64, 32)
    c["force_num_warps"] = 8
    c["double_buffer"] = True
    expect = []
    for key in sorted(c):
        v = c[key]
        if isinstance(v, bool):
            expect.append(1.0 if v else 0.0)
        elif isinstance(v, (int, float)):
            expect.append(float(v))
        elif isinstance(v, list):
            assert v == []
        else:  # strings and null
            expect.append(0.0)
    assert T.to_vector(c) == expect


def test_malformed_json_is_an_error_not_a_crash():
    with pytest.raises(ValueError):
        T.validate("{not json")
    with pytest.raises(ValueError):
        T.to_vector('{"m_tile": "sixty-four"}')


# ---- HardwareProfile ----------------------------------------------------------------
def test_golden_config_is_not_pruned_on_the_reference_profile():
    golden = T.pipeline_config(3, 128, 128, 32)
    golden.update(force_num_warps=8, instruction="CudaMMA", swizzle_mode="Xor4", intrinsic_shape="M16N8K16")
    assert T.check_feasibility(golden, 2048, "rtx3070") is None
    # by hand: 8 warps of 32 lanes = 256 threads; regs = 128*128*3/256 + 32 = 224;
    # 65536 / (256*224) = 1 block; by warps 48/8 = 6; 1/16 of the block limit
    assert T.estimate_occupancy(golden, "rtx3070") == pytest.approx(1 / 16)


def test_feasibility_reasons():
    big = T.pipeline_config(4, 256, 256, 64)  # (256*64*2)*2 B * 4 stages = 256 KiB
    assert T.check_feasibility(big, 4096, "mi355x") == "SharedMemoryOverflow"
    ok = T.pipeline_config(2, 256, 256, 64)  # 128 KiB fits 160 KiB of LDS
    assert T.check_feasibility(ok, 4096, "mi355x") is None
    assert T.check_feasibility(ok, 4096, "mi250") == "SharedMemoryOverflow"
    deep = T.pipeline_config(9, 16, 16, 16)
    assert T.check_feasibility(deep, 64, "mi355x").startswith("ForbiddenZone")
    tiny = T.pipeline_config(2, 8, 64, 16)
    assert "Excessive tile-overhead" in T.check_feasibility(tiny, 2048, "mi355x")
    assert T.check_feasibility(tiny, 1024, "mi355x") is None
    # occupancy below 5 %: 32 warps x 32 lanes x (256*256*2/1024 + 32 = 160) registers
    # = 163840 > 65536 per SM -> no block fits
    fat = T.pipeline_config(2, 256, 256, 16)
    fat.update(force_num_warps=32, instruction="CudaMMA")
    assert T.check_feasibility(fat, 256, "a100") == "LowOccupancy(0)"
    assert T.estimate_occupancy(fat, "a100") == 0.0


def test_occupancy_by_hand_on_mi355x():
    c = T.pipeline_config(2, 256, 256, 64)
    c.update(force_num_warps=4, instruction="RocmMFMA")
    # 256 threads; regs = 65536*2/256 + 32 = 544 -> clamped to 512; 256*512 = 131072;
    # 524288 / 131072 = 4 blocks; by waves 32/4 = 8; limit 16 -> 4/16
    assert T.estimate_occupancy(c, "mi355x") == pytest.approx(0.25)
    c["instruction"] = "None"  # 32 registers: by registers 64, by waves 8 -> 8/16
    assert T.estimate_occupancy(c, "mi355x") == pytest.approx(0.5)


def test_profile_numbers():
    p = T.hardware_profile("mi355x")
    assert p["wavefront_size"] == 64 and p["shared_memory_per_block"] == 160 * 1024
    assert p["peak_tflops_tensor"] == 2500.0 and p["mem_bw_gbps"] == 8000.0
    r = T.hardware_profile("rtx3070")
    assert (r["peak_tflops_standard"], r["peak_tflops_tensor"], r["mem_bw_gbps"]) == \
        (pytest.approx(20.3), pytest.approx(40.6), 448.0)
    with pytest.raises(ValueError):
        T.hardware_profile("h100")


# ---- GaussianProcess ----------------------------------------------------------------
def test_gp_interpolates_the_reference_observations():
    gp = T.GaussianProcess("rtx3070", noise_sigma=0.001)
    cfgs = [T.pipeline_config(1, 16, 16, 16), T.pipeline_config(2, 32, 32, 16), T.pipeline_config(2, 64, 64, 16)]
    scores = [15.5, 42.1, 28.3]
    for c, s in zip(cfgs, scores):
        gp.observe(256, 256, 256, c, s)
    for c, s in zip(cfgs, scores):
        mean, std = gp.predict(256, 256, 256, c)
        assert abs(mean - s) < 0.2
        assert std < 0.1


def test_gp_without_observations_returns_the_roofline_prior():
    gp = T.GaussianProcess("rtx3070")
    c = T.pipeline_config(2, 64, 64, 16)
    # 256^3: intensity 2*256^3 / (3*256^2*2) = 85.33 flop/B; 448 GB/s * 85.33 / 1000 = 38.2 > 20.3 peak
    assert gp.predict(256, 256, 256, c) == (pytest.approx(20.3), 1.0)
    c["instruction"] = "CudaMMA"
    assert gp.predict(256, 256, 256, c)[0] == pytest.approx(448.0 * (256 / 3) / 1000.0, rel=1e-6)
    assert T.roofline_prior(16, 16, 16, c, "rtx3070") == pytest.approx(448.0 * (16 / 3) / 1000.0, rel=1e-6)


def _correlated_problem():
    """Five configs that differ by one pipeline stage or unroll step, so that the
    kernel matrix has large off-diagonal entries."""
    cfgs = []
    for stages, unroll in ((2, 1), (3, 1), (4, 1), (2, 2), (3, 2)):
        c = T.pipeline_config(stages, 64, 64, 32)
        c["k_unroll"] = unroll
        cfgs.append(c)
    scores = [18.0, 19.5, 19.0, 17.0, 20.5]
    return cfgs, scores


def _numpy_posterior(feats, y, prior, x, sigma, scales=None):
    f = np.asarray(feats, np.float64)
    ls = np.ones(f.shape[1]) if scales is None else np.asarray(scales, np.float64)
    def kern(a, b):
        d = ((a[:, None, :] - b[None, :, :]) / ls) ** 2
        return np.exp(-0.5 * d.sum(-1))
    K = kern(f, f) + sigma ** 2 * np.eye(len(f))
    ks = kern(np.asarray([x], np.float64), f)[0]
    alpha = np.linalg.solve(K, np.asarray(y) - prior)
    mean = prior + ks @ alpha
    var = max(1.0 - ks @ np.linalg.solve(K, ks), 1e-6)
    sign, logdet = np.linalg.slogdet(K)
    r = np.asarray(y) - prior
    mll = -0.5 * r @ np.linalg.solve(K, r) - 0.5 * logdet - 0.5 * len(f) * math.log(2 * math.pi)
    return mean, math.sqrt(var), mll


def test_gp_posterior_and_likelihood_match_an_independent_solve():
    cfgs, scores = _correlated_problem()
    gp = T.GaussianProcess("rtx3070", noise_sigma=0.3)
    for c, s in zip(cfgs, scores):
        gp.observe(512, 512, 512, c, s)
    feats = [T.features(512, 512, 512, c) for c in cfgs]
    assert len(feats[0]) == 5 + 25 + 3
    np.testing.assert_allclose(feats[0][:5], [9.0, 9.0, 9.0, 1.0, 1.0])
    np.testing.assert_allclose(feats[0][-3:], [64 / 512, 64 / 512, 32 / 512])
    prior = T.roofline_prior(512, 512, 512, cfgs[0], "rtx3070")
    probe = T.pipeline_config(3, 64, 64, 32)
    probe["k_unroll"] = 3  # not an observation
    for target in cfgs + [probe]:
        mean, std, mll = _numpy_posterior(feats, scores, prior, T.features(512, 512, 512, target), 0.3)
        got_mean, got_std = gp.predict(512, 512, 512, target)
        assert got_mean == pytest.approx(mean, abs=2e-4)
        assert got_std == pytest.approx(std, abs=2e-4)
    assert gp.marginal_log_likelihood() == pytest.approx(mll, abs=1e-3)
    # the posterior is not the trivial one: neighbours pull the probe away from the prior
    assert abs(gp.predict(512, 512, 512, probe)[0] - prior) > 0.1


def test_acquisition_functions():
    cfgs, scores = _correlated_problem()
    gp = T.GaussianProcess("rtx3070", noise_sigma=0.3, exploration_beta=2.0)
    for c, s in zip(cfgs, scores):
        gp.observe(512, 512, 512, c, s)
    probe = T.pipeline_config(4, 64, 64, 32)
    probe["k_unroll"] = 2
    mu, sd = gp.predict(512, 512, 512, probe)
    assert gp.ucb(512, 512, 512, probe) == pytest.approx(mu + 2.0 * sd, rel=1e-6)
    best = max(scores)
    z = (mu - best) / sd
    ei = (mu - best) * 0.5 * (1 + math.tanh(z / math.sqrt(2))) + sd * math.exp(-0.5 * z * z) / math.sqrt(2 * math.pi)
    assert gp.expected_improvement(512, 512, 512, probe, best) == pytest.approx(ei, rel=1e-4, abs=1e-6)
    # Thompson: repeatable per seed, distributed as N(mu, sd)
    a = gp.thompson_sample(512, 512, 512, probe, seed=7)
    assert a == gp.thompson_sample(512, 512, 512, probe, seed=7)
    draws = np.array([gp.thompson_sample(512, 512, 512, probe, seed=s) for s in range(1, 2001)])
    assert draws.mean() == pytest.approx(mu, abs=4 * sd / math.sqrt(2000))
    assert draws.std() == pytest.approx(sd, rel=0.08)


def test_hyperparameter_search_does_not_lower_the_likelihood():
    cfgs, scores = _correlated_problem()
    gp = T.GaussianProcess("rtx3070", noise_sigma=0.3)
    for c, s in zip(cfgs, scores):
        gp.observe(512, 512, 512, c, s)
    assert gp.length_scales == [1.0] * 28  # one per config feature
    before = gp.marginal_log_likelihood()
    gp.optimize_hyperparams()
    after = gp.marginal_log_likelihood()
    assert after >= before
    scales = gp.length_scales
    assert all(0.1 <= s <= 10.0 for s in scales)
    assert any(s != 1.0 for s in scales)
    # and the fitted scales are the ones the posterior uses: positions of the
    # scale vector pair with positions of the full feature vector
    feats = [T.features(512, 512, 512, c) for c in cfgs]
    prior = T.roofline_prior(512, 512, 512, cfgs[0], "rtx3070")
    full_scales = scales + [1.0] * (len(feats[0]) - len(scales))
    mean, std, mll = _numpy_posterior(feats, scores, prior, feats[1], 0.3, full_scales)
    assert gp.predict(512, 512, 512, cfgs[1]) == (pytest.approx(mean, abs=5e-4), pytest.approx(std, abs=5e-4))
    assert after == pytest.approx(mll, abs=2e-3)


def test_sixth_to_tenth_observation_triggers_a_refit():
    gp = T.GaussianProcess("rtx3070", noise_sigma=0.3)
    for i in range(10):
        c = T.pipeline_config(2 + i % 4, 64, 64, 32)
        c["k_unroll"] = 1 + i // 4
        gp.observe(512, 512, 512, c, 15.0 + i)
        if i < 9:
            assert gp.length_scales == [1.0] * 28
    assert gp.length_scales != [1.0] * 28  # the 10th observation: len % 5 == 0 and len > 5


# ---- candidates ---------------------------------------------------------------------
def test_proposed_configs_name_compiled_variants():
    from tracea_amd import capi
    names = capi.variants("gemm")
    conv_only = {i for i, nm in enumerate(names) if nm.endswith(("_patch", "_resident", "_ksplit", "_thin"))}
    assert conv_only, "the build has patch-resident convolution variants"
    for propose, expect in ((T.propose_gemm_configs, set(range(len(names))) - conv_only),
                            (T.propose_conv_configs, set(range(len(names))))):
        cands = propose(4096, 4096, 4096)
        idx = [T.variant_for_config(c) for c in cands]
        assert len(idx) == len(set(idx)) and set(idx) == expect  # each eligible variant exactly once
        assert all(T.validate(c) is None for c in cands)
        assert all(c["instruction"] == "RocmMFMA" for c in cands)
        # the MFMA shape is part of the search space: 16x16x32 members under the reference's M16N16K4
        shapes = {names[T.variant_for_config(c)]: c["intrinsic_shape"] for c in cands}
        assert all(sh == ("M16N16K4" if nm.endswith("_m16") or "_w16_" in nm else "M32N32K2") for nm, sh in shapes.items())
        assert sum(nm.endswith("_m16") for nm in shapes) >= 3
    first = T.propose_gemm_configs(4096, 4096, 4096)[0]
    assert T.variant_for_config(first) == capi.lib().tracea_select_variant(b"gemm", 4096, 4096, 4096)
    att = T.propose_attention_configs(128)
    assert att and all(c["attention_variant"] == "FlashV2" for c in att)
    assert T.propose_attention_configs(96) == []


def test_search_space_product_order_and_defaults():
    cands = T.search_space(tile_m=[64, 128], tile_n=[32], tile_k=[16, 32], warps=[4, 8], stages=[2, 3])
    assert len(cands) == 16
    assert [(c["m_tile"], c["k_tile"], c["force_num_warps"], c["num_stages"]) for c in cands[:5]] == \
        [(64, 16, 4, 2), (64, 16, 4, 3), (64, 16, 8, 2), (64, 16, 8, 3), (64, 32, 4, 2)]
    # stages > 2 set the copy distance to stages - 1 (src/optimizer/mod.rs:811-814)
    assert all(c["cp_async_distance"] == (c["num_stages"] - 1 if c["num_stages"] > 2 else 0) for c in cands)
    assert all(c["instruction"] == "RocmMFMA" for c in cands)
    plain = T.search_space(tile_m=[64], use_tensor_core=False, swizzles=["None", "Xor4"])
    assert [c["swizzle_mode"] for c in plain] == ["None", "Xor4"]
    assert plain[0]["instruction"] == "None" and plain[0]["n_tile"] == 64 and plain[0]["num_stages"] == 2


def test_magic_number_strategy():
    assert T.magic_number_strategy(64) == "PowerOfTwo"
    assert T.magic_number_strategy(56 * 56) == "FastSmall"
    assert T.magic_number_strategy(65535) == "FastSmall"
    assert T.magic_number_strategy(65537) == "Standard"
    assert T.magic_number_strategy(0) == "FastSmall"  # the reference's order of tests


# ---- cache --------------------------------------------------------------------------
@pytest.fixture
def cache_file(tmp_path, monkeypatch):
    path = tmp_path / "cache" / "tuning_cache_v2.json"
    monkeypatch.setenv("TRACEA_TUNING_CACHE", str(path))
    T.cache_reload()
    yield path
    monkeypatch.delenv("TRACEA_TUNING_CACHE")
    T.cache_reload()


def test_cache_keys():
    assert T.key_gemm(4096, 4096, 4096, "AMD Instinct MI355X") == "gemm_4096_4096_4096_AMD Instinct MI355X"
    assert T.key_conv2d(32, 56, 56, 64, 64, 3, 3, 1, 1, "gfx950") == "conv_32_56_56_64_64_3_3_1_1_gfx950"


def test_cache_file_format_and_reload(cache_file):
    assert T.cache_path() == str(cache_file)
    assert T.cache_get("gemm_1_2_3_dev") is None
    cfg = T.pipeline_config(2, 128, 128, 64)
    T.cache_put("gemm_1_2_3_dev", cfg, 12.5, 1700000000)
    on_disk = json.loads(cache_file.read_text())
    assert list(on_disk) == ["gemm_1_2_3_dev"]
    entry = on_disk["gemm_1_2_3_dev"]
    assert set(entry) == {"config", "score", "timestamp"}
    assert entry["config"] == cfg and entry["score"] == 12.5 and entry["timestamp"] == 1700000000
    assert "\n  " in cache_file.read_text()  # pretty-printed, as serde_json::to_writer_pretty
    # a file written by another process (or the reference) is picked up after a reload
    on_disk["gemm_9_9_9_dev"] = {"config": {"num_stages": 3, "m_tile": 64, "n_tile": 64, "k_tile": 32},
                                 "score": 1.5, "timestamp": 5}
    cache_file.write_text(json.dumps(on_disk))
    assert T.cache_get("gemm_9_9_9_dev") is None
    T.cache_reload()
    got = T.cache_get("gemm_9_9_9_dev")
    assert got["score"] == 1.5 and got["config"]["num_stages"] == 3 and got["config"]["fusion_count"] == 1


# ---- tuning history (src/optimizer/history.rs:7-51) -----------------------------------
def test_history_file_format_and_reload(tmp_path, monkeypatch):
    path = tmp_path / "tuning_history.json"
    monkeypatch.setenv("TRACEA_TUNING_HISTORY", str(path))
    T.history_reload()
    try:
        assert T.history_path() == str(path)
        assert T.history_query("all:gemm:FP16") is None
        cfg = T.pipeline_config(2, 128, 128, 64)
        T.history_record("all:gemm:FP16", cfg, 1234.567, 0, "Selected based on highest benchmarking score in real-time.")
        on_disk = json.loads(path.read_text())
        assert list(on_disk) == ["all:gemm:FP16"]
        entry = on_disk["all:gemm:FP16"]
        # HistoryEntry's fields (history.rs:7-13); DeviceBackend::Rocm as serde spells a unit variant
        assert set(entry) == {"backend", "config", "tflops", "timestamp", "explanation"}
        assert entry["backend"] == "Rocm" and entry["config"] == cfg and entry["timestamp"] == 0
        assert abs(entry["tflops"] - 1234.567) < 1e-3
        # generate_explanation (history.rs:47-52): "{:?}" of the backend, "{:.2}" of the score
        assert entry["explanation"] == ("Selected Rocm because it achieved 1234.57 TFLOPS. Reason: "
                                        "Selected based on highest benchmarking score in real-time.")
        assert "\n  " in path.read_text()  # to_string_pretty
        # record replaces (HashMap::insert)
        T.history_record("all:gemm:FP16", cfg, 2.0, 7, "again")
        assert T.history_query("all:gemm:FP16")["tflops"] == 2.0
        # a file written by the reference (another backend, the placeholder timestamp) is read after a reload
        on_disk["all:conv:FP16"] = {"backend": "Cuda", "config": {"num_stages": 3, "m_tile": 64, "n_tile": 64, "k_tile": 32},
                                    "tflops": 9.5, "timestamp": 0, "explanation": "Selected Cuda because it achieved 9.50 TFLOPS. Reason: x"}
        path.write_text(json.dumps(on_disk))
        assert T.history_query("all:conv:FP16") is None
        T.history_reload()
        got = T.history_query("all:conv:FP16")
        assert got["backend"] == "Cuda" and got["tflops"] == 9.5 and got["config"]["m_tile"] == 64
        # a file that does not parse is an empty history (load_or_create)
        path.write_text("{ not json")
        T.history_reload()
        assert T.history_query("all:conv:FP16") is None
        with pytest.raises(ValueError):
            T.history_record("", cfg, 1.0)
    finally:
        monkeypatch.delenv("TRACEA_TUNING_HISTORY")
        T.history_reload()


# ---- AutoTuner ----------------------------------------------------------------------
def test_autotune_grid_search_caches_the_winner(cache_file):
    cands = T.propose_gemm_configs(1024, 1024, 1024)
    calls = []

    def measure(cfg):
        calls.append(cfg)
        return 100.0 - abs(cfg["m_tile"] - 128) / 8 - abs(cfg["n_tile"] - 64) / 8 - cfg["cp_async_distance"]

    best, score = T.autotune_candidates("gemm_1024_1024_1024_test", cands, measure)
    assert len(calls) == len(cands)
    assert (best["m_tile"], best["n_tile"], best["cp_async_distance"]) == (128, 64, 0)
    assert score == pytest.approx(100.0)
    assert json.loads(cache_file.read_text())["gemm_1024_1024_1024_test"]["config"] == best
    # second call: served from the cache, nothing measured
    calls.clear()
    again, score2 = T.autotune_candidates("gemm_1024_1024_1024_test", cands, measure)
    assert again == best and score2 == pytest.approx(100.0) and calls == []


def test_autotune_without_a_key_returns_the_first_candidate_unmeasured(cache_file):
    cands = T.propose_attention_configs(128)
    called = []
    best, score = T.autotune_candidates("", cands, lambda c: called.append(c) or 1.0)
    assert best == cands[0] and called == [] and score == 0.0
    assert not cache_file.exists()


def test_autotune_with_no_candidates_falls_back(cache_file):
    best, _ = T.autotune_candidates("gemm_8_8_8_x", [], lambda c: 1.0)
    assert (best["num_stages"], best["m_tile"], best["n_tile"], best["k_tile"]) == (2, 64, 64, 32)


def test_failed_candidates_never_win(cache_file):
    cands = T.propose_gemm_configs(512, 512, 512)

    def measure(cfg):
        if cfg["m_tile"] == 256:
            raise RuntimeError("launch failed")
        return float(cfg["m_tile"])

    best, score = T.autotune_candidates("gemm_512_512_512_t", cands, measure)
    assert best["m_tile"] == 128 and score == 128.0


def test_guided_search_respects_the_budget_and_prunes():
    cands = T.propose_gemm_configs(2048, 2048, 2048)
    bad = T.pipeline_config(9, 64, 64, 32)  # > 8 stages: pruned, never measured
    calls = []

    def measure(cfg):
        calls.append(cfg)
        return 900.0 + cfg["m_tile"] + cfg["n_tile"] - 40.0 * abs(cfg["cp_async_distance"] - 2)

    for acq in (T.EI, T.UCB, T.THOMPSON):
        calls.clear()
        best, score = T.autotune_guided(2048, 2048, 2048, [bad] + cands, measure, iterations=6, acquisition=acq)
        assert len(calls) == 6
        assert all(c["num_stages"] <= 8 for c in calls)
        assert len({json.dumps(c, sort_keys=True) for c in calls}) == 6  # no candidate twice
        assert score == pytest.approx(max(measure(c) for c in calls[:6]))
    # a budget above the candidate count measures each feasible candidate once
    calls.clear()
    best, score = T.autotune_guided(2048, 2048, 2048, [bad] + cands, measure, iterations=100)
    assert len(calls) == len(cands)
    assert (best["m_tile"], best["n_tile"], best["cp_async_distance"]) == (256, 256, 2)


def test_guided_search_finds_the_optimum_on_a_landscape_the_kernel_can_model():
    """The surrogate has unit signal variance and unit length scales on raw
    feature values (the reference's model), so it generalises between configs
    that differ by a few pipeline stages or unroll steps and whose scores lie
    within a few TFLOP/s of the roofline prior.  On such a landscape a budget of
    9 of the 20 feasible candidates must reach the best one."""
    cands = T.search_space(tile_m=[64], tile_n=[64], tile_k=[32], warps=[4], stages=[2, 3, 4, 5, 6, 7, 8],
                           k_unroll=[1, 2, 3, 4], use_tensor_core=False)

    def measure(cfg):
        return 19.0 - 0.3 * (cfg["num_stages"] - 6) ** 2 - 0.5 * (cfg["k_unroll"] - 3) ** 2

    feasible = [c for c in cands if T.check_feasibility(c, 512, "rtx3070") is None]
    assert len(feasible) == 20  # 7 and 8 stages overflow 48 KiB
    top = max(measure(c) for c in feasible)
    for acq in (T.EI, T.UCB):
        seen = []
        best, score = T.autotune_guided(512, 512, 512, cands, lambda c: seen.append(c) or measure(c),
                                        iterations=9, acquisition=acq, profile="rtx3070")
        assert len(seen) == 9
        assert score == pytest.approx(top)
        assert (best["num_stages"], best["k_unroll"]) == (6, 3)

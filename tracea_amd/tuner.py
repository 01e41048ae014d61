"""Tuner objects over the C ABI of ``include/tracea_tuner.h``.

Python counterpart of what the reference exposes to Python and Rust callers:
``PipelineConfig`` records (src/core/config.rs:297-448), ``HardwareProfile``
and ``GaussianProcess`` (src/optimizer/mod.rs:15-576), candidate lists
(src/policy/standard.rs:33-113), the tuning cache (src/core/tuning.rs) and the
``AutoTuner`` loop (src/optimizer/mod.rs:578-760).  Configurations are plain
dicts with the reference's JSON field names.  All logic runs in libtracea.so.
"""
import ctypes as C
import json
import math

from . import capi

EI, UCB, THOMPSON = 0, 1, 2


def _cfg(config):
    return (config if isinstance(config, str) else json.dumps(config)).encode()


def _require(text, what):
    if text is None:
        raise ValueError("%s: %s" % (what, capi.last_error()))
    return text


def _floats(call):
    n = call(None, 0)
    if n < 0:
        raise ValueError(capi.last_error())
    buf = (C.c_float * n)()
    call(buf, n)
    return list(buf)


# ---- PipelineConfig ---------------------------------------------------------------
def pipeline_config(num_stages, m_tile, n_tile, k_tile):
    """PipelineConfig::new as a dict."""
    L = capi.lib()
    return json.loads(capi.take_string(L.tracea_pipeline_config_new(num_stages, m_tile, n_tile, k_tile)))


def normalize(config):
    """from_json -> to_json: missing fields filled with the defaults."""
    text = capi.take_string(capi.lib().tracea_pipeline_config_normalize(_cfg(config)))
    return json.loads(_require(text, "normalize"))


def validate(config):
    """None when valid, else the reference's message."""
    msg = C.c_void_p()
    rc = capi.lib().tracea_pipeline_config_validate(_cfg(config), C.byref(msg))
    if rc < 0:
        raise ValueError(capi.last_error())
    return capi.take_string(msg.value) if rc == 1 else None


def to_vector(config):
    L = capi.lib()
    text = _cfg(config)
    return _floats(lambda buf, n: L.tracea_pipeline_config_to_vector(text, buf, n))


# ---- HardwareProfile --------------------------------------------------------------
def hardware_profile(name="mi355x"):
    text = capi.take_string(capi.lib().tracea_hardware_profile_json(name.encode()))
    return json.loads(_require(text, "hardware_profile"))


def check_feasibility(config, m, profile="mi355x"):
    """None when feasible, else the pruning reason."""
    reason = C.c_void_p()
    rc = capi.lib().tracea_check_feasibility(profile.encode(), _cfg(config), m, C.byref(reason))
    if rc < 0:
        raise ValueError(capi.last_error())
    return capi.take_string(reason.value) if rc == 1 else None


def estimate_occupancy(config, profile="mi355x"):
    v = capi.lib().tracea_estimate_occupancy(profile.encode(), _cfg(config))
    if v < 0:
        raise ValueError(capi.last_error())
    return v


# ---- GaussianProcess --------------------------------------------------------------
class GaussianProcess:
    def __init__(self, profile="mi355x", noise_sigma=None, exploration_beta=None):
        self._L = capi.lib()
        self._h = self._L.tracea_gp_create()
        self.profile = profile.encode()
        if noise_sigma is not None:
            self._L.tracea_gp_set_noise_sigma(self._h, noise_sigma)
        if exploration_beta is not None:
            self._L.tracea_gp_set_exploration_beta(self._h, exploration_beta)

    def __del__(self):
        if getattr(self, "_h", None):
            self._L.tracea_gp_destroy(self._h)
            self._h = None

    def observe(self, m, n, k, config, score):
        if self._L.tracea_gp_observe(self._h, m, n, k, _cfg(config), score, self.profile) != 0:
            raise ValueError(capi.last_error())

    def predict(self, m, n, k, config):
        mean, std = C.c_float(), C.c_float()
        if self._L.tracea_gp_predict(self._h, m, n, k, _cfg(config), self.profile, C.byref(mean),
                                     C.byref(std)) != 0:
            raise ValueError(capi.last_error())
        return mean.value, std.value

    def _acq(self, kind, m, n, k, config, best_y=0.0, seed=0):
        v = self._L.tracea_gp_acquisition(self._h, kind, m, n, k, _cfg(config), self.profile, best_y, seed)
        if math.isnan(v):
            raise ValueError(capi.last_error())
        return v

    def expected_improvement(self, m, n, k, config, best_y):
        return self._acq(EI, m, n, k, config, best_y)

    def ucb(self, m, n, k, config):
        return self._acq(UCB, m, n, k, config)

    def thompson_sample(self, m, n, k, config, seed):
        return self._acq(THOMPSON, m, n, k, config, 0.0, seed)

    def marginal_log_likelihood(self):
        return self._L.tracea_gp_marginal_log_likelihood(self._h, self.profile)

    def optimize_hyperparams(self):
        self._L.tracea_gp_optimize_hyperparams(self._h, self.profile)

    @property
    def length_scales(self):
        return _floats(lambda buf, n: self._L.tracea_gp_length_scales(self._h, buf, n))


def features(m, n, k, config):
    L = capi.lib()
    text = _cfg(config)
    return _floats(lambda buf, cap: L.tracea_gp_features(m, n, k, text, buf, cap))


def roofline_prior(m, n, k, config, profile="mi355x"):
    return capi.lib().tracea_gp_roofline_prior(m, n, k, _cfg(config), profile.encode())


# ---- candidates -------------------------------------------------------------------
def propose_gemm_configs(m, n, k):
    return json.loads(capi.take_string(capi.lib().tracea_propose_gemm_configs(m, n, k)))


def propose_conv_configs(m, n, k):
    return json.loads(capi.take_string(capi.lib().tracea_propose_conv_configs(m, n, k)))


def propose_attention_configs(head_dim):
    return json.loads(capi.take_string(capi.lib().tracea_propose_attention_configs(head_dim)))


def search_space(**axes):
    """SearchSpace product, e.g. search_space(tile_m=[64, 128], stages=[2, 3])."""
    text = capi.take_string(capi.lib().tracea_search_space_enumerate(json.dumps(axes).encode()))
    return json.loads(_require(text, "search_space"))


def variant_for_config(config):
    return capi.lib().tracea_variant_for_config(_cfg(config))


def magic_number_strategy(divisor):
    return capi.lib().tracea_magic_number_strategy(divisor).decode()


# ---- tuning cache -----------------------------------------------------------------
def cache_path():
    return capi.take_string(capi.lib().tracea_tuning_cache_path())


def cache_get(key):
    text = capi.take_string(capi.lib().tracea_tuning_cache_get(key.encode()))
    return None if text is None else json.loads(text)


def cache_put(key, config, score, timestamp=0):
    if capi.lib().tracea_tuning_cache_put(key.encode(), _cfg(config), score, timestamp) != 0:
        raise ValueError(capi.last_error())


def cache_reload():
    capi.lib().tracea_tuning_cache_reload()


# ---- tuning history (src/optimizer/history.rs) ---------------------------------------
def history_path():
    return capi.take_string(capi.lib().tracea_tuning_history_path())


def history_record(key, config, tflops, timestamp=0, reason=""):
    if capi.lib().tracea_tuning_history_record(key.encode(), _cfg(config), tflops, timestamp, reason.encode()) != 0:
        raise ValueError(capi.last_error())


def history_query(key):
    text = capi.take_string(capi.lib().tracea_tuning_history_query(key.encode()))
    return None if text is None else json.loads(text)


def history_reload():
    capi.lib().tracea_tuning_history_reload()


def key_gemm(m, n, k, device):
    return capi.take_string(capi.lib().tracea_tuning_key_gemm(m, n, k, device.encode()))


def key_conv2d(batch, h, w, c, k, r, s, stride, pad, device):
    return capi.take_string(
        capi.lib().tracea_tuning_key_conv2d(batch, h, w, c, k, r, s, stride, pad, device.encode()))


# ---- AutoTuner --------------------------------------------------------------------
def _wrap(measure):
    def thunk(text, _user):
        try:
            return float(measure(json.loads(text.decode())))
        except Exception:  # a failing candidate scores 0, as a failed launch does
            return 0.0
    return capi.MEASURE_FN(thunk)


def _result(res, what):
    ok, score, cfg, err = capi.take_result(res)
    if not ok:
        raise RuntimeError("%s: %s" % (what, err))
    return json.loads(cfg), score


def autotune_candidates(key, candidates, measure):
    """optimize_v2: cached key wins, else grid search; returns (config, score)."""
    cb = _wrap(measure)
    res = capi.lib().tracea_autotune_candidates((key or "").encode(), json.dumps(candidates).encode(), cb, None)
    return _result(res, "autotune_candidates")


def autotune_guided(m, n, k, candidates, measure, iterations, acquisition=EI, seed=1, profile="mi355x"):
    cb = _wrap(measure)
    res = capi.lib().tracea_autotune_guided(profile.encode(), m, n, k, json.dumps(candidates).encode(), cb,
                                            None, iterations, acquisition, seed)
    return _result(res, "autotune_guided")


def autotune_gemm(m, n, k, iterations=0):
    """On the device; needs capi.init()."""
    return _result(capi.lib().tracea_autotune_gemm(m, n, k, iterations), "autotune_gemm")


def autotune_conv2d(n, c, h, w, k, r, s, stride=1, pad=0, dilation=1, iterations=0):
    return _result(capi.lib().tracea_autotune_conv2d(n, c, h, w, k, r, s, stride, pad, dilation, iterations),
                   "autotune_conv2d")

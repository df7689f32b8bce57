"""Host-side surface: dtype aliases, config defaults, enums, string parsers.

The expected literals are the ones the reference's own tests hold
(tests/optim/test_fp8.py:36-97 aliases, :103-159 defaults, :165-169 enums,
:175-201 parser aliases and error text; tests/model/test_transformer_engine_transform.py:174-200
transform-config defaults), restated here.
"""
import pytest
import torch

from optimus_dl_amd.core.dtype import get_fp8_format_from_dtype, is_fp8_dtype, str_to_dtype
from optimus_dl_amd.modules.amp import (
    AmpConfig,
    Fp8Config,
    Fp8Format,
    Fp8RecipeConfig,
    Fp8RecipeType,
    get_fp8_format_from_string,
    get_fp8_recipe_type_from_string,
    is_transformer_engine_available,
)
from optimus_dl_amd.modules.model_transforms.transformer_engine import TransformerEngineTransformConfig


@pytest.mark.parametrize("name", ["float8_e4m3fn", "fp8_e4m3fn", "e4m3fn", "e4m3", "float8_e4m3", "fp8_e4m3"])
def test_e4m3_aliases(name):
    assert str_to_dtype(name) == torch.float8_e4m3fn
    assert str_to_dtype("torch." + name) == torch.float8_e4m3fn


@pytest.mark.parametrize("name", ["float8_e5m2", "fp8_e5m2", "e5m2fn", "e5m2", "float8_e5m2fn", "fp8_e5m2fn"])
def test_e5m2_aliases(name):
    assert str_to_dtype(name) == torch.float8_e5m2
    assert str_to_dtype("torch." + name) == torch.float8_e5m2


def test_plain_dtypes_and_errors():
    assert str_to_dtype("torch.bfloat16") == torch.bfloat16 and str_to_dtype("bf16") == torch.bfloat16
    assert str_to_dtype("fp16") == torch.float16 and str_to_dtype("float32") == torch.float32
    with pytest.raises(ValueError, match="Unsupported dtype string"):
        str_to_dtype("fp7")


def test_fp8_dtype_predicates():
    assert is_fp8_dtype(torch.float8_e4m3fn) and is_fp8_dtype(torch.float8_e5m2)
    assert not is_fp8_dtype(torch.bfloat16) and not is_fp8_dtype(torch.float16) and not is_fp8_dtype(torch.float32)
    assert get_fp8_format_from_dtype(torch.float8_e4m3fn) == "e4m3fn"
    assert get_fp8_format_from_dtype(torch.float8_e5m2) == "e5m2"
    assert get_fp8_format_from_dtype(torch.bfloat16) is None


def test_fp8_config_defaults():
    c = Fp8Config()
    assert c.enabled is False and c.format == "hybrid" and c.recipe == "delayed" and c.param is False
    assert c.margin == 0 and c.amax_history_len == 1024 and c.amax_compute_algo == "max" and c.reduce_amax is True
    assert c.wgrad is True and c.fp8_dpa is False and c.fp8_mha is False and c.first_last_layers_bf16 is False
    assert c.num_layers_at_start_in_bf16 == 1 and c.num_layers_at_end_in_bf16 == 1 and c.tp_only_amax_red is False


def test_amp_config():
    a = AmpConfig(enabled=True, dtype="torch.float8_e4m3fn", enable_scaler=False, fp8=Fp8Config(enabled=True, format="hybrid"))
    assert a.enabled and a.dtype == "torch.float8_e4m3fn" and a.enable_scaler is False
    assert a.fp8.enabled and a.fp8.format == "hybrid"
    d = AmpConfig()
    assert d.enabled is False and d.dtype == "torch.bfloat16" and d.init_scale == 2 ** 16
    assert d.growth_factor == 2.0 and d.backoff_factor == 0.5 and d.growth_interval == 2000 and d.fp8.enabled is False
    # the scaler default is "on for fp16 only"
    assert AmpConfig(dtype="torch.float16").resolved_enable_scaler() is True
    assert AmpConfig(dtype="torch.bfloat16").resolved_enable_scaler() is False
    # YAML-shaped nested dicts are accepted
    y = AmpConfig(enabled=True, dtype="torch.float8_e4m3fn", fp8={"enabled": True, "format": "e4m3", "amax_history_len": 16})
    assert y.fp8.amax_history_len == 16 and y.fp8.format == "e4m3"


def test_enums():
    assert Fp8Format.HYBRID.value == "hybrid" and Fp8Format.E4M3.value == "e4m3" and Fp8Format.E5M2.value == "e5m2"
    assert Fp8RecipeType.DELAYED.value == "delayed" and Fp8RecipeType.TENSORWISE.value == "tensorwise"
    assert Fp8RecipeType.BLOCKWISE.value == "blockwise" and Fp8RecipeType.MXFP8.value == "mxfp8"
    assert Fp8RecipeType("delayed") is Fp8RecipeType.DELAYED and Fp8RecipeType.DELAYED == "delayed"


def test_format_parser():
    for s in ("hybrid", "HYBRID", "hybrid_fp8", "fp8_hybrid"):
        assert get_fp8_format_from_string(s) == Fp8Format.HYBRID
    for s in ("e4m3", "fp8_e4m3", "e4m3fn", "float8_e4m3fn", "E4M3"):
        assert get_fp8_format_from_string(s) == Fp8Format.E4M3
    for s in ("e5m2", "fp8_e5m2", "e5m2fn", "float8_e5m2"):
        assert get_fp8_format_from_string(s) == Fp8Format.E5M2
    with pytest.raises(ValueError, match="Unknown FP8 format"):
        get_fp8_format_from_string("invalid_format")
    # the message names the lower-cased string, as optimus_dl/modules/amp/fp8.py:109,116 prints it
    with pytest.raises(ValueError, match=r"Unknown FP8 format: bogus_fmt\. Supported formats: hybrid, e4m3, e5m2"):
        get_fp8_format_from_string("Bogus_FMT")


def test_recipe_parser():
    # alias sets transcribed from optimus_dl/modules/amp/fp8.py:134-147
    table = {
        Fp8RecipeType.DELAYED: ("delayed", "delayed_scaling", "Delayed"),
        Fp8RecipeType.TENSORWISE: ("tensorwise", "tensor_wise", "current", "current_scaling"),
        Fp8RecipeType.BLOCKWISE: ("blockwise", "block_wise", "float8_block"),
        Fp8RecipeType.MXFP8: ("mxfp8", "mxfp8_block"),
        Fp8RecipeType.ROWWISE: ("rowwise",),
    }
    for want, names in table.items():
        for n in names:
            assert get_fp8_recipe_type_from_string(n) == want
    with pytest.raises(ValueError, match="Unknown FP8 recipe type"):
        get_fp8_recipe_type_from_string("nope")
    with pytest.raises(ValueError, match=r"Unknown FP8 recipe type: nope_x\. Supported types: delayed, tensorwise, blockwise, mxfp8"):
        get_fp8_recipe_type_from_string("NOPE_x")


def test_recipe_config_defaults():
    c = Fp8RecipeConfig()
    assert (c.recipe_type, c.format, c.margin, c.amax_history_len, c.amax_compute_algo, c.reduce_amax, c.fp8_dpa, c.fp8_mha) == \
        ("delayed", "hybrid", 0, 1024, "max", True, False, False)


def test_availability_is_bool():
    assert isinstance(is_transformer_engine_available(), bool)


def test_transform_config_defaults_and_custom():
    c = TransformerEngineTransformConfig()
    assert c.enabled is True and c.replace_linear is True and c.replace_norm is True and c.replace_attention is False
    assert c.linear_kwargs == {} and c.norm_kwargs == {} and c.attention_kwargs == {}
    assert c.replace_inplace is True and c.verbose is False
    c2 = TransformerEngineTransformConfig(enabled=False, replace_linear=False, linear_kwargs={"sequence_parallel": True}, verbose=True)
    assert c2.enabled is False and c2.replace_linear is False and c2.linear_kwargs == {"sequence_parallel": True} and c2.verbose


def test_yaml_presets_of_the_reference_parse():
    """The key sets of the reference's YAML groups (configs/train/optimization/amp/fp8_hybrid.yaml,
    configs/model/transforms/transformer_engine.yaml), typed here as literals."""
    import yaml

    amp_yaml = yaml.safe_load("""
enabled: true
dtype: torch.float8_e4m3fn
enable_scaler: false
fp8:
  enabled: true
  format: hybrid
  recipe: delayed
  param: false
  margin: 0
  amax_history_len: 1024
  amax_compute_algo: max
  reduce_amax: true
  wgrad: true
  fp8_dpa: false
  fp8_mha: false
""")
    a = AmpConfig(**amp_yaml)
    assert a.fp8.enabled and a.fp8.recipe == "delayed" and is_fp8_dtype(str_to_dtype(a.dtype))
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    t = build_model_transform(yaml.safe_load("""
_name: transformer_engine
enabled: true
replace_linear: true
replace_norm: false
replace_attention: false
linear_kwargs: {sequence_parallel: false}
replace_inplace: true
verbose: false
an_unknown_key: 3
"""))
    assert t.cfg.replace_norm is False and t.cfg.linear_kwargs == {"sequence_parallel": False} and t.cfg["an_unknown_key"] == 3

"""Host logic and the C ABI surface; runs without a GPU."""
import ctypes as C
import json
import os
import re

import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import ROOT, has_gpu
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth


def test_library_exports_every_symbol_the_header_declares():
    header = open(os.path.join(ROOT, "include", "rbmoe.h")).read()
    declared = set(re.findall(r"\b(rbmoe_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = L.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared in rbmoe.h but not exported"
    assert declared == set(L.SIGNATURES), (declared ^ set(L.SIGNATURES))
    assert b"gfx950" in lib.rbmoe_version()


def test_config_struct_layout_matches_the_header():
    assert C.sizeof(L.Config) == 11 * 4
    assert C.sizeof(L.Routing) == 8 * C.sizeof(C.c_void_p)


def test_config_init_gives_the_reference_defaults():
    cfg = L.Config()
    assert L.load().rbmoe_config_init(C.byref(cfg), 64, 8, 2, 32) == L.OK
    assert (cfg.d_model, cfg.num_experts, cfg.experts_per_token, cfg.d_ff) == (64, 8, 2, 32)
    assert cfg.shared_expert == 0
    assert abs(cfg.aux_loss_weight - 0.01) < 1e-9 and abs(cfg.router_z_loss_weight - 1e-3) < 1e-9


def test_invalid_top_k_is_rejected():
    # reference src/moe.rs:704-710
    for cfg in (rb.MoeConfig.new(4, 0, 6), rb.MoeConfig.new(4, 5, 6), rb.MoeConfig.new(0, 1, 6)):
        with pytest.raises(rb.InvalidConfig):
            cfg.validate()
    rb.MoeConfig.new(4, 4, 6).validate()


def test_validate_uses_the_reference_wording():
    with pytest.raises(rb.InvalidConfig, match="a MoE layer needs at least one expert"):
        rb.MoeConfig.new(0, 1, 6).validate()
    with pytest.raises(rb.InvalidConfig, match=r"experts_per_token must be between 1 and num_experts \(4\), got 5"):
        rb.MoeConfig.new(4, 5, 6).validate()
    with pytest.raises(rb.InvalidConfig, match="expert d_ff must be non-zero"):
        rb.MoeConfig.new(4, 2, 0).validate()


def test_limits_are_reported_as_unsupported():
    with pytest.raises(rb.Unsupported):
        rb.MoeConfig.new(512, 2, 8).validate()
    with pytest.raises(rb.Unsupported):
        rb.MoeConfig.new(64, 40, 8).validate()


def test_builder_methods_and_with_methods_mirror_the_reference():
    cfg = rb.MoeConfig.new(8, 2, 32).with_shared_expert(True).with_aux_loss_weight(0.5).with_router_z_loss_weight(0.0)
    assert cfg.shared_expert and cfg.aux_loss_weight == 0.5 and cfg.router_z_loss_weight == 0.0
    b = (rb.TransformerBuilder().d_model(768).experts(16, 2).moe_layers([1, 3]).shared_expert(False)
         .moe_d_ff(1408).aux_loss_weight(0.02).router_z_loss_weight(0.0))
    mc = b._config.moe_config()
    assert mc == rb.MoeConfig(16, 2, 1408, False, 0.02, 0.0)
    assert b._config.is_moe_layer(3) and not b._config.is_moe_layer(2)


def test_default_parameter_accounting_is_exact():
    # reference README.md:96 / src/transformer.rs:194-227: 55.2M total / 35.7M active (1.54x)
    c = rb.TransformerBuilder().parameter_counts()
    assert (c.total, c.active) == (55_181_824, 35_717_632)
    assert f"{c.total / 1e6:.1f}M / {c.active / 1e6:.1f}M ({c.total / c.active:.2f}x)" == "55.2M / 35.7M (1.54x)"


def test_parameter_table_of_the_tutorial():
    # reference tutorials/15_mixture_of_experts.md:276-283
    want = {1: ("32.5", "32.5"), 2: ("35.7", "35.7"), 4: ("42.2", "35.7"), 8: ("55.2", "35.7"),
            16: ("81.2", "35.7"), 32: ("133.1", "35.8")}
    for n, (total, active) in want.items():
        c = rb.TransformerBuilder().experts(n, min(2, n)).parameter_counts()
        assert (f"{c.total / 1e6:.1f}", f"{c.active / 1e6:.1f}") == (total, active)


def test_layer_parameter_counts_through_the_abi():
    cfg = rb.MoeConfig.new(8, 2, 352).with_shared_expert(True)._c(512)
    total, active = C.c_uint64(), C.c_uint64()
    assert L.load().rbmoe_parameter_counts(C.byref(cfg), C.byref(total), C.byref(active)) == L.OK
    expert = 3 * 512 * 352
    assert total.value == 8 * 512 + 8 * expert + expert
    assert active.value == 8 * 512 + 2 * expert + expert


def test_an_invalid_configuration_is_rejected_before_allocation():
    # reference src/transformer.rs:3020-3026 — no device is needed to be told so
    tiny = lambda: rb.TransformerBuilder().n_layers(2).moe_layers([1]).experts(4, 2)
    for bad in (tiny().heads(4, 3, 4), tiny().heads(4, 2, 5), tiny().moe_layers([9]), tiny().experts(2, 4)):
        with pytest.raises(rb.InvalidConfig):
            bad.build_moe_layers(device=None)


def test_layout_check():
    # reference src/batch.rs:254-268
    rb.Layout().check(7)
    rb.Layout(seq_len=4).check(8)
    with pytest.raises(rb.InvalidConfig, match="9 rows do not divide into sequences of 4"):
        rb.Layout(seq_len=4).check(9)
    with pytest.raises(rb.InvalidConfig, match="padding mask covers 3 rows, not 4"):
        rb.Layout(valid=[True, False, True]).check(4)
    assert rb.Layout(valid=[True, False]).is_valid(0) and not rb.Layout(valid=[True, False]).is_valid(1)


@pytest.mark.skipif(has_gpu(), reason="checks the fail-closed path of a machine without a GPU")
def test_opening_a_device_without_a_gpu_fails_closed():
    with pytest.raises(rb.BackendUnavailable):
        rb.Device.open(0)


def test_null_arguments_are_reported_not_dereferenced():
    lib = L.load()
    assert lib.rbmoe_validate(None, None, 0) == L.NULL_POINTER
    assert lib.rbmoe_ctx_create(0, 0, None) == L.NULL_POINTER
    assert lib.rbmoe_forward(None, None, 1, 1, None, None, None, None) == L.NULL_POINTER
    assert lib.rbmoe_get_losses(None, None, None) == L.NULL_POINTER
    assert lib.rbmoe_set_weight(None, 0, 0, None, 0, None, 1, 1) == L.NULL_POINTER
    assert b"NULL" in lib.rbmoe_last_global_error()


# ------------------------------------------------------------------ synthetic data
def test_generator_matches_its_golden_values():
    gold = json.load(open(os.path.join(ROOT, "tests", "golden", "synth_golden.json")))
    assert synth.uniform((6,), 1.0, 42, 7).tolist() == gold["uniform_seed42_stream7"]
    assert synth.normal((6,), 1.0, 42, 7).tolist() == gold["normal_seed42_stream7"]
    t = synth.make("c2_decode_d768_e8")
    assert t.x[0, :4].tolist() == gold["c2_x_first4"]
    assert t.experts[3]["down"][5, :4].tolist() == gold["c2_expert3_down_row5_first4"]


def test_generator_distributions():
    x = synth.normal((200_000,), 1.0, 5, 1)
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1.0) < 0.01
    w = synth.xavier_uniform(1408, 768, 5, 2)
    bound = np.sqrt(6.0 / (1408 + 768))
    assert np.abs(w).max() <= bound and np.abs(w).max() > 0.999 * bound
    assert abs(float(w.std()) - bound / np.sqrt(3)) < 1e-3


def test_bf16_rounding_is_nearest_even():
    vals = np.array([1.0, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, 1.0 + 2 ** -9, -2.5, 3.0e38], np.float32)
    bits = synth.f32_to_bf16_bits(vals)
    back = synth.bf16_bits_to_f32(bits)
    assert back.tolist()[:5] == [1.0, 1.0, 1.0 + 2 ** -6, 1.0, -2.5]  # ties go to the even mantissa
    assert np.isinf(back[5]) or back[5] > 2.9e38
    again = synth.round_bf16(back)
    assert np.array_equal(again, back)


def test_skewed_workload_puts_about_thirty_percent_on_expert_zero():
    t = synth.make("c3_prefill_d768_e16", tokens=2048)
    logits = t.x.astype(np.float64) @ t.router.astype(np.float64).T + t.router_bias
    top = np.argsort(-logits, axis=1, kind="stable")[:, :2]
    assert 0.28 <= float(np.mean(top == 0)) <= 0.32


def test_weight_gradient_workspace_holds_every_batch_up_to_max_tokens():
    """The ordered weight gradients keep one partial matrix per further chunk of a cut expert.  How many a launch
    cuts out depends on its own row count (not monotonically), the buffer is sized once for max_tokens: it must
    hold what every token count up to max_tokens asks for."""
    import ctypes as C
    lib = L.load()
    fn = lib.rbmoe_internal_weight_grad_slots
    fn.restype = C.c_int
    fn.argtypes = [C.c_int32] * 8 + [C.POINTER(C.c_int64)] * 2
    cases = [(768, 2048, 16, 0, 2, 1, 1200), (4096, 768, 16, 0, 2, 1, 2000), (768, 2048, 16, 0, 2, 1, 3072),
             (768, 1408, 16, 0, 2, 1, 1536), (1024, 704, 64, 0, 6, 1, 900), (512, 1408, 8, 0, 2, 0, 1024),
             (768, 1408, 1, 1, 1, 1, 1300), (2816, 768, 1, 1, 1, 1, 700)]
    for M, N, groups, dense, k, bf16, max_tokens in cases:
        need, held = C.c_int64(), C.c_int64()
        worst = 0
        for tokens in range(1, max_tokens + 1):
            assert fn(M, N, groups, dense, tokens, k, bf16, max_tokens, C.byref(need), C.byref(held)) == L.OK
            worst = max(worst, need.value)
            assert need.value <= held.value, (M, N, groups, tokens, need.value, held.value)
        assert worst == held.value   # and no more than the worst case asks for


def test_bench_helper_library_exports_what_its_header_declares():
    header = open(os.path.join(ROOT, "include", "rbmoe_bench.h")).read()
    declared = set(re.findall(r"\b(rbbench_[a-z_0-9]+)\s*\(", header))
    assert declared == set(L.BENCH_SIGNATURES), (declared ^ set(L.BENCH_SIGNATURES))
    lib = L.load_bench()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared in rbmoe_bench.h but not exported"
    # ... and the layer's library holds none of it
    main = L.load()
    assert not [n for n in declared if hasattr(main, n)]
    assert not hasattr(main, "rbmoe_calibrate_mfma")

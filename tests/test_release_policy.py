"""Release kernel plan and environment validation against the cases of the reference's own test
(`tests/test_release_policy.py:12-52`, held as data in tests/golden/release_policy_cases.json) and against the
kernel families its policy names for the benchmark configurations (`release_policy.py:377-494`)."""
import json
import os

import pytest

from jetfire_amd.adapter.release_policy import (EXPERIMENTAL_RELEASE_ENV, RELEASE_MODES, RELEASE_TOP_K, STAGE_OPERATORS,
                                                ReleasePolicyError, iter_release_matrix, plan_release_graph,
                                                validate_release_environment)

CASES = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "release_policy_cases.json")))


@pytest.fixture
def clean_env(monkeypatch):
    for name in list(os.environ):
        if name.startswith("JETFIRE_"):
            monkeypatch.delenv(name)
    return monkeypatch


def test_batched_int4_v_policy_has_required_stage_a_statistics(clean_env):
    c = CASES["batched_int4_v"]
    for k_bits in c["k_bits"]:
        for top_k in c["top_k"]:
            plan = plan_release_graph(mode=f"SymInt{k_bits}K_SymInt4V", group_size=c["group_size"], top_k=top_k,
                                      max_graph_batch=c["max_graph_batch"], stageb_candidate=c["stageb_candidate"],
                                      require_ready=c["require_ready"])
            if plan.stage_b == "sv_int8tc_reg_stats":
                assert plan.stage_a == "qk_int8tc_stats"
            else:
                assert plan.stage_b == "sv_int4_wvs2_scores"
    # and the cells themselves: only INT4 keys at a width the int8 Stage A takes get the int8-weight Stage B
    assert plan_release_graph(mode="SymInt4K_SymInt4V", group_size=128, top_k=256, max_graph_batch=2).stage_b == "sv_int8tc_reg_stats"
    assert plan_release_graph(mode="SymInt4K_SymInt4V", group_size=128, top_k=32, max_graph_batch=2).stage_a == "qk_int4_split_topk"
    assert plan_release_graph(mode="SymInt3K_SymInt4V", group_size=128, top_k=256, max_graph_batch=2).stage_b == "sv_int4_wvs2_scores"


@pytest.mark.parametrize("case", CASES["environment"], ids=lambda c: ",".join(sorted(c["set"]))[-60:])
def test_release_environment_cases(clean_env, case):
    for k, v in case["set"].items():
        clean_env.setenv(k, v)
    if case["raises"]:
        with pytest.raises(ReleasePolicyError, match=case["raises"]):
            validate_release_environment()
    else:
        validate_release_environment()


@pytest.mark.parametrize("cfg", CASES["configurations"], ids=lambda c: f'{c["mode"]}-g{c["group_size"]}-k{c["top_k"]}-b{c["max_graph_batch"]}')
def test_benchmark_configurations_get_the_reference_kernel_families(clean_env, cfg):
    plan = plan_release_graph(mode=cfg["mode"], group_size=cfg["group_size"], top_k=cfg["top_k"],
                              max_graph_batch=cfg["max_graph_batch"], require_ready=True)
    for key in ("stage_a", "stage_b", "num_quant_groups", "release_ready"):
        assert getattr(plan, key) == cfg[key], key
    assert plan.correction_sync == "cpu_topk_host_join" and plan.graph_scope == "decode_only"
    from jetfire_amd import ops
    for name in plan.operators():
        assert name is not None and callable(getattr(ops, name))


def test_policy_is_total_and_strict(clean_env):
    plans = iter_release_matrix()
    assert len(plans) == len(RELEASE_MODES) * 2 * len(RELEASE_TOP_K) and all(p.release_ready for p in plans)
    assert {p.stage_a for p in plans} | {p.stage_b for p in plans} <= set(STAGE_OPERATORS)
    for bad in (dict(mode="AsymInt2K_SymInt2V"), dict(group_size=32), dict(top_k=48), dict(head_dim=64), dict(max_graph_batch=0)):
        args = dict(mode="SymInt3K_SymInt2V", group_size=64, top_k=256)
        args.update(bad)
        with pytest.raises(ReleasePolicyError):
            plan_release_graph(**args)
    # a Stage B candidate is a non-release plan: it exists, says why it is blocked, and cannot be required
    cand = plan_release_graph(mode="SymInt3K_SymInt2V", group_size=128, top_k=256, stageb_candidate="int2-v2")
    assert not cand.release_ready and cand.stage_b == "sv_int2_v2" and "promotion evidence" in cand.blockers[0]
    with pytest.raises(ReleasePolicyError, match="not ready"):
        cand.assert_ready()
    with pytest.raises(ReleasePolicyError, match="require_ready=False"):
        plan_release_graph(mode="SymInt3K_SymInt2V", group_size=128, top_k=256, stageb_candidate="int2-v2", require_ready=True)
    with pytest.raises(ReleasePolicyError, match="one V scale group"):
        plan_release_graph(mode="SymInt3K_SymInt2V", group_size=64, top_k=256, stageb_candidate="int2-wvs2")
    with pytest.raises(ReleasePolicyError, match="only applies to INT2 V"):
        plan_release_graph(mode="SymInt4K_SymInt4V", group_size=128, top_k=256, stageb_candidate="int2-v2")


def test_environment_validation_details(clean_env):
    validate_release_environment()                                   # policy off: anything goes
    clean_env.setenv("JETFIRE_USE_FUSED_ATTN_TOPK", "1")
    validate_release_environment()
    clean_env.setenv("JETFIRE_RELEASE_GRAPH_POLICY", "1")
    with pytest.raises(ReleasePolicyError, match="JETFIRE_USE_FUSED_ATTN_TOPK"):
        validate_release_environment()
    clean_env.delenv("JETFIRE_USE_FUSED_ATTN_TOPK")
    clean_env.setenv("JETFIRE_USE_INT8_TC", "1")                      # the canonical value of a switch is allowed
    clean_env.setenv("JETFIRE_SHADOW_DEVICE", "CPU")
    validate_release_environment()
    clean_env.setenv("JETFIRE_USE_INT8_TC", "0")
    with pytest.raises(ReleasePolicyError, match="JETFIRE_USE_INT8_TC='0'"):
        validate_release_environment()
    clean_env.setenv("JETFIRE_USE_INT8_TC", "1")
    clean_env.setenv("JETFIRE_GRAPH_GPU_WAIT_CPU_TOPK", "1")
    with pytest.raises(ReleasePolicyError):
        validate_release_environment()
    clean_env.setenv("JETFIRE_ALLOW_EXPERIMENTAL_GRAPH_CPU_TOPK", "1")   # is itself an experimental switch
    with pytest.raises(ReleasePolicyError, match="JETFIRE_ALLOW_EXPERIMENTAL_GRAPH_CPU_TOPK"):
        validate_release_environment()
    clean_env.delenv("JETFIRE_ALLOW_EXPERIMENTAL_GRAPH_CPU_TOPK")
    clean_env.delenv("JETFIRE_GRAPH_GPU_WAIT_CPU_TOPK")
    clean_env.setenv("JETFIRE_RELEASE_STAGEB_CANDIDATE", "int4-x")
    with pytest.raises(ReleasePolicyError, match="JETFIRE_RELEASE_STAGEB_CANDIDATE"):
        validate_release_environment()
    clean_env.delenv("JETFIRE_RELEASE_STAGEB_CANDIDATE")
    # prefill chunk sizes: uniform, or exactly a named profile
    clean_env.setenv("JETFIRE_MLP_CHUNK_TOKENS", "1024")
    clean_env.setenv("JETFIRE_EMBED_CHUNK_TOKENS", "2048")
    with pytest.raises(ReleasePolicyError, match="inconsistent prefill chunk envs"):
        validate_release_environment()
    clean_env.setenv("JETFIRE_EMBED_CHUNK_TOKENS", "1024")
    validate_release_environment()
    clean_env.setenv("JETFIRE_PREFILL_PARTITION_PROFILE", "default")
    with pytest.raises(ReleasePolicyError, match="does not match release prefill partition profile"):
        validate_release_environment()
    for name in ("JETFIRE_EMBED_CHUNK_TOKENS", "JETFIRE_MLP_CHUNK_TOKENS", "JETFIRE_ATTN_O_PROJ_CHUNK_TOKENS",
                 "JETFIRE_PREFILL_ATTN_CHUNK_TOKENS", "JETFIRE_PREFILL_QKV_CHUNK_TOKENS"):
        clean_env.setenv(name, "2048")
    validate_release_environment()
    assert "JETFIRE_DEBUG_APPROX_ONLY" in EXPERIMENTAL_RELEASE_ENV

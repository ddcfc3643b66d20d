"""Release kernel plan and environment validation (`jetfire_vllm/adapter/release_policy.py:377-568`, pinned by
`tests/test_release_policy.py:12-52` of the reference).

Given a quantisation mode, group size, correction width and the largest captured batch, `plan_release_graph`
names exactly one Stage A / Stage B kernel family or raises; nothing falls through to another path.  The family
names are the reference's; `ReleaseKernelPlan.operators()` maps them to this library's operators
(`jetfire_amd.ops`).  `validate_release_environment` refuses the experimental environment switches while
`JETFIRE_RELEASE_GRAPH_POLICY=1`.  Standard library only."""
from __future__ import annotations

import os
from dataclasses import dataclass, field

from .config import SCHEMES

RELEASE_POLICY_ENV = "JETFIRE_RELEASE_GRAPH_POLICY"
RELEASE_REQUIRE_READY_ENV = "JETFIRE_RELEASE_REQUIRE_READY"
RELEASE_STAGEB_CANDIDATE_ENV = "JETFIRE_RELEASE_STAGEB_CANDIDATE"
RELEASE_ACCURACY_ABLATION_ENV = "JETFIRE_RELEASE_ACCURACY_ABLATION"
PREFILL_PARTITION_PROFILE_ENV = "JETFIRE_PREFILL_PARTITION_PROFILE"

RELEASE_HEAD_DIM = 128
RELEASE_BLOCK_SIZE = 16
RELEASE_GROUP_SIZES = (64, 128)
RELEASE_TOP_K = tuple(32 << i for i in range(9))                       # 32 ... 8192
RELEASE_MODES = ("SymInt3K_SymInt2V", "SymInt4K_SymInt4V") + tuple(
    f"SymInt{k}K_SymInt{v}V" for k, v in ((4, 3), (4, 2), (3, 4), (3, 3), (2, 4), (2, 3), (2, 2)))
RELEASE_STAGEB_CANDIDATES = ("", "int2-v2", "int2-wvs2")
INT8TC_TOP_K = tuple(k for k in RELEASE_TOP_K if k >= 64)

# Switches that change which kernels or which synchronisation a decode step uses.  Under the release policy a
# switch may only be set to the value listed for it here (None: it may not be set at all).
_KNOBS: dict[str, str | None] = {name: None for name in (
    "JETFIRE_USE_FUSED_ATTN_TOPK", "JETFIRE_FUSED_KERNEL", "JETFIRE_INT8TC_QK_FUSED_TOPK",
    "JETFIRE_INT8TC_QK_GROUP_FUSED_TOPK", "JETFIRE_ALLOW_EXPERIMENTAL_QK_TOPK", "JETFIRE_FUSED_SOFTMAX_V",
    "JETFIRE_WVS_VARIANT", "JETFIRE_INT4_SVS_VARIANT", "JETFIRE_INT4_SVS", "JETFIRE_ALLOW_UNSTABLE_INT2_STAGEB",
    "JETFIRE_GRAPH_INLINE_CPU_TOPK", "JETFIRE_GRAPH_SYNC_CPU_TOPK", "JETFIRE_ALLOW_EXPERIMENTAL_GRAPH_CPU_TOPK",
    "JETFIRE_GRAPH_STAGEB_INPLACE", "JETFIRE_USE_BLEND_KERNEL", "JETFIRE_DEBUG_CPU_TOPK_ONLY",
    "JETFIRE_DEBUG_APPROX_ONLY", "JETFIRE_DEBUG_CORRECTION_MODE", "JETFIRE_RELEASE_RESIDUAL_SCALE",
    "JETFIRE_DEBUG_RESIDUAL_SCALE")}
_KNOBS.update({
    "JETFIRE_USE_PERSISTENT_WORKER": "0", "JETFIRE_FUSED_JOIN_BLEND": "0", "JETFIRE_USE_INT8_TC": "1",
    "JETFIRE_USE_CUSTOM_BACKEND": "1", "JETFIRE_CPU_CORRECTION": "1", "JETFIRE_DECODE_CPU_ATTN": "1",
    "JETFIRE_SKIP_NATIVE_KV": "1", "JETFIRE_SYNC_CPU_ATTN": "0", "JETFIRE_DISABLE_ASYNC_SCHEDULING": "1",
    "JETFIRE_USE_INT8_TC_SV": "0", "JETFIRE_GRAPH_DEVICE_SIGNAL_CPU_TOPK": "0", "JETFIRE_GRAPH_GPU_WAIT_CPU_TOPK": "0",
    "JETFIRE_GRAPH_HOST_JOIN_CPU_TOPK": "1", "JETFIRE_FUSED_QUANT": "1", "JETFIRE_FUSED_QUANT_WRITE": "1",
    "JETFIRE_FUSED_KV_QUANT_WRITE": "1", "JETFIRE_PREFILL_PIPELINE": "1", "JETFIRE_PREFILL_STREAM_TOKENS": "0",
    "JETFIRE_PIPELINE_MIN_TOKENS": "64", "JETFIRE_SHADOW": "1", "JETFIRE_SHADOW_DEVICE": "cpu",
    "JETFIRE_SHADOW_DTYPE": "bf16", "JETFIRE_ZERO_INIT_CACHE": "0", "JETFIRE_SHADOW_DIRECT_D2H": "0"})
EXPERIMENTAL_RELEASE_ENV = tuple(_KNOBS)
CANONICAL_RELEASE_ENV = {k: (v,) for k, v in _KNOBS.items() if v is not None}
# an A/B run of the graph-mode synchronisation may set these while JETFIRE_ALLOW_EXPERIMENTAL_GRAPH_CPU_TOPK=1
_GRAPH_SYNC_AB = frozenset(("JETFIRE_GRAPH_DEVICE_SIGNAL_CPU_TOPK", "JETFIRE_GRAPH_GPU_WAIT_CPU_TOPK",
                            "JETFIRE_GRAPH_HOST_JOIN_CPU_TOPK", "JETFIRE_GRAPH_INLINE_CPU_TOPK",
                            "JETFIRE_GRAPH_SYNC_CPU_TOPK", "JETFIRE_USE_BLEND_KERNEL", "JETFIRE_FUSED_JOIN_BLEND"))

# prefill chunk sizes (tokens) per partition profile, in the order of RELEASE_PREFILL_CHUNK_ENV; every profile but
# "default" is stated for hidden 8192 / local intermediate 14336 and rescaled to the model's shape
RELEASE_PREFILL_CHUNK_ENV = ("JETFIRE_EMBED_CHUNK_TOKENS", "JETFIRE_MLP_CHUNK_TOKENS", "JETFIRE_ATTN_O_PROJ_CHUNK_TOKENS",
                             "JETFIRE_PREFILL_ATTN_CHUNK_TOKENS", "JETFIRE_PREFILL_QKV_CHUNK_TOKENS")
RELEASE_PREFILL_PARTITION_SHAPE_ENV = ("JETFIRE_PREFILL_PARTITION_HIDDEN", "JETFIRE_PREFILL_PARTITION_LOCAL_INTERMEDIATE",
                                       "JETFIRE_PREFILL_PARTITION_ATTN_ELEMS")
RELEASE_PREFILL_PARTITION_PROFILES = {
    "default": (2048, 2048, 2048, 2048, 2048), "perf_12g": (4096, 4096, 2048, 2048, 2048),
    "relaxed_10g5": (4096, 3072, 1536, 1536, 1536), "balanced_9g": (2048, 2048, 1024, 1024, 1024),
    "balanced_7g5": (2048, 1536, 768, 768, 768), "tight_6g25": (2048, 1024, 512, 512, 512),
    "tight_5g5": (1024, 512, 480, 480, 480), "tight_5g25": (1024, 512, 384, 384, 384),
    "floor_0g": (1024, 384, 256, 256, 256)}
_PARTITION_REFERENCE_SHAPE = (8192, 28672 // 2, 8192)     # hidden, local intermediate (TP 2), attention elements
_CHUNK_SCALES_WITH = (0, 1, 2, 2, 2)                      # which shape entry rescales each chunk size


class ReleasePolicyError(ValueError):
    """The requested configuration is outside the release contract."""


# Stage family -> operator of jetfire_amd.ops that implements it
STAGE_OPERATORS = {
    "qk_int8tc_stats": "int8tc_qk_scores_topk_stats",
    "qk_int2_split_topk": "int2_qk_scores_topk", "qk_int3_split_topk": "int3_qk_scores_topk",
    "qk_int4_split_topk": "int4_qk_scores_topk_stats",
    "sv_int8tc_reg_stats": "int8tc_softmax_v_with_pre_corr_reg_stats",
    "sv_int4_wvs2_scores": "int4_softmax_v_with_pre_corr_wvs2_scores",
    "sv_int2_wvs2": "int2_softmax_v_with_pre_corr_wvs2", "sv_int3_wvs2": "int3_softmax_v_with_pre_corr_wvs2",
    "sv_int4_wvs2": "int4_softmax_v_with_pre_corr_wvs2", "sv_int2_v2": "int2_softmax_v_with_pre_corr",
}


@dataclass(frozen=True)
class ReleaseKernelPlan:
    mode: str
    k_nbits: int
    v_nbits: int
    group_size: int
    top_k: int
    head_dim: int
    num_quant_groups: int
    stage_a: str
    stage_b: str
    correction_sync: str
    graph_scope: str
    promotion_state: str
    release_ready: bool
    blockers: tuple = field(default=())
    notes: tuple = field(default=())

    def assert_ready(self) -> None:
        if self.release_ready:
            return
        why = "; ".join(self.blockers) or "unknown blocker"
        raise ReleasePolicyError(f"release graph plan is not ready for {self.mode} g{self.group_size} "
                                 f"top_k={self.top_k}: {why}")

    def operators(self) -> tuple:
        """(Stage A, Stage B) operator names of `jetfire_amd.ops` (None where this library has no such kernel)."""
        return STAGE_OPERATORS.get(self.stage_a), STAGE_OPERATORS.get(self.stage_b)


def release_policy_enabled() -> bool:
    return os.environ.get(RELEASE_POLICY_ENV, "0") == "1"


def release_require_ready() -> bool:
    return os.environ.get(RELEASE_REQUIRE_READY_ENV, "0") == "1"


def release_stageb_candidate() -> str:
    return os.environ.get(RELEASE_STAGEB_CANDIDATE_ENV, "").strip()


def _member(name: str, value, allowed) -> None:
    if value not in tuple(allowed):
        raise ReleasePolicyError(f"{name}={value!r} is not in release matrix {tuple(allowed)!r}")


_INT2_NOTE = ("INT2 V wvs2 is promoted for the single-GPU release graph path; TP=2 long-context performance remains "
              "validation-only until the full graph-level chunk-size sweep is complete.")


def _stage_a(k_nbits: int, groups: int, top_k: int) -> tuple:
    if k_nbits == 4 and groups == 1 and top_k in INT8TC_TOP_K:
        return "qk_int8tc_stats", ()
    notes = ()
    if k_nbits == 4 and groups != 1:
        notes = ("K4 g64 uses split QK because current INT8TC QK expects one scale group per head.",)
    return f"qk_int{k_nbits}_split_topk", notes


def _stage_b(v_nbits: int, groups: int, group_size: int, head_dim: int, batch: int, stage_a: str, candidate: str) -> tuple:
    """-> (family, promotion state, ready, blockers, notes)"""
    if candidate:
        _member(RELEASE_STAGEB_CANDIDATE_ENV, candidate, RELEASE_STAGEB_CANDIDATES)
        if v_nbits != 2:
            raise ReleasePolicyError(f"{RELEASE_STAGEB_CANDIDATE_ENV}={candidate!r} only applies to INT2 V modes")
        if candidate == "int2-wvs2" and groups != 1:
            raise ReleasePolicyError("INT2 wvs2 Stage-B requires one V scale group per head "
                                     f"(group_size={group_size}, head_dim={head_dim})")
        blocker = f"candidate Stage-B override {candidate!r} requires graph-level promotion evidence before release."
        return {"int2-v2": "sv_int2_v2", "int2-wvs2": "sv_int2_wvs2"}[candidate], "candidate", False, (blocker,), ()
    if groups == 1:
        if v_nbits == 4:
            # only the int8 Stage A hands over the softmax statistics the int8-weight Stage B consumes
            batched = stage_a == "qk_int8tc_stats" and batch > 1
            return ("sv_int8tc_reg_stats" if batched else "sv_int4_wvs2_scores"), "ready", True, (), ()
        return f"sv_int{v_nbits}_wvs2", "ready", True, (), ((_INT2_NOTE,) if v_nbits == 2 else ())
    if groups == 2:
        notes = ("multi-group wvs2 Stage-B is promoted for group_size=64.",) + ((_INT2_NOTE,) if v_nbits == 2 else ())
        return f"sv_int{v_nbits}_wvs2", "ready", True, (), notes
    blockers = (("INT2 V Stage-B for this shape has no promoted release kernel.",) if v_nbits == 2 else ()) + (
        "multi-group Stage-B for group_size < head_dim currently uses split implementation instead of wvs2/WMMA "
        "release kernel.",)
    return f"sv_int{v_nbits}_split_multigroup", "candidate", False, blockers, ()


def plan_release_graph(*, mode: str, group_size: int, top_k: int, head_dim: int = RELEASE_HEAD_DIM,
                       num_query_heads: int = 32, num_kv_heads: int = 8, max_graph_batch: int = 1,
                       stageb_candidate: str | None = None, require_ready: bool = False) -> ReleaseKernelPlan:
    """The one kernel plan of a release matrix cell, or ReleasePolicyError.  `release_ready=False`: the cell runs,
    but on a path that is not promoted."""
    _member("mode", mode, RELEASE_MODES)
    scheme = SCHEMES.get(mode)
    if scheme is None:
        raise ReleasePolicyError(f"mode={mode!r} has no release kernel module")
    group_size, top_k, head_dim, batch = int(group_size), int(top_k), int(head_dim), int(max_graph_batch)
    _member("group_size", group_size, RELEASE_GROUP_SIZES)
    _member("top_k", top_k, RELEASE_TOP_K)
    if head_dim != RELEASE_HEAD_DIM:
        raise ReleasePolicyError(f"head_dim={head_dim} is not release head_dim=128")
    if head_dim % group_size:
        raise ReleasePolicyError(f"group_size={group_size} does not divide head_dim={head_dim}")
    if batch < 1:
        raise ReleasePolicyError("max_graph_batch must be >= 1")
    candidate = release_stageb_candidate() if stageb_candidate is None else stageb_candidate
    if candidate and require_ready:
        raise ReleasePolicyError(f"{RELEASE_STAGEB_CANDIDATE_ENV}={candidate!r} is only allowed when require_ready=False")
    groups = head_dim // group_size
    stage_a, notes_a = _stage_a(scheme.k_nbits, groups, top_k)
    stage_b, state, ready, blockers, notes_b = _stage_b(scheme.v_nbits, groups, group_size, head_dim, batch, stage_a, candidate)
    plan = ReleaseKernelPlan(mode=mode, k_nbits=scheme.k_nbits, v_nbits=scheme.v_nbits, group_size=group_size, top_k=top_k,
                             head_dim=head_dim, num_quant_groups=groups, stage_a=stage_a, stage_b=stage_b,
                             correction_sync="cpu_topk_host_join", graph_scope="decode_only", promotion_state=state,
                             release_ready=ready, blockers=blockers, notes=notes_a + notes_b)
    if require_ready:
        plan.assert_ready()
    return plan


def iter_release_matrix(*, modes=RELEASE_MODES, group_sizes=RELEASE_GROUP_SIZES, top_ks=RELEASE_TOP_K,
                        max_graph_batch: int = 1) -> list:
    return [plan_release_graph(mode=m, group_size=g, top_k=k, max_graph_batch=max_graph_batch)
            for m in modes for g in group_sizes for k in top_ks]


# ------------------------------------------------------------------ environment
def _positive_int(raw) -> int | None:
    try:
        value = int(raw)
    except (TypeError, ValueError):
        return None
    return value if value > 0 else None


def _partition_shape() -> tuple | None:
    shape = tuple(_positive_int(os.environ.get(name)) for name in RELEASE_PREFILL_PARTITION_SHAPE_ENV)
    return None if None in shape else shape


def _expected_chunks(profile: str) -> dict | None:
    base = RELEASE_PREFILL_PARTITION_PROFILES.get(profile)
    if base is None:
        return None
    if profile == "default":
        return dict(zip(RELEASE_PREFILL_CHUNK_ENV, base))
    shape = _partition_shape()
    if shape is None:
        return None

    def rescale(tokens: int, which: int) -> int:
        scaled = tokens * _PARTITION_REFERENCE_SHAPE[which] / shape[which]
        return 0 if scaled <= 0 else max(16, int(scaled // 16) * 16)

    return {name: rescale(tokens, which) for name, tokens, which in zip(RELEASE_PREFILL_CHUNK_ENV, base, _CHUNK_SCALES_WITH)}


def _knob_offenders() -> list:
    env = os.environ
    graph_ab = env.get("JETFIRE_ALLOW_EXPERIMENTAL_GRAPH_CPU_TOPK", "0") == "1"
    ablation = env.get(RELEASE_ACCURACY_ABLATION_ENV, "0") == "1"
    bad = []
    for name, canonical in _KNOBS.items():
        raw = env.get(name)
        if raw is None or (graph_ab and name in _GRAPH_SYNC_AB):
            continue
        if ablation and name == "JETFIRE_DEBUG_APPROX_ONLY" and raw == "1":
            continue        # a marked accuracy ablation may switch the correction off, and nothing else
        if canonical is not None and raw.lower() == canonical:
            continue
        bad.append(f"{name}={raw!r}")
    return bad


def _prefill_offenders() -> list:
    env = os.environ
    bad = []
    profile = env.get(PREFILL_PARTITION_PROFILE_ENV)
    known = profile in RELEASE_PREFILL_PARTITION_PROFILES
    if profile is not None and not known and profile != "user_uniform":
        bad.append(f"{PREFILL_PARTITION_PROFILE_ENV}={profile!r}")
    if known and profile != "default" and _partition_shape() is None:
        bad.append("invalid release prefill partition shape metadata: "
                   + ", ".join(f"{n}={env.get(n)!r}" for n in RELEASE_PREFILL_PARTITION_SHAPE_ENV))
    chunks = {}
    for name in RELEASE_PREFILL_CHUNK_ENV:
        raw = env.get(name)
        if raw is None:
            continue
        try:
            value = int(raw)
        except ValueError:
            value = -1
        if value < 0:
            bad.append(f"{name}={raw!r}")
        else:
            chunks[name] = value
    if profile is not None and not chunks:
        bad.append(f"{PREFILL_PARTITION_PROFILE_ENV}={profile!r}")
    if chunks and known:
        if chunks != _expected_chunks(profile):
            bad.append(f"{PREFILL_PARTITION_PROFILE_ENV}={profile!r} does not match release prefill partition profile: "
                       + ", ".join(f"{k}={chunks.get(k)!r}" for k in RELEASE_PREFILL_CHUNK_ENV))
    elif len(set(chunks.values())) > 1:
        bad.append("inconsistent prefill chunk envs: " + ", ".join(f"{k}={v!r}" for k, v in sorted(chunks.items())))
    return bad


def validate_release_environment() -> None:
    """While the release policy is on, refuse environment switches that would silently change the kernel path."""
    if not release_policy_enabled():
        return
    offenders = _knob_offenders() + _prefill_offenders()
    if offenders:
        raise ReleasePolicyError("release graph policy rejects experimental env knobs: " + ", ".join(sorted(offenders)))
    _member(RELEASE_STAGEB_CANDIDATE_ENV, release_stageb_candidate(), RELEASE_STAGEB_CANDIDATES)

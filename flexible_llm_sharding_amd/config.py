"""Model configuration (Llama family) read from an HF ``config.json``.

The reference builds the model shell from ``AutoConfig.from_pretrained``
(``/root/reference/utils.py:101``) and instantiates HF ``LlamaForCausalLM`` on
the meta device (``utils.py:111-113``).  We only need the architecture
numbers: the model itself is our own packed-weight implementation.
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, field
from typing import Optional

# Reference hard-codes the maximum sequence length (utils.py:14).
MAX_TOKEN_LEN = 4096


@dataclass
class ModelConfig:
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_attention_heads: int = 32
    num_key_value_heads: int = 32
    num_hidden_layers: int = 32
    vocab_size: int = 32000
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    max_position_embeddings: int = 4096
    tie_word_embeddings: bool = False
    attention_bias: bool = False        # q/k/v projection biases (Qwen2; Llama attention_bias)
    o_proj_bias: bool = False           # o_proj bias (Llama attention_bias=True)
    qk_norm: bool = False               # Qwen3: RMSNorm over head_dim on every q / k head, before RoPE
    # Mistral / Phi-3: every call's sequences must fit the window (checked per call by the runner)
    sliding_window: Optional[int] = None
    # RoPE frequency scaling (HF ``rope_scaling`` / v5 ``rope_parameters``): linear, llama3, yarn,
    # longrope (Phi-3)
    rope_scaling: Optional[dict] = None
    explicit_head_dim: Optional[int] = None   # HF ``head_dim`` when != hidden / heads (Mistral-Nemo)
    # sparse mixture-of-experts FFN (Mixtral, Qwen3-MoE): 0 = dense SwiGLU MLP.  Each token's
    # post-attention RMSNorm output goes to its top-k experts (router softmax in fp32, top-k,
    # renormalised when norm_topk_prob), each a SwiGLU MLP of moe_intermediate_size (Mixtral:
    # intermediate_size), and the weighted expert outputs are summed into the residual
    num_local_experts: int = 0
    num_experts_per_tok: int = 2
    moe_intermediate_size: Optional[int] = None
    norm_topk_prob: bool = True
    # Qwen2-MoE: a dense SwiGLU "shared expert" of this width on every token, scaled by
    # sigmoid(h . shared_expert_gate) and added to the routed experts' sum (0: none)
    shared_expert_intermediate_size: int = 0
    # Granite (HF GraniteModel / GraniteDecoderLayer / GraniteForCausalLM): token embeddings x
    # embedding_multiplier; each sub-layer output x residual_multiplier before the residual add;
    # attention scores x attention_multiplier (instead of head_dim^-1/2); logits / logits_scaling
    embedding_multiplier: float = 1.0
    residual_multiplier: float = 1.0
    attention_multiplier: Optional[float] = None
    logits_scaling: float = 1.0
    bos_token_id: int = 1
    eos_token_id: int = 2
    torch_dtype: str = "float16"
    model_type: str = "llama"
    architectures: list = field(default_factory=lambda: ["LlamaForCausalLM"])

    # ------------------------------------------------------------------ derived
    @property
    def head_dim(self) -> int:
        return self.explicit_head_dim or self.hidden_size // self.num_attention_heads

    @property
    def attn_scale(self) -> float:
        """Softmax scale of the attention scores (Granite: attention_multiplier)."""
        return self.attention_multiplier if self.attention_multiplier is not None else self.head_dim ** -0.5

    @property
    def is_moe(self) -> bool:
        return self.num_local_experts > 0

    @property
    def expert_intermediate(self) -> int:
        """Rows of one expert's gate (= up) projection (the dense MLP's for non-MoE models)."""
        return self.moe_intermediate_size or self.intermediate_size

    @property
    def fused_projections(self) -> bool:
        """Phi-3 checkpoints store ``qkv_proj`` ([q; k; v] rows) and ``gate_up_proj`` ([gate; up]
        rows) as single tensors: the same row order as the packed ``wqkv`` / ``wgu`` slots."""
        return self.model_type == "phi3"

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def qkv_size(self) -> int:
        return self.q_size + 2 * self.kv_size

    @property
    def num_layers_total(self) -> int:
        """embed + decoder layers + final norm + lm_head (reference utils.py:106-107)."""
        return self.num_hidden_layers + 3

    def layer_names(self) -> list:
        """Ordered layer list, identical to ``ShardedLlama.layer_names`` (utils.py:106-107)."""
        return (["model.embed_tokens"]
                + [f"model.layers.{i}" for i in range(self.num_hidden_layers)]
                + ["model.norm", "lm_head"])

    def decoder_layer_params(self) -> int:
        """Parameters stored per decoder layer (every expert of an MoE layer)."""
        return self._decoder_params(self.num_local_experts)

    def decoder_active_params(self) -> int:
        """Parameters one token multiplies per decoder layer (MoE: router + its top-k experts)."""
        return self._decoder_params(self.num_experts_per_tok) if self.is_moe else self.decoder_layer_params()

    def _decoder_params(self, experts: int) -> int:
        h = self.hidden_size
        n = h * self.qkv_size + self.q_size * h + 2 * h
        if self.is_moe:
            n += self.num_local_experts * h + experts * 3 * h * self.expert_intermediate
            n += 3 * h * self.shared_expert_intermediate_size + (h if self.shared_expert_intermediate_size else 0)
        else:
            n += 3 * h * self.intermediate_size
        return (n + (self.qkv_size if self.attention_bias else 0) + (h if self.o_proj_bias else 0)
                + (2 * self.head_dim if self.qk_norm else 0))

    def total_params(self) -> int:
        emb = self.vocab_size * self.hidden_size
        head = 0 if self.tie_word_embeddings else emb
        return emb + head + self.hidden_size + self.num_hidden_layers * self.decoder_layer_params()

    def validate(self) -> None:
        if self.explicit_head_dim is None and self.hidden_size % self.num_attention_heads:
            raise ValueError("hidden_size must be divisible by num_attention_heads")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ValueError("num_attention_heads must be a multiple of num_key_value_heads")
        if self.head_dim % 32:
            raise ValueError("head_dim must be a multiple of 32 (RoPE pair blocks of 16)")
        if self.is_moe and not 1 <= self.num_experts_per_tok <= min(self.num_local_experts, MAX_TOP_K):
            raise ValueError(f"num_experts_per_tok must be in 1..min(num_local_experts, {MAX_TOP_K})")
        if self.is_moe and self.residual_multiplier != 1.0:
            # the MoE combine kernel adds the experts' sum to the residual unscaled
            raise NotImplementedError("residual_multiplier with a mixture-of-experts MLP")
        if self.num_local_experts > MAX_EXPERTS:
            raise NotImplementedError(f"num_local_experts={self.num_local_experts} > {MAX_EXPERTS}")
        rs = self.rope_scaling
        if rs:
            kind = rs.get("rope_type", rs.get("type"))
            if kind not in ROPE_SCALING_TYPES:
                raise NotImplementedError(f"rope_scaling type {kind!r}: supported are {sorted(ROPE_SCALING_TYPES)}"
                                          " (dynamic NTK depends on each call's length: not supported)")
            if float(rs.get("factor") or 1.0) <= 0:
                raise ValueError(f"rope_scaling factor must be > 0: {rs}")
            if kind == "longrope":
                for key in ("short_factor", "long_factor"):
                    if len(rs.get(key) or ()) != self.head_dim // 2:
                        raise ValueError(f"longrope {key} must hold head_dim/2 = {self.head_dim // 2} values")
                orig = int(rs.get("original_max_position_embeddings") or self.max_position_embeddings)
                if orig < MAX_TOKEN_LEN:
                    # HF switches to long_factor once a sequence exceeds the original context;
                    # static tables are exact only while no sequence can
                    raise NotImplementedError(f"longrope with original_max_position_embeddings={orig} < the "
                                              f"{MAX_TOKEN_LEN}-token cap (length-dependent tables)")

    # ---------------------------------------------------------------------- io
    @classmethod
    def from_dict(cls, d: dict) -> "ModelConfig":
        kw = {}
        for f in cls.__dataclass_fields__:
            if f in d and d[f] is not None:
                kw[f] = d[f]
        if "num_key_value_heads" not in d or d.get("num_key_value_heads") is None:
            kw["num_key_value_heads"] = d.get("num_attention_heads", cls.num_attention_heads)
        rp = d.get("rope_parameters")          # transformers v5 form: {"rope_type", "rope_theta", ...}
        if isinstance(rp, dict):
            if "rope_theta" in rp:
                kw["rope_theta"] = rp["rope_theta"]
            if rp.get("rope_type", "default") != "default":
                kw["rope_scaling"] = {k: v for k, v in rp.items() if k != "rope_theta"}
        rs = kw.get("rope_scaling")
        if rs and rs.get("rope_type", rs.get("type")) == "default":
            kw.pop("rope_scaling")
        rs = kw.get("rope_scaling")
        if rs and rs.get("rope_type", rs.get("type")) in ("su", "longrope"):
            # Phi-3: "su" is the old name; the pretraining context sits at the config's top level
            rs = dict(rs, rope_type="longrope")
            rs.pop("type", None)
            if "original_max_position_embeddings" not in rs and d.get("original_max_position_embeddings"):
                rs["original_max_position_embeddings"] = d["original_max_position_embeddings"]
            kw["rope_scaling"] = rs
        for src in (d, rp if isinstance(rp, dict) else {}, rs or {}):
            if float(src.get("partial_rotary_factor", 1.0) or 1.0) != 1.0:
                raise NotImplementedError("partial_rotary_factor < 1 (RoPE on part of each head) is not supported")
        mt = d.get("model_type", "llama")
        if mt not in SUPPORTED_MODEL_TYPES:
            why = llama_like_rejection(d)
            if why:
                raise NotImplementedError(f"model_type={mt!r}: supported are {sorted(SUPPORTED_MODEL_TYPES)}, or a "
                                          f"Llama-structured config ({why})")
            # an unlisted family with the Llama block: run as Llama; every layer file must then hold
            # exactly the Llama tensors (models/layout.py check_layer_tensors), so a different block
            # structure fails at load instead of running wrong
            kw["model_type"] = mt
        if mt in ("qwen3_moe", "qwen2_moe"):
            kw["num_local_experts"] = int(d.get("num_experts") or d.get("num_local_experts") or 0)
            if mt == "qwen3_moe" and d.get("shared_expert_intermediate_size"):
                raise NotImplementedError("shared experts in a Qwen3-MoE config")
            if d.get("mlp_only_layers") or int(d.get("decoder_sparse_step", 1) or 1) != 1:
                raise NotImplementedError("dense layers between the MoE layers (mlp_only_layers / "
                                          "decoder_sparse_step) are not supported")
        if mt == "mixtral":
            kw["norm_topk_prob"] = True           # HF MixtralTopKRouter always renormalises
        elif mt in ("qwen3_moe", "qwen2_moe"):
            kw["norm_topk_prob"] = bool(d.get("norm_topk_prob", False))     # HF Qwen3MoeConfig default
        if d.get("mlp_bias"):
            raise NotImplementedError("mlp_bias=True is not supported")
        hdim = d.get("head_dim")
        if hdim is not None and hdim * d.get("num_attention_heads", cls.num_attention_heads) != d.get(
                "hidden_size", cls.hidden_size):
            kw["explicit_head_dim"] = int(hdim)
        if d.get("hidden_act", "silu") != "silu":
            raise NotImplementedError(f"hidden_act={d.get('hidden_act')!r} (SwiGLU/silu only)")
        if mt == "qwen2" or (mt == "qwen2_moe" and d.get("qkv_bias", d.get("attention_bias", True))):
            # HF Qwen2Attention / Qwen2MoeAttention (qkv_bias, default True): q/k/v Linear with
            # bias, o_proj without
            kw["attention_bias"], kw["o_proj_bias"] = True, False
        elif d.get("attention_bias"):
            kw["attention_bias"], kw["o_proj_bias"] = True, True
        if mt in ("qwen3", "qwen3_moe"):
            # HF Qwen3Attention: q_norm / k_norm (RMSNorm over head_dim) on every head before RoPE;
            # q/k/v/o biases only with attention_bias (off in every released Qwen3 config)
            kw["qk_norm"] = True
        # HF Phi3Model / Mixtral apply their sliding_window whenever it is set; Qwen2/3 only with
        # use_sliding_window
        if not d.get("use_sliding_window", mt in ("mistral", "phi3", "mixtral")):
            kw.pop("sliding_window", None)
        if isinstance(kw.get("eos_token_id"), list):
            kw["eos_token_id"] = kw["eos_token_id"][0]
        cfg = cls(**kw)
        cfg.validate()
        return cfg

    @classmethod
    def from_pretrained(cls, model_path: str) -> "ModelConfig":
        with open(os.path.join(model_path, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict:
        d = asdict(self)
        d["head_dim"] = self.head_dim
        return d

    def save(self, model_path: str) -> None:
        os.makedirs(model_path, exist_ok=True)
        d = asdict(self)
        d["head_dim"] = self.head_dim           # HF key (also read back by from_dict)
        if self.model_type in ("qwen3_moe", "qwen2_moe"):
            d["num_experts"] = self.num_local_experts          # the HF key of these families
        with open(os.path.join(model_path, "config.json"), "w") as f:
            json.dump(d, f, indent=2)


# Llama-structured causal LMs (model.embed_tokens / model.layers.N / model.norm / lm_head with
# q/k/v/o + gate/up/down + two RMSNorms per layer) -- what the reference's AutoModelForCausalLM
# path (utils.py:101-115) runs in practice.
SUPPORTED_MODEL_TYPES = {"llama", "mistral", "qwen2", "qwen3", "phi3", "mixtral", "qwen3_moe", "qwen2_moe",
                         "granite"}

# config keys of other families whose block differs from Llama's while its tensors may look the same
# (MiniCPM's embedding / depth scales, Gemma-2's soft-capping, DeepSeek's latent attention, Cohere's
# logit scale, parallel attention + MLP blocks, experts under other names)
_NON_LLAMA_KEYS = ("scale_emb", "scale_depth", "dim_model_base", "attn_logit_softcapping",
                   "final_logit_softcapping", "query_pre_attn_scalar", "kv_lora_rank", "q_lora_rank",
                   "logit_scale", "use_parallel_residual", "parallel_attn", "parallel_block", "n_routed_experts",
                   "num_experts", "num_local_experts", "moe_intermediate_size", "use_qk_norm", "qk_layernorm",
                   "layer_norm_eps", "norm_epsilon", "embedding_multiplier", "residual_multiplier")


def llama_like_rejection(d: dict) -> str:
    """'' when an unlisted model_type's config.json describes the Llama block (the fields Llama reads,
    SwiGLU, RMSNorm, full RoPE, none of the keys that change the block), else the reason not."""
    need = ("hidden_size", "intermediate_size", "num_attention_heads", "num_hidden_layers", "vocab_size",
            "rms_norm_eps")
    missing = [k for k in need if k not in d]
    if missing:
        return f"missing {', '.join(missing)}"
    # (1 / 0 / false are the neutral values: this framework's own config.json lists every field)
    extra = [k for k in _NON_LLAMA_KEYS if d.get(k) not in (None, False, 0, 1)]
    if extra:
        return f"{', '.join(extra)} change the block"
    if d.get("hidden_act", "silu") != "silu":
        return f"hidden_act={d.get('hidden_act')!r}"
    return ""
# MoE limits of the routing kernels (csrc/kernels/moe.hip): experts per layer, experts per token
MAX_EXPERTS = 256
MAX_TOP_K = 8
# static RoPE scalings: they only change the cos/sin tables (models/llama.py rope_inv_freq)
ROPE_SCALING_TYPES = {"linear", "llama3", "yarn", "longrope"}

# Standard HF configs.
PRESETS = {
    "llama2-7b": dict(hidden_size=4096, intermediate_size=11008, num_attention_heads=32,
                      num_key_value_heads=32, num_hidden_layers=32),
    "llama2-13b": dict(hidden_size=5120, intermediate_size=13824, num_attention_heads=40,
                       num_key_value_heads=40, num_hidden_layers=40),
    "llama2-70b": dict(hidden_size=8192, intermediate_size=28672, num_attention_heads=64,
                       num_key_value_heads=8, num_hidden_layers=80),
    "mistral-7b": dict(hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
                       num_key_value_heads=8, num_hidden_layers=32, rope_theta=1e6,
                       model_type="mistral", architectures=["MistralForCausalLM"]),
    "qwen2-7b": dict(hidden_size=3584, intermediate_size=18944, num_attention_heads=28,
                     num_key_value_heads=4, num_hidden_layers=28, vocab_size=152064, rope_theta=1e6,
                     rms_norm_eps=1e-6, attention_bias=True, model_type="qwen2",
                     architectures=["Qwen2ForCausalLM"]),
    # tiny configs for tests (GQA 2:1, head_dim 64)
    "tiny": dict(hidden_size=256, intermediate_size=512, num_attention_heads=4,
                 num_key_value_heads=2, num_hidden_layers=2, vocab_size=512,
                 max_position_embeddings=4096),
    "tiny-qwen2": dict(hidden_size=256, intermediate_size=512, num_attention_heads=4,
                       num_key_value_heads=2, num_hidden_layers=2, vocab_size=512, rope_theta=1e6,
                       rms_norm_eps=1e-6, attention_bias=True, model_type="qwen2",
                       architectures=["Qwen2ForCausalLM"]),
    # Qwen3 dense: per-head q/k RMSNorm, explicit head_dim 128 (hidden 4096 = 32 x 128 here)
    "qwen3-8b": dict(hidden_size=4096, intermediate_size=12288, num_attention_heads=32,
                     num_key_value_heads=8, num_hidden_layers=36, vocab_size=151936, rope_theta=1e6,
                     rms_norm_eps=1e-6, qk_norm=True, explicit_head_dim=128, max_position_embeddings=40960,
                     model_type="qwen3", architectures=["Qwen3ForCausalLM"]),
    "tiny-qwen3": dict(hidden_size=256, intermediate_size=512, num_attention_heads=4,
                       num_key_value_heads=2, num_hidden_layers=2, vocab_size=512, rope_theta=1e6,
                       rms_norm_eps=1e-6, qk_norm=True, explicit_head_dim=128, model_type="qwen3",
                       architectures=["Qwen3ForCausalLM"]),
    # Phi-3 family: fused qkv_proj / gate_up_proj tensors; Phi-3-medium-4k (sliding window 2047)
    # and Phi-4 (14B, 100k vocab) have head_dim 128
    "phi3-medium": dict(hidden_size=5120, intermediate_size=17920, num_attention_heads=40,
                        num_key_value_heads=10, num_hidden_layers=40, vocab_size=32064, sliding_window=2047,
                        eos_token_id=32000, model_type="phi3", architectures=["Phi3ForCausalLM"]),
    "phi4": dict(hidden_size=5120, intermediate_size=17920, num_attention_heads=40, num_key_value_heads=10,
                 num_hidden_layers=40, vocab_size=100352, rope_theta=250000.0, max_position_embeddings=16384,
                 bos_token_id=100257, eos_token_id=100265, model_type="phi3", architectures=["Phi3ForCausalLM"]),
    # Phi-3-mini-4k: multi-head attention with head_dim 96 (unfused RoPE pass, 12-chunk LDS rows)
    "phi3-mini": dict(hidden_size=3072, intermediate_size=8192, num_attention_heads=32, num_key_value_heads=32,
                      num_hidden_layers=32, vocab_size=32064, sliding_window=2047, eos_token_id=32000,
                      model_type="phi3", architectures=["Phi3ForCausalLM"]),
    "tiny-phi3-mini": dict(hidden_size=384, intermediate_size=768, num_attention_heads=4, num_key_value_heads=4,
                           num_hidden_layers=2, vocab_size=512, model_type="phi3",
                           architectures=["Phi3ForCausalLM"]),
    # tiny Phi-3-128k-style config: longrope short/long factors, attention factor from 131072 / 4096
    "tiny-phi3": dict(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=2, vocab_size=512, max_position_embeddings=131072,
                      rope_scaling={"rope_type": "longrope", "original_max_position_embeddings": 4096,
                                    "short_factor": [1.0 + 0.05 * i for i in range(32)],
                                    "long_factor": [2.0 + 0.5 * i for i in range(32)]},
                      model_type="phi3", architectures=["Phi3ForCausalLM"]),
    # Llama-3.1 geometry (GQA 8:1, 128k vocab, llama3 RoPE scaling)
    "llama3.1-8b": dict(hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
                        num_key_value_heads=8, num_hidden_layers=32, vocab_size=128256, rope_theta=500000.0,
                        max_position_embeddings=131072, bos_token_id=128000, eos_token_id=128001,
                        rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                      "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}),
    # sparse MoE: Mixtral-8x7B (8 experts, top-2, 32k vocab) and Qwen3-30B-A3B (128 experts of
    # 768 rows, top-8, q/k norm); tiny variants keep every GEMM on the grouped MFMA path
    "mixtral-8x7b": dict(hidden_size=4096, intermediate_size=14336, num_attention_heads=32, num_key_value_heads=8,
                         num_hidden_layers=32, vocab_size=32000, rope_theta=1e6, max_position_embeddings=32768,
                         num_local_experts=8, num_experts_per_tok=2, model_type="mixtral",
                         architectures=["MixtralForCausalLM"]),
    "qwen3-30b-a3b": dict(hidden_size=2048, intermediate_size=6144, num_attention_heads=32, num_key_value_heads=4,
                          num_hidden_layers=48, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6, qk_norm=True,
                          explicit_head_dim=128, max_position_embeddings=40960, num_local_experts=128,
                          num_experts_per_tok=8, moe_intermediate_size=768, norm_topk_prob=True,
                          model_type="qwen3_moe", architectures=["Qwen3MoeForCausalLM"]),
    "tiny-mixtral": dict(hidden_size=256, intermediate_size=256, num_attention_heads=4, num_key_value_heads=2,
                         num_hidden_layers=2, vocab_size=512, rope_theta=1e6, num_local_experts=4,
                         num_experts_per_tok=2, model_type="mixtral", architectures=["MixtralForCausalLM"]),
    "tiny-qwen3-moe": dict(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                           num_hidden_layers=2, vocab_size=512, rope_theta=1e6, rms_norm_eps=1e-6, qk_norm=True,
                           explicit_head_dim=128, num_local_experts=8, num_experts_per_tok=3,
                           moe_intermediate_size=128, norm_topk_prob=False, model_type="qwen3_moe",
                           architectures=["Qwen3MoeForCausalLM"]),
    # Qwen1.5-MoE-A2.7B: 60 routed experts (top 4, not renormalised) + a gated shared expert
    "qwen1.5-moe-a2.7b": dict(hidden_size=2048, intermediate_size=5632, num_attention_heads=16,
                              num_key_value_heads=16, num_hidden_layers=24, vocab_size=151936, rope_theta=1e6,
                              rms_norm_eps=1e-6, attention_bias=True, num_local_experts=60, num_experts_per_tok=4,
                              moe_intermediate_size=1408, shared_expert_intermediate_size=5632,
                              norm_topk_prob=False, bos_token_id=151643, eos_token_id=151643,
                              model_type="qwen2_moe", architectures=["Qwen2MoeForCausalLM"]),
    "tiny-qwen2-moe": dict(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                           num_hidden_layers=2, vocab_size=512, rope_theta=1e6, rms_norm_eps=1e-6,
                           attention_bias=True, num_local_experts=8, num_experts_per_tok=3,
                           moe_intermediate_size=128, shared_expert_intermediate_size=256, norm_topk_prob=False,
                           model_type="qwen2_moe", architectures=["Qwen2MoeForCausalLM"]),
    # Granite-3.0-8B: Llama geometry with the four Granite scalars and a tied 49k head
    "granite-3-8b": dict(hidden_size=4096, intermediate_size=12800, num_attention_heads=32, num_key_value_heads=8,
                         num_hidden_layers=40, vocab_size=49155, rope_theta=10000.0, tie_word_embeddings=True,
                         embedding_multiplier=12.0, residual_multiplier=0.22, attention_multiplier=0.0078125,
                         logits_scaling=16.0, bos_token_id=0, eos_token_id=0, model_type="granite",
                         architectures=["GraniteForCausalLM"]),
    "tiny-granite": dict(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                         num_hidden_layers=2, vocab_size=512, embedding_multiplier=6.0, residual_multiplier=0.4,
                         attention_multiplier=0.09, logits_scaling=3.0, model_type="granite",
                         architectures=["GraniteForCausalLM"]),
    "small": dict(hidden_size=1024, intermediate_size=2816, num_attention_heads=8,
                  num_key_value_heads=2, num_hidden_layers=4, vocab_size=32000),
}


def preset(name: str, **overrides) -> ModelConfig:
    if name not in PRESETS:
        raise KeyError(f"unknown preset {name!r}; choose from {sorted(PRESETS)}")
    d = dict(PRESETS[name])
    d.update(overrides)
    cfg = ModelConfig(**d)
    cfg.validate()
    return cfg


def resolve_dtype(name: Optional[str]):
    import torch
    table = {"float16": torch.float16, "fp16": torch.float16, "half": torch.float16,
             "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
             "float32": torch.float32, "fp32": torch.float32}
    if name is None:
        return torch.float16
    if name not in table:
        raise ValueError(f"unsupported dtype {name}")
    return table[name]


# ----------------------------------------------------------------------------- hybrid stacks
# A second kind of model: a stack whose layers differ (softmax attention over a chunk of the
# sequence, gated linear recurrences, state-space layers), each with its own sizes, served step by
# step from a per-request state (runtime/seq_state.py) instead of the (prefix, suffixes) scoring
# pass.  config.json names it with "architecture".

@dataclass
class HybridLayer:
    """One layer of a hybrid stack: its mixer ``type`` and sizes, and its feed-forward (or None)."""
    type: str                  # attention | rglru | mamba2
    mixer: dict
    mlp: Optional[dict]

    @property
    def ff_kind(self) -> str:
        return "none" if self.mlp is None else self.mlp["kind"]


MIXER_TYPES = ("attention", "rglru", "mamba2")


@dataclass
class KagolixConfig:
    """Kagolix: sandwich-normed (group RMS norm before and after each sublayer) hybrid decoder.
    Everything is read from config.json: ``width``, ``vocab``, ``norm`` {eps, groups},
    ``logit_softcap``, and ``layers`` (per layer ``type``, ``mixer`` sizes, ``mlp``)."""
    width: int
    vocab: int
    norm_eps: float
    norm_groups: int
    logit_softcap: float
    layers: list
    family = "kagolix"
    model_type = "kagolix"
    is_moe = False              # (the dense-family switches of the engine: off)
    sliding_window = None
    tie_word_embeddings = False

    # names the engine shares with the dense family
    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def num_layers_total(self) -> int:
        return len(self.layers) + 3

    def layer_names(self) -> list:
        """Checkpoint prefixes, in execution order: the image of each is one weight slot."""
        return ["embed"] + [f"l{i}" for i in range(len(self.layers))] + ["final.norm", "head"]

    def layer(self, name: str) -> HybridLayer:
        return self.layers[int(name[1:])]

    def validate(self) -> None:
        D = self.width
        if D % self.norm_groups:
            raise ValueError("width must be divisible by norm.groups")
        for i, l in enumerate(self.layers):
            m = l.mixer
            if l.type not in MIXER_TYPES:
                raise NotImplementedError(f"layer {i}: mixer type {l.type!r}")
            if l.type == "attention":
                if m["heads"] % m["kv_heads"]:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                if int(m["mask"]["size"]) < 1:
                    raise ValueError(f"layer {i}: mask.size must be >= 1")
            elif l.type == "rglru":
                if m["width"] % m["blocks"]:
                    raise ValueError(f"layer {i}: width must be divisible by blocks")
            elif l.type == "mamba2":
                if m["heads"] % m["groups"] or (m["heads"] * m["vdim"]) % m["norm_groups"]:
                    raise ValueError(f"layer {i}: heads / groups / norm_groups do not divide")
                if m["state"] > 256:
                    raise NotImplementedError(f"layer {i}: state={m['state']} > 256")
            if l.mlp is not None:
                if l.mlp["kind"] not in ("dense", "moe"):
                    raise NotImplementedError(f"layer {i}: mlp kind {l.mlp['kind']!r}")
                if l.mlp["kind"] == "moe":
                    r = l.mlp["router"]
                    # (the routing kernel of csrc/kernels/seq keeps up to 16 choices per token)
                    if not 1 <= r["top"] <= min(r["experts"], 16) or r["experts"] > 1024:
                        raise NotImplementedError(f"layer {i}: router {r}")

    @classmethod
    def from_dict(cls, d: dict) -> "KagolixConfig":
        layers = [HybridLayer(l["type"], dict(l["mixer"]), None if l.get("mlp") is None else dict(l["mlp"]))
                  for l in d["layers"]]
        cfg = cls(int(d["width"]), int(d["vocab"]), float(d["norm"]["eps"]), int(d["norm"]["groups"]),
                  float(d["logit_softcap"]), layers)
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": "Kagolix", "width": self.width, "vocab": self.vocab,
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "logit_softcap": self.logit_softcap,
                "layers": [{"type": l.type, "mixer": l.mixer, "mlp": l.mlp} for l in self.layers]}

    def save(self, model_path: str) -> None:
        os.makedirs(model_path, exist_ok=True)
        with open(os.path.join(model_path, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=1)

    def total_params(self) -> int:
        from .models.layout import layer_layout_of
        return sum(sum(s.numel for s in layer_layout_of(self, n).slots) for n in self.layer_names())


SISAVIK_MIXERS = ("latent_attention", "parallel")


@dataclass
class SisavikConfig:
    """Sisavik: a hybrid decoder whose sublayers read the residual stream through a short causal
    convolution (``canon.taps``) and whose outputs are RMS-normed (weight stored around zero) before
    they join it.  Mixers: latent attention (keys and values made from a cached low-rank latent plus
    one rotated key part, sliding window, optionally reading another layer's latent: ``kv_from``) and
    a parallel pair (sigmoid-weighted sliding-window attention with kept first tokens beside a
    generalized delta-rule recurrence).  Everything is read from config.json: ``width``, ``vocab``,
    ``norm.eps``, ``canon.taps`` and ``layers`` (per layer ``type``, ``mixer`` sizes, ``mlp``)."""
    width: int
    vocab: int
    norm_eps: float
    canon_taps: int
    layers: list
    family = "sisavik"
    model_type = "sisavik"
    is_moe = False
    sliding_window = None
    tie_word_embeddings = False

    hidden_size = KagolixConfig.hidden_size
    vocab_size = KagolixConfig.vocab_size
    num_hidden_layers = KagolixConfig.num_hidden_layers
    num_layers_total = KagolixConfig.num_layers_total
    layer_names = KagolixConfig.layer_names
    layer = KagolixConfig.layer
    save = KagolixConfig.save
    total_params = KagolixConfig.total_params

    def kv_owner(self, i: int) -> int:
        """The layer whose cached latent layer ``i`` reads (itself unless it names ``kv_from``)."""
        j = self.layers[i].mixer.get("kv_from")
        return i if j is None else int(j)

    def validate(self) -> None:
        if self.canon_taps < 1:
            raise ValueError("canon.taps must be >= 1")
        for i, l in enumerate(self.layers):
            m = l.mixer
            if l.type not in SISAVIK_MIXERS:
                raise NotImplementedError(f"layer {i}: mixer type {l.type!r}")
            if l.type == "latent_attention":
                if int(m["rot"]["dims"]) != int(m["rot_dim"]) or int(m["rot_dim"]) % 2:
                    raise ValueError(f"layer {i}: the rotated key part is rot_dim wide, an even number")
                if int(m["mask"]["size"]) < 1:
                    raise ValueError(f"layer {i}: mask.size must be >= 1")
                if int(m["kv_rank"]) > 512 or int(m["kv_rank"]) + int(m["rot_dim"]) > 1024 or int(m["rot_dim"]) > 512:
                    # (the paged attention kernel of csrc/kernels/seq: a latent row is its key and its value)
                    raise NotImplementedError(f"layer {i}: kv_rank {m['kv_rank']} > 512")
                j = m.get("kv_from")
                if j is not None:
                    o = self.layers[int(j)] if 0 <= int(j) < i else None
                    if o is None or o.type != "latent_attention" or o.mixer.get("kv_from") is not None:
                        raise ValueError(f"layer {i}: kv_from must name an earlier latent attention layer with a latent of its own")
                    if any(o.mixer[k] != m[k] for k in ("kv_rank", "rot_dim")) or o.mixer["rot"] != m["rot"]:
                        raise ValueError(f"layer {i}: kv_rank, rot_dim and rotation must equal layer {j}'s")
            else:
                a, r = m["left"], m["right"]
                if a["heads"] % a["kv_heads"]:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                if a["vdim"] != a["dim"]:
                    raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
                if int(a["rot"]["dims"]) > a["dim"] or int(a["rot"]["dims"]) % 2:
                    raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
                if int(a["mask"]["size"]) < 1 or int(a["mask"].get("keep_first", 0)) < 0:
                    raise ValueError(f"layer {i}: mask {a['mask']}")
                if a["dim"] > 512:
                    raise NotImplementedError(f"layer {i}: attention head size {a['dim']} > 512")
                if not 1 <= r["dim"] <= 128:
                    # (the recurrence kernel of csrc/kernels/seq keeps a head's state in one block's registers)
                    raise NotImplementedError(f"layer {i}: delta-rule head size {r['dim']} > 128")
            if l.mlp is not None and l.mlp["kind"] != "dense":
                raise NotImplementedError(f"layer {i}: mlp kind {l.mlp['kind']!r}")

    @classmethod
    def from_dict(cls, d: dict, model_path: Optional[str] = None) -> "SisavikConfig":
        """``model_path``: the rank of the decay's two-layer map is no key of config.json; where a layer
        does not name it (``right.decay_rank``), the checkpoint's tensor shapes give it."""
        layers = [HybridLayer(l["type"], json.loads(json.dumps(l["mixer"])), None if l.get("mlp") is None else dict(l["mlp"]))
                  for l in d["layers"]]
        shapes = None
        for i, l in enumerate(layers):
            if l.type == "parallel" and "decay_rank" not in l.mixer.get("right", {}):
                if shapes is None:
                    if model_path is None:
                        raise ValueError(f"layer {i}: right.decay_rank is neither given nor readable from a checkpoint")
                    from .utils.safetensors_io import read_header
                    shapes = {k: tuple(v.shape) for k, v in read_header(os.path.join(model_path, "model.safetensors"))[0].items()}
                l.mixer["right"]["decay_rank"] = int(shapes[f"l{i}.mix.right.w1"][0])
        cfg = cls(int(d["width"]), int(d["vocab"]), float(d["norm"]["eps"]), int(d["canon"]["taps"]), layers)
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": "Sisavik", "width": self.width, "vocab": self.vocab, "norm": {"eps": self.norm_eps},
                "canon": {"taps": self.canon_taps},
                "layers": [{"type": l.type, "mixer": l.mixer, "mlp": l.mlp} for l in self.layers]}


@dataclass
class GizezenConfig:
    """Gizezen: a pre-norm decoder of sliding-window attention layers with mixture-of-experts
    feed-forwards.  x <- x + m * mixer(N1(x)), x <- x + m * ff(N2(x)) with m = ``residual_mult`` and N
    a Dynamic Tanh norm, tanh(alpha x) w + b (no row statistics).  The attention runs a short causal
    convolution over q, k and v right after their projections, rotates pairs of q and k (frequencies
    optionally rescaled by wavelength, ``rot.scaling``), divides them by their root mean square per
    head, adds a silent key of score 0 to the softmax, and gates each head's output by a sigmoid of the
    layer's input; a layer with ``kv_from`` reads another layer's cached keys and values.  The
    feed-forward picks ``router.top`` experts by their logits (softmax over the chosen) and may add a
    sigmoid-gated shared expert.  Everything is read from config.json: ``width``, ``vocab``,
    ``norm.eps``, ``residual_mult``, ``embedding.scale`` and ``layers`` (per layer ``type``, ``mixer``
    sizes, ``mlp``)."""
    width: int
    vocab: int
    norm_eps: float
    residual_mult: float
    embedding_scale: float
    layers: list
    family = "gizezen"
    model_type = "gizezen"
    is_moe = False
    sliding_window = None
    tie_word_embeddings = False

    hidden_size = KagolixConfig.hidden_size
    vocab_size = KagolixConfig.vocab_size
    num_hidden_layers = KagolixConfig.num_hidden_layers
    num_layers_total = KagolixConfig.num_layers_total
    layer_names = KagolixConfig.layer_names
    layer = KagolixConfig.layer
    save = KagolixConfig.save
    total_params = KagolixConfig.total_params

    def kv_owner(self, i: int) -> int:
        """The layer whose cached keys and values layer ``i`` reads (itself unless it names ``kv_from``)."""
        j = self.layers[i].mixer.get("kv_from")
        return i if j is None else int(j)

    def validate(self) -> None:
        for i, l in enumerate(self.layers):
            m = l.mixer
            if l.type != "attention":
                raise NotImplementedError(f"layer {i}: mixer type {l.type!r}")
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            if int(m.get("conv", 1)) < 1:
                raise ValueError(f"layer {i}: conv must be >= 1 taps")
            rot = m.get("rot")
            if rot is not None and (int(rot["dims"]) > m["dim"] or int(rot["dims"]) % 2):
                raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
            if m.get("mask") is not None and int(m["mask"]["size"]) < 1:
                raise ValueError(f"layer {i}: mask.size must be >= 1")
            if m["dim"] > 512 or m["vdim"] > 512:
                # (head_norm_rope keeps a head in one wave's registers, the paged attention 8 value columns a lane)
                raise NotImplementedError(f"layer {i}: head sizes above 512")
            j = m.get("kv_from")
            if j is not None:
                o = self.layers[int(j)] if 0 <= int(j) < i else None
                if o is None or o.mixer.get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from must name an earlier layer with keys and values of its own")
                if any(o.mixer[k] != m[k] for k in ("kv_heads", "dim", "vdim")) or o.mixer.get("rot") != m.get("rot"):
                    raise ValueError(f"layer {i}: kv_heads, dim, vdim and rotation must equal layer {j}'s")
            if l.mlp is not None:
                if l.mlp.get("kind", "moe") != "moe":
                    raise NotImplementedError(f"layer {i}: mlp kind {l.mlp['kind']!r}")
                r = l.mlp["router"]
                if not 1 <= r["top"] <= min(r["experts"], 16) or r["experts"] > 1024:
                    raise NotImplementedError(f"layer {i}: router {r}")

    @classmethod
    def from_dict(cls, d: dict) -> "GizezenConfig":
        layers = [HybridLayer(l["type"], json.loads(json.dumps(l["mixer"])),
                              None if l.get("mlp") is None else json.loads(json.dumps(l["mlp"]))) for l in d["layers"]]
        cfg = cls(int(d["width"]), int(d["vocab"]), float(d["norm"]["eps"]), float(d.get("residual_mult", 1.0)),
                  float((d.get("embedding") or {}).get("scale", 1.0)), layers)
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": "Gizezen", "width": self.width, "vocab": self.vocab, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "embedding": {"scale": self.embedding_scale},
                "layers": [{"type": l.type, "mixer": l.mixer, "mlp": l.mlp} for l in self.layers]}


LOPILIX_MIXERS = ("attention", "hgrn2", "latent_attention")


@dataclass
class LopilixConfig:
    """Lopilix: a pre-norm decoder over several residual streams.  Sublayer q of a layer reads
    u = sum_s in_q[s] x_s through an RMS norm, its output is gated element by element by
    sigmoid(W_rg norm(u) + b), and the streams become x_t <- sum_s mix_q[s, t] x_s + m out_q[t] y
    (m = ``residual_mult``).  Mixers: differential attention (two softmax maps per head over shared
    values, the second subtracted lambda times, the difference unit-normed per head), HGRN2 (a gated
    linear recurrence whose forget gate also sets what is written) and latent attention (keys and
    values made from one cached latent row, a rotated key part shared by all heads, frequencies
    rescaled by how often an entry turns over the original context, a sigmoid output gate).
    Feed-forwards: SiLU-gated dense with biases, or a mixture of ungated GeLU experts chosen by
    sigmoid scores among the best groups of experts.  A learned position vector joins the embedding;
    the logits come from the embedding table, times ``logit_scale``.  ``loop``: layers start .. stop - 1
    run ``times`` times in a row on the same weights, every pass with a state of its own; a pass is a
    layer name of its own (``l2@1``) that shares layer 2's weight image."""
    width: int
    vocab: int
    norm_eps: float
    residual_mult: float
    streams: int
    logit_scale: float
    max_positions: int
    loop: Optional[dict]
    layers: list
    hyper: bool = True           # the checkpoint holds stream coefficients (else: one stream, plain sum)
    gated: bool = True           # the checkpoint holds the residual gates
    family = "lopilix"
    model_type = "lopilix"
    is_moe = False
    sliding_window = None
    tie_word_embeddings = True

    hidden_size = KagolixConfig.hidden_size
    vocab_size = KagolixConfig.vocab_size
    save = KagolixConfig.save

    def total_params(self) -> int:
        from .models.layout import layer_image, layer_layout_of
        images = dict.fromkeys(layer_image(n) for n in self.layer_names() if n != "head")     # (the head is the embedding table)
        return sum(sum(s.numel for s in layer_layout_of(self, n).slots) for n in images)

    @property
    def state_width(self) -> int:
        """Columns of the activation that passes from layer to layer: every stream's row side by side."""
        return self.streams * self.width

    def order(self) -> list:
        """[(layer number, pass)] in execution order."""
        n = len(self.layers)
        lp = self.loop
        if not lp or int(lp["times"]) == 1:
            return [(i, 0) for i in range(n)]
        a, b, k = int(lp["start"]), int(lp["stop"]), int(lp["times"])
        return [(i, 0) for i in range(a)] + [(i, p) for p in range(k) for i in range(a, b)] + [(i, 0) for i in range(b, n)]

    @property
    def num_hidden_layers(self) -> int:
        return len(self.order())

    @property
    def num_layers_total(self) -> int:
        return len(self.order()) + 3

    def layer_names(self) -> list:
        return ["embed"] + [f"l{i}" + (f"@{p}" if p else "") for i, p in self.order()] + ["final.norm", "head"]

    def layer(self, name: str) -> HybridLayer:
        return self.layers[int(name.split("@", 1)[0][1:])]

    def validate(self) -> None:
        if self.streams < 1 or self.streams > 8:
            raise NotImplementedError(f"streams={self.streams}: 1 to 8 residual streams")
        lp = self.loop
        if lp and not (0 <= int(lp["start"]) <= int(lp["stop"]) <= len(self.layers) and int(lp["times"]) >= 1):
            raise ValueError(f"loop {lp} does not fit {len(self.layers)} layers")
        for i, l in enumerate(self.layers):
            m = l.mixer
            if l.type not in LOPILIX_MIXERS:
                raise NotImplementedError(f"layer {i}: mixer type {l.type!r}")
            rot = m.get("rot")
            if l.type == "attention":
                if m["heads"] % m["kv_heads"]:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                if rot is not None and (int(rot["dims"]) > m["dim"] or int(rot["dims"]) % 2):
                    raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
            elif l.type == "latent_attention":
                if rot is not None and (int(rot["dims"]) > m["rot_dim"] or int(rot["dims"]) % 2):
                    raise ValueError(f"layer {i}: rot.dims must be even and at most rot_dim")
                if int(m["kv_rank"]) > 512 or int(m["kv_rank"]) + int(m["rot_dim"]) > 1024:
                    raise NotImplementedError(f"layer {i}: latent rows above 512 + 512")
            if max(int(m["dim"]), int(m["vdim"])) > 512:
                raise NotImplementedError(f"layer {i}: head sizes above 512")
            if l.type == "hgrn2" and int(m["dim"]) > 256:
                # (the scan keeps a value column's state rows in the registers of 16 lanes, 16 rows each)
                raise NotImplementedError(f"layer {i}: a recurrent state of more than 256 rows per head")
            if l.mlp is not None:
                if l.mlp["kind"] not in ("dense", "moe"):
                    raise NotImplementedError(f"layer {i}: mlp kind {l.mlp['kind']!r}")
                if l.mlp["kind"] == "moe":
                    r = l.mlp["router"]
                    if not 1 <= r["top"] <= min(r["experts"], 16) or r["experts"] > 1024:
                        raise NotImplementedError(f"layer {i}: router {r}")
                    g = r.get("groups")
                    if g and int(g["count"]) > 64:
                        raise NotImplementedError(f"layer {i}: more than 64 expert groups")
                    if g and (r["experts"] % int(g["count"]) or not 1 <= int(g["keep"]) <= int(g["count"])
                              or int(g["keep"]) * (r["experts"] // int(g["count"])) < r["top"]):
                        raise ValueError(f"layer {i}: router groups {g} do not fit {r['experts']} experts, top {r['top']}")

    @classmethod
    def from_dict(cls, d: dict, model_path: Optional[str] = None) -> "LopilixConfig":
        layers = [HybridLayer(l["type"], json.loads(json.dumps(l["mixer"])),
                              None if l.get("mlp") is None else json.loads(json.dumps(l["mlp"]))) for l in d["layers"]]
        hyper, gated = "streams" in d, True
        if model_path is not None and os.path.exists(os.path.join(model_path, "model.safetensors")):
            # which optional parts a checkpoint has shows in its tensor names
            from .utils.safetensors_io import read_header
            names = set(read_header(os.path.join(model_path, "model.safetensors"))[0])
            hyper, gated = "l0.hc1.in" in names, "l0.rg1" in names
        cfg = cls(int(d["width"]), int(d["vocab"]), float(d["norm"]["eps"]), float(d.get("residual_mult", 1.0)),
                  int(d.get("streams", 1)) if hyper else 1, float(d.get("logit_scale", 1.0)), int(d["max_positions"]),
                  json.loads(json.dumps(d.get("loop"))), layers, hyper, gated)
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        d = {"architecture": "Lopilix", "width": self.width, "vocab": self.vocab, "norm": {"eps": self.norm_eps},
             "residual_mult": self.residual_mult, "logit_scale": self.logit_scale, "max_positions": self.max_positions,
             "layers": [{"type": l.type, "mixer": l.mixer, "mlp": l.mlp} for l in self.layers]}
        if self.hyper:
            d["streams"] = self.streams
        if self.loop:
            d["loop"] = self.loop
        return d


# "architecture" of config.json -> config class of a stateful hybrid family
ARCHITECTURES = {"Kagolix": KagolixConfig, "Sisavik": SisavikConfig, "Gizezen": GizezenConfig, "Lopilix": LopilixConfig}


def load_config(model_path: str):
    """The config of the model in ``model_path``: a hybrid family when config.json names one with
    "architecture", else the dense (Llama-structured) family's ModelConfig."""
    with open(os.path.join(model_path, "config.json")) as f:
        d = json.load(f)
    arch = d.get("architecture")
    if arch is not None:
        if arch not in ARCHITECTURES:
            raise NotImplementedError(f"architecture {arch!r}: supported are {sorted(ARCHITECTURES)}")
        if arch in ("Sisavik", "Lopilix"):             # (they read what config.json leaves open from the checkpoint's header)
            return ARCHITECTURES[arch].from_dict(d, model_path)
        return ARCHITECTURES[arch].from_dict(d)
    return ModelConfig.from_dict(d)


def is_hybrid(cfg) -> bool:
    return getattr(cfg, "family", "dense") != "dense"

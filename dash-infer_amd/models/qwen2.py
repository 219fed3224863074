"""Qwen2 / Qwen2-MoE: config.json -> decoder.ModelConfig of the quantised decode runner (decoder.DecodeSession)."""
from . import register


@register("Qwen2ForCausalLM", "qwen2", "Qwen2MoeForCausalLM", "qwen2_moe")
class Qwen2Family:
    engine = "decode_session"

    @staticmethod
    def model_config(config):
        from ..decoder import ModelConfig, MoEConfig
        moe = None
        if config.get("num_experts"):
            moe = MoEConfig(int(config["num_experts"]), int(config["num_experts_per_tok"]), int(config["moe_intermediate_size"]))
        hidden, heads = int(config["hidden_size"]), int(config["num_attention_heads"])
        inter = int(config.get("shared_expert_intermediate_size") or config["intermediate_size"]) if moe else int(config["intermediate_size"])
        return ModelConfig(config.get("_name_or_path") or "Qwen2", hidden, int(config["num_hidden_layers"]), heads,
                           int(config.get("num_key_value_heads") or heads), int(config.get("head_dim") or hidden // heads), inter,
                           int(config["vocab_size"]), float(config.get("rms_norm_eps", 1e-6)), float(config.get("rope_theta", 1e6)), moe)

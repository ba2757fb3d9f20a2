"""The Qwen3 dense decoder as a ModelSpec
(src/qwen3_from_scratch/models/qwen3.py:9-84): token embedding, L pre-norm
layers of grouped-head attention with per-head q/k RMSNorm and rotary position
plus a SwiGLU feed-forward, a final RMSNorm, and a linear head that is the
embedding when `tie_word_embeddings` is set."""

from ..config.model_config import ModelConfig
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .spec import ModelSpec, RunStep, pre_norm_layer


def qwen3_spec(config):
    norm = PartSpec.of("norm", "rms", size=config.hidden_size, eps=config.rms_norm_eps)
    mixer = PartSpec.of(
        "mixer", "attention",
        hidden_size=config.hidden_size,
        num_heads=config.num_attention_heads,
        num_kv_heads=config.num_key_value_heads,
        head_dim=config.head_dim,
        qk_norm=True,
        qk_norm_eps=config.rms_norm_eps,
        window=0,
    )
    feed_forward = PartSpec.of(
        "feed_forward", "swiglu",
        hidden_size=config.hidden_size, intermediate_size=config.intermediate_size)
    layers = tuple(
        pre_norm_layer("model.layers.%d" % i, mixer=mixer, feed_forward=feed_forward,
                       mixer_norm=norm, feed_forward_norm=norm)
        for i in range(config.num_hidden_layers)
    )
    tied = config.tie_word_embeddings
    return ModelSpec(
        hidden_size=config.hidden_size,
        vocab_size=config.vocab_size,
        embedding=PartSpec.of("embedding", "token", vocab_size=config.vocab_size,
                              hidden_size=config.hidden_size),
        embedding_prefix="model.embed_tokens",
        position=PartSpec.of("position", "rotary", rotary_dim=config.head_dim,
                             theta=config.rope_theta, max_positions=config.max_position_embeddings),
        layers=layers,
        order=tuple(RunStep(i) for i in range(len(layers))),
        final_norm=norm,
        final_norm_prefix="model.norm",
        head=PartSpec.of("head", "linear", hidden_size=config.hidden_size, vocab_size=config.vocab_size,
                         weight_name="model.embed_tokens.weight" if tied else "lm_head.weight"),
        # a tied checkpoint may still carry a copy of the head; it is not read
        ignorable_tensors=("lm_head.weight",) if tied else (),
    )


register_architecture("Qwen3ForCausalLM", ModelConfig, qwen3_spec)

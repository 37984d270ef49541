"""The Llama decoder as a list of parts chosen by LlamaConfig: per layer an
RMSNorm, grouped-query attention with rotary embedding, an RMSNorm and a gated
feed-forward in the pre-norm arrangement; tensor names are the Hugging Face
ones the reference binds (runtime/model.py:38-55, runtime/checkpoint.py:44-58).
"""
from ..config.base import register_architecture
from ..config.llama import LlamaConfig
from ..parts import make_part, TokenEmbedding, LMHead
from .model import Model


def build_llama(config):
    c = config
    embedding = TokenEmbedding("model.embed_tokens", c.vocab_size, c.hidden_size)
    layers = []
    # one position part for the whole model: every layer turns by the same angles, so the tables exist once
    position = make_part("position", "rotary", head_dim=c.head_dim, theta=c.rope_theta,
                         max_positions=c.max_position_embeddings)
    for i in range(c.num_hidden_layers):
        p = f"model.layers.{i}"
        mixer = make_part("mixer", "attention", name=p + ".self_attn", hidden=c.hidden_size,
                          heads=c.num_attention_heads, kv_heads=c.num_key_value_heads, head_dim=c.head_dim,
                          position=position)
        ffn = make_part("ffn", "gated_mlp", name=p + ".mlp", hidden=c.hidden_size, intermediate=c.intermediate_size)
        layers.append(make_part(
            "block", "prenorm",
            mixer_norm=make_part("norm", "rmsnorm", name=p + ".input_layernorm", dim=c.hidden_size, eps=c.rms_norm_eps),
            mixer=mixer,
            ffn_norm=make_part("norm", "rmsnorm", name=p + ".post_attention_layernorm", dim=c.hidden_size, eps=c.rms_norm_eps),
            ffn=ffn))
    final_norm = make_part("norm", "rmsnorm", name="model.norm", dim=c.hidden_size, eps=c.rms_norm_eps)
    head = LMHead("lm_head", c.vocab_size, c.hidden_size, tied_to=embedding if c.tie_word_embeddings else None)
    return Model(c, embedding, layers, final_norm, head, max_positions=c.max_position_embeddings, vocab_size=c.vocab_size)


register_architecture(["LlamaForCausalLM", "llama"], LlamaConfig, build_llama)

"""OPT as a `ModelSpec`: which parts, with which sizes, under which tensor names.

Tensor names are the checkpoint's (reference: the module tree of
opt/model.py:195-270 and the table of opt/gen_random_pretrained.py:49-76), plus
`project_in`/`project_out` when the embedding width differs from the hidden one.
"""
from .config import OPTConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec

# OPT reads row `position + 2` of its position table (opt/model.py:237-244): a
# constant of the architecture, not of a checkpoint.
POSITION_OFFSET = 2


def opt_spec(cfg: OPTConfig) -> ModelSpec:
    h, e = cfg.hidden_size, cfg.word_embed_proj_dim
    norm = PartSpec("layer_norm", dict(width=h, eps=cfg.layer_norm_eps, affine=cfg.layer_norm_elementwise_affine))
    mixer = PartSpec("attention", dict(width=h, num_heads=cfg.num_attention_heads, head_size=cfg.head_size,
                                       num_kv_heads=cfg.num_attention_heads, bias=cfg.enable_bias,
                                       names=("q_proj", "k_proj", "v_proj", "out_proj")))
    ffn = PartSpec("dense", dict(width=h, inner=cfg.ffn_dim, activation=cfg.activation_function,
                                 bias=cfg.enable_bias, up_name="fc1", down_name="fc2"))
    block = "pre_norm" if cfg.do_layer_norm_before else "post_norm"
    layers = tuple(
        LayerSpec(prefix=f"model.decoder.layers.{i}.", block=block, mixer=mixer, feed_forward=ffn,
                  mixer_norm=norm, feed_forward_norm=norm,
                  mixer_name="self_attn.", feed_forward_name="",
                  mixer_norm_name="self_attn_layer_norm", feed_forward_norm_name="final_layer_norm")
        for i in range(cfg.num_hidden_layers))
    embedding = PartSpec("token_table", dict(
        vocab=cfg.vocab_size, embed_width=e, width=h,
        position=PartSpec("learned", dict(width=h, max_positions=cfg.max_position_embeddings,
                                          offset=POSITION_OFFSET)),
        table_name="model.decoder.embed_tokens.weight",
        projection_name="model.decoder.project_in.weight",
        position_name="model.decoder.embed_positions"))
    head = PartSpec("vocab_projection", dict(
        vocab=cfg.vocab_size, embed_width=e, width=h,
        norm=norm if cfg.do_layer_norm_before and not cfg._remove_final_layer_norm else None,
        weight_name="lm_head.weight",
        tied_to="model.decoder.embed_tokens.weight" if cfg.tie_word_embeddings else None,
        projection_name="model.decoder.project_out.weight",
        norm_name="model.decoder.final_layer_norm"))
    return ModelSpec(hidden_size=h, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
                     embedding=embedding, layers=layers, schedule=ModelSpec.sequential(cfg.num_hidden_layers),
                     head=head, init_std=cfg.init_std, base_model_prefix="model.")


ARCHITECTURE = register_architecture("OPTForCausalLM", "opt", OPTConfig, opt_spec,
                                     model_class="transformers_neuronx_amd.opt.model:OPTForSampling")

"""OPT: learned positions (offset 2), LayerNorm, ReLU feed-forward, biased
multi-head attention; pre-norm with a final norm, or post-norm without one.

This module turns OPT's config.json into a ``ModelSpec`` (which parts, which
sizes, which tensor names) and registers it under ``"OPTForCausalLM"``.  The
reference's counterpart is ``GetOptHyperParam`` (src/csrc/model/gpt/gpt_hyper_param.h:51-77)
plus the tensor names its loader reads (src/csrc/model/gpt/gpt_weight.cc:274-321);
the names here are those of the model folder's safetensors file, where q, k and v
are separate tensors stored [out, in]."""
from __future__ import annotations

from ..config.hyper_param import OptHyperParam
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def build_opt_spec(hp: OptHyperParam) -> ModelSpec:
    hp.validate()
    dec = "model.decoder"
    norm_params = {"eps": hp.layer_norm_eps, "affine": hp.layer_norm_elementwise_affine}
    layers = []
    for i in range(hp.num_hidden_layers):
        p = f"{dec}.layers.{i}"
        layers.append(LayerSpec(
            arrangement=PartSpec("pre_norm" if hp.do_layer_norm_before else "post_norm"),
            mixer_norm=PartSpec("layer_norm", dict(norm_params),
                                {"weight": f"{p}.self_attn_layer_norm.weight",
                                 "bias": f"{p}.self_attn_layer_norm.bias"}),
            mixer=PartSpec("paged_attention",
                           {"num_heads": hp.num_attention_heads, "num_kv_heads": hp.num_kv_heads,
                            "head_dim": hp.head_dim,
                            # score scale head_dim**-0.5 (src/csrc/layer/attention.cc:91)
                            "scale": float(hp.head_dim) ** -0.5,
                            "bias": hp.enable_bias, "window": 0},
                           {f"{n}.{t}": f"{p}.self_attn.{n}_proj.{t}"
                            for n in ("q", "k", "v", "out") for t in ("weight", "bias")}),
            ffn_norm=PartSpec("layer_norm", dict(norm_params),
                              {"weight": f"{p}.final_layer_norm.weight",
                               "bias": f"{p}.final_layer_norm.bias"}),
            feed_forward=PartSpec("dense",
                                  {"inner": hp.ffn_dim, "activation": hp.activation_function,
                                   "bias": hp.enable_bias},
                                  {f"{n}.{t}": f"{p}.{n}.{t}" for n in ("fc1", "fc2")
                                   for t in ("weight", "bias")}),
        ))
    embed_name = f"{dec}.embed_tokens.weight"
    return ModelSpec(
        hidden_size=hp.hidden_size,
        vocab_size=hp.vocab_size,
        max_positions=hp.max_position_embeddings,
        embedding=PartSpec("token", {"vocab_size": hp.vocab_size, "embed_dim": hp.word_embed_proj_dim},
                           {"weight": embed_name, "project_in": f"{dec}.project_in.weight"}),
        position=PartSpec("learned", {"max_positions": hp.max_position_embeddings,
                                      "offset": hp.position_offset},
                          {"weight": f"{dec}.embed_positions.weight"}),
        layers=layers,
        schedule=[ScheduleEntry(layer=i, cache=i) for i in range(hp.num_hidden_layers)],
        final_norm=(PartSpec("layer_norm", dict(norm_params),
                             {"weight": f"{dec}.final_layer_norm.weight",
                              "bias": f"{dec}.final_layer_norm.bias"})
                    if hp.has_final_norm else None),
        head=PartSpec("linear", {"vocab_size": hp.vocab_size, "embed_dim": hp.word_embed_proj_dim,
                                 "tied_to": embed_name if hp.tie_word_embeddings else None},
                      {"weight": "lm_head.weight", "project_out": f"{dec}.project_out.weight"}),
        eos_token_id=hp.eos_token_id,
    ).validate()


def _presets(name: str, **overrides) -> OptHyperParam:
    from ..config.presets import preset
    return preset(name, **overrides)


register_architecture("OPTForCausalLM", OptHyperParam, build_opt_spec, short_name="opt", presets=_presets)

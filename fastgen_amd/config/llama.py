"""The dense Llama decoder as a layout of parts.

Layer composition follows ``fastgen/forward.py:412-499`` (pre-norm
attention, pre-norm SwiGLU, both added to the residual stream) and the
tensor names ``fastgen/utils/loading.py:88-143``.
"""

from __future__ import annotations

from typing import Any, Mapping

from .layout import LayerSpec, ModelLayout, PartSpec, RunEntry
from .model_args import ModelArgs
from .registry import register_architecture


class LlamaArchitecture:
    name = "LlamaForCausalLM"

    def parse(self, config: Mapping[str, Any]) -> ModelArgs:
        return ModelArgs.from_hf_config(config)

    def to_hf_config(self, args: ModelArgs) -> dict:
        return args.to_hf_config()

    def layout(self, args: ModelArgs) -> ModelLayout:
        rope = PartSpec(
            "rope",
            options=dict(
                head_dim=args.head_dim,
                rotary_dim=args.head_dim,
                theta=args.rope.theta,
                scaled=args.rope.scaled,
                original_context=args.rope.original_context,
                factor=args.rope.factor,
                low_freq_factor=args.rope.low_freq_factor,
                high_freq_factor=args.rope.high_freq_factor,
            ),
        )

        def norm(prefix: str) -> PartSpec:
            return PartSpec("rmsnorm", prefix, dict(dim=args.dim, eps=args.norm_eps))

        layers = []
        for i in range(args.n_layers):
            p = f"model.layers.{i}"
            layers.append(
                LayerSpec(
                    mixer=PartSpec(
                        "attention",
                        f"{p}.self_attn",
                        dict(
                            dim=args.dim,
                            n_heads=args.n_heads,
                            n_kv_heads=args.n_kv_heads,
                            head_dim=args.head_dim,
                            scale=args.head_dim**-0.5,
                            window=None,
                            position=rope,
                        ),
                    ),
                    ffn=PartSpec(
                        "swiglu",
                        f"{p}.mlp",
                        dict(dim=args.dim, hidden_dim=args.ffn_dim),
                    ),
                    mixer_norm=norm(f"{p}.input_layernorm"),
                    ffn_norm=norm(f"{p}.post_attention_layernorm"),
                    arrangement="pre_norm",
                )
            )
        return ModelLayout(
            dim=args.dim,
            vocab_size=args.vocab_size,
            embed=PartSpec(
                "embedding",
                "model.embed_tokens",
                dict(vocab_size=args.vocab_size, dim=args.dim),
            ),
            layers=tuple(layers),
            order=tuple(RunEntry(i) for i in range(args.n_layers)),
            final_norm=norm("model.norm"),
            head=PartSpec(
                "lm_head",
                "lm_head",
                dict(
                    vocab_size=args.vocab_size,
                    dim=args.dim,
                    tied_to="model.embed_tokens" if args.tie_embeddings else None,
                ),
            ),
        )


LLAMA = register_architecture(LlamaArchitecture())

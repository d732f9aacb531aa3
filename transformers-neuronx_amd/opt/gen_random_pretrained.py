"""Write an OPT model folder with random weights.

    opt_gen_random_pretrained NAME SAVE [--seed N] [--dtype DTYPE]

NAME is the path of a config.json (or of a folder that holds one), or
`facebook/opt-175b`, whose configuration is built in as in the reference
(opt/gen_random_pretrained.py:105-140). The reference's `--empty` (shapes only,
weights drawn at load time) has no use here: `--seed` makes a folder repeatable.
"""
import argparse
import json
import os

from .config import OPTConfig
from ..weights.random_init import write_random_model


def opt_175b_config() -> dict:
    """The sizes of the largest published OPT (opt/gen_random_pretrained.py:105-140)."""
    return dict(architectures=["OPTForCausalLM"], model_type="opt", activation_function="relu",
                bos_token_id=2, eos_token_id=2, pad_token_id=1, do_layer_norm_before=True,
                hidden_size=12288, ffn_dim=49152, num_hidden_layers=96, num_attention_heads=96,
                max_position_embeddings=2048, vocab_size=50272, word_embed_proj_dim=12288,
                init_std=0.02, torch_dtype="float16")


def gen_random_pretrained(model_name: str, save: str, seed: int = 0, dtype=None) -> str:
    if model_name == "facebook/opt-175b":
        raw = opt_175b_config()
    else:
        path = os.path.join(model_name, "config.json") if os.path.isdir(model_name) else model_name
        if not os.path.exists(path):
            raise FileNotFoundError(f"{model_name}: no such config.json (there is no network to fetch a model name)")
        with open(path) as fp:
            raw = json.load(fp)
    return write_random_model(OPTConfig.from_dict(raw), save, seed, dtype)


def main(argv=None):
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("name", help="path to config.json, or facebook/opt-175b")
    parser.add_argument("save", help="target folder to save the model")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--dtype", default=None, choices=["float32", "float16", "bfloat16"],
                        help="storage dtype of matrices (default: the config's torch_dtype)")
    args = parser.parse_args(argv)
    out = gen_random_pretrained(args.name, args.save, args.seed, args.dtype)
    print(f"done saving {out}")


if __name__ == "__main__":
    main()

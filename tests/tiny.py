"""The tiny configurations of the tests, and helpers that write their model folders.

A and B are the two configurations the benchmark description names; C adds sizes that are no
power of two anywhere (a feed-forward width that is no multiple of 8, an odd vocabulary, as
many key heads as query heads, two taps); D has heads 64 wide.  Weights are drawn with a standard deviation of
0.1 rather than 0.02, so that every sub-layer moves the stream by about as much as the stream
itself holds and a fault in any of them shows in the logits.
"""
import os

import torch

from gesso_amd.config import Lfm2Config
from gesso_amd.weights import write_model_folder

STD = 0.1

TINY_A = Lfm2Config(
    vocab_size=256, hidden_size=64, num_hidden_layers=4, num_attention_heads=4, num_key_value_heads=2,
    layer_types=("conv", "full_attention", "conv", "full_attention"), conv_L_cache=3, conv_bias=False,
    intermediate_size=192, norm_eps=1e-5, rope_theta=1e4, tie_word_embeddings=True, max_position_embeddings=256)

TINY_B = Lfm2Config(
    vocab_size=512, hidden_size=96, num_hidden_layers=6, num_attention_heads=3, num_key_value_heads=1,
    layer_types=("full_attention", "conv", "full_attention", "conv", "conv", "full_attention"), conv_L_cache=4,
    conv_bias=True, intermediate_size=320, norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False,
    max_position_embeddings=512)

TINY_C = Lfm2Config(
    vocab_size=301, hidden_size=144, num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=3,
    layer_types=("full_attention", "full_attention", "conv"), conv_L_cache=2, conv_bias=False,
    intermediate_size=100, norm_eps=1e-4, rope_theta=5e5, tie_word_embeddings=True, max_position_embeddings=384)

# D has the head width of the benchmark's model (64), so that the kernels written for it (attention on the matrix
# cores for prompts and for decoding, the 16-byte head norm and rotation) run inside a whole model, two query
# heads to a key head
TINY_D = Lfm2Config(
    vocab_size=200, hidden_size=128, num_hidden_layers=3, num_attention_heads=2, num_key_value_heads=1,
    layer_types=("full_attention", "conv", "full_attention"), conv_L_cache=3, conv_bias=False,
    intermediate_size=136, norm_eps=1e-5, rope_theta=1e5, tie_word_embeddings=True, max_position_embeddings=320)

CONFIGS = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3)}


def write_tiny(root: str, name: str, dtype=torch.float32) -> str:
    cfg, seed = CONFIGS[name]
    d = os.path.join(root, f"tiny_{name}_{str(dtype).split('.')[-1]}")
    if not os.path.exists(os.path.join(d, "model.safetensors")):
        write_model_folder(d, cfg, seed, dtype, std=STD)
    return d


def random_ids(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()

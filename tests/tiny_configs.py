"""The two tiny Falcon-H1 configurations of the test-suite.  They differ in every size
and option: layers, width, heads and groups, head size, feed-forward width, SSM heads,
head size, state size, groups, conv taps, chunk, biases, gated norm, tied embeddings,
multipliers, rope base, norm eps and vocabulary."""
import torch

from macllm_infer_amd.config import FalconH1Config
from macllm_infer_amd.weights.random_init import write_random_model

TINY_A = dict(
    architectures=["FalconH1ForCausalLM"], model_type="falcon_h1",
    hidden_size=64, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    intermediate_size=128, vocab_size=256, max_position_embeddings=1024, rms_norm_eps=1e-5, rope_theta=1e4,
    mamba_n_heads=8, mamba_d_head=8, mamba_d_ssm=64, mamba_d_state=16, mamba_n_groups=1, mamba_d_conv=4,
    mamba_chunk_size=16, mamba_conv_bias=False, mamba_proj_bias=False, mamba_rms_norm=False,
    attention_bias=False, mlp_bias=False, tie_word_embeddings=True)

TINY_B = dict(
    architectures=["FalconH1ForCausalLM"], model_type="falcon_h1",
    hidden_size=96, num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=3, head_dim=32,
    intermediate_size=160, vocab_size=320, max_position_embeddings=768, rms_norm_eps=3e-6, rope_theta=1e11,
    mamba_n_heads=6, mamba_d_head=16, mamba_d_ssm=96, mamba_d_state=32, mamba_n_groups=2, mamba_d_conv=3,
    mamba_chunk_size=8, mamba_conv_bias=True, mamba_proj_bias=True, mamba_rms_norm=True,
    attention_bias=True, mlp_bias=True, tie_word_embeddings=False,
    embedding_multiplier=1.7, lm_head_multiplier=0.6, attention_in_multiplier=1.3,
    attention_out_multiplier=0.8, key_multiplier=0.7, ssm_in_multiplier=1.2, ssm_out_multiplier=0.9,
    ssm_multipliers=[0.8, 1.4, 0.6, 1.5, 1.1], mlp_multipliers=[1.25, 0.75])

# Small, but with the head size, state size and widths that the matrix-core and fused decode
# kernels cover (head_dim 64, widths that are multiples of 32), so that replay runs through them.
TINY_C = dict(
    architectures=["FalconH1ForCausalLM"], model_type="falcon_h1",
    hidden_size=128, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
    intermediate_size=96, vocab_size=200, max_position_embeddings=640, rms_norm_eps=1e-5, rope_theta=1e6,
    mamba_n_heads=4, mamba_d_head=16, mamba_d_ssm=64, mamba_d_state=32, mamba_n_groups=1, mamba_d_conv=4,
    mamba_chunk_size=32, mamba_conv_bias=True, mamba_proj_bias=False, mamba_rms_norm=False,
    attention_bias=False, mlp_bias=False, tie_word_embeddings=True,
    embedding_multiplier=1.2, lm_head_multiplier=0.8, key_multiplier=0.9, ssm_multipliers=[1.0, 1.2, 0.9, 1.1, 1.0])

# One wide layer: the hidden size is beyond what the norm prologue of the fused decode kernels
# holds in LDS (norms then run as kernels of their own), head_dim 128, 6 query heads on one kv head.
TINY_D = dict(
    architectures=["FalconH1ForCausalLM"], model_type="falcon_h1",
    hidden_size=2112, num_hidden_layers=1, num_attention_heads=6, num_key_value_heads=1, head_dim=128,
    intermediate_size=64, vocab_size=120, max_position_embeddings=640, rms_norm_eps=1e-5, rope_theta=1e5,
    mamba_n_heads=8, mamba_d_head=16, mamba_d_ssm=128, mamba_d_state=64, mamba_n_groups=1, mamba_d_conv=4,
    mamba_chunk_size=64, mamba_conv_bias=True, mamba_proj_bias=False, mamba_rms_norm=False,
    attention_bias=False, mlp_bias=False, tie_word_embeddings=False)

CONFIGS = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3)}


def config(name):
    return FalconH1Config.from_dict(CONFIGS[name][0])


def make_model_dir(name, folder, dtype=torch.float32, preset="unit"):
    raw, seed = CONFIGS[name]
    return write_random_model(FalconH1Config.from_dict(raw), seed, str(folder), dtype, preset)


def random_config(seed, odd=False):
    """(configuration, page size, the generator that drew them) with every size and option drawn at random:
    head sizes in steps of 16, head counts and groups that are no powers of two, widths and vocabularies that
    are no multiples of anything, multipliers between 0.5 and 2.  ``odd``: widths, state sizes and chunks
    that no matrix-core kernel takes (the scalar paths of every part)."""
    import random
    rng = random.Random(seed)
    divisors = lambda n: [d for d in range(1, n + 1) if n % d == 0]
    heads = rng.choice([1, 2, 3, 4, 6, 8, 12])
    mamba_heads = rng.choice([1, 2, 3, 4, 6, 8])
    head = rng.choice([4, 12, 20, 36] if odd else [8, 16, 24, 32, 64])
    factor = lambda: rng.uniform(0.5, 2)
    raw = dict(
        architectures=["FalconH1ForCausalLM"], model_type="falcon_h1",
        hidden_size=rng.choice([30, 50, 66, 90, 34] if odd else [40, 72, 100, 128, 136, 256, 520]),
        num_hidden_layers=rng.choice([1, 2]),
        num_attention_heads=heads, num_key_value_heads=rng.choice(divisors(heads)),
        head_dim=rng.choice([16, 32, 48, 64, 80, 128]),
        intermediate_size=rng.choice([10, 30, 50, 7] if odd else [24, 100, 136, 256]),
        vocab_size=rng.choice([33, 50, 129] if odd else [97, 320, 1003]), max_position_embeddings=512,
        rms_norm_eps=rng.choice([1e-5, 1e-6, 3e-4]), rope_theta=rng.choice([1e4, 1e6, 1e11]),
        mamba_n_heads=mamba_heads, mamba_d_head=head, mamba_d_ssm=mamba_heads * head,
        mamba_d_state=rng.choice([4, 12, 24, 20] if odd else [8, 16, 32, 40, 64, 128]),
        mamba_n_groups=rng.choice(divisors(mamba_heads)),
        mamba_d_conv=rng.choice([2, 3, 4]), mamba_chunk_size=rng.choice([5, 16, 48, 100] if odd else [8, 32, 64, 128]),
        mamba_conv_bias=rng.random() < 0.5, mamba_proj_bias=rng.random() < 0.5, mamba_rms_norm=rng.random() < 0.5,
        attention_bias=rng.random() < 0.5, mlp_bias=rng.random() < 0.5, tie_word_embeddings=rng.random() < 0.5,
        embedding_multiplier=factor(), lm_head_multiplier=factor(), key_multiplier=factor(),
        attention_in_multiplier=factor(), attention_out_multiplier=factor(), ssm_in_multiplier=factor(),
        ssm_out_multiplier=factor(), ssm_multipliers=[factor() for _ in range(5)],
        mlp_multipliers=[factor() for _ in range(2)])
    return raw, rng.choice([4, 8, 16, 64]), rng

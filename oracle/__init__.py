"""CPU oracle for the AERIS window-partitioned Swin denoiser hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may use it, and only as the checker.

The oracle restates, in plain fp32 PyTorch and numpy on the CPU, what
``src/aeris_wp_inference/model.py`` and ``src/aeris_wp_inference/inference.py``
of the reference compute on the hot path, extended with the classic Swin-v1
features (LayerNorm, relative-position bias, cyclic-shift mask, GELU MLP,
Linear biases) that the benchmark configurations ask for.

Pinning status (the reference ships no tests, fixtures or golden vectors, so
every function is pinned by library routines, closed forms, invariants and
brute force on tiny inputs in ``tests/test_oracle_*.py``):

  index maps (partition / reverse / roll)   pinned  (einops + torch.roll + loops)
  relative-position index, shift mask       pinned  (brute-force loops)
  window attention                          pinned  (float64 loops, SDPA, invariants)
  norms, modulate, MLPs, modulation MLP     pinned  (torch.nn library modules, closed forms)
  timestep embedding, 2-D positional enc.   pinned  (closed forms, known answers)
  block / model composition                 pinned  (identity + plain-pre-norm invariants,
                                                     roll-equivalence of the folded shift)
  sampler schedule and Heun update          pinned  (closed forms, linear test field)
"""
from .index_maps import (  # noqa: F401
    window_token_index,
    window_token_index_loops,
    relative_position_index,
    relative_position_index_loops,
    shift_region_ids,
    shift_attention_mask,
)
from .swin_oracle import (  # noqa: F401
    OracleConfig,
    init_block_weights,
    init_model_weights,
    layer_norm,
    rms_norm,
    modulate,
    modulation_mlp,
    timestep_embedding,
    positional_encoding_2d,
    window_attention,
    attention_branch,
    mlp_branch,
    block_forward,
    input_stage,
    output_stage,
    model_forward,
)
from .sampler_oracle import sigma_schedule, sample, rollout  # noqa: F401

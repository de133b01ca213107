"""CPU oracle for the one-GPU DiT denoise-step hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the shipped
product: it may be imported only by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py``, and there only as the checker
or as the timed CPU baseline.  The product package never imports it.

The oracle restates, in explicit fp32 formulas on the CPU, what the reference
computes for the MMDiT / DiT transformer block.  The reference owns the
attention wrapper, the attention processors, ``apply_rotary_emb``, the
FeedForward wrapper, the block-loop callers and the KV ``CacheManager``
(``hetu_dit/model_executor/diffusion_executor/layers/attention_processor.py``,
``.../layers/feedforward.py``, ``hetu_dit/core/resource_manager/cache_manager.py``).
The block arithmetic itself (adaLN-Zero, LayerNorm, gated residual, GELU-tanh
MLP, RMSNorm, RoPE tables) lives in the third-party ``diffusers`` package
(``setup.py:27``, ``diffusers>=0.31``, no upper pin), which is neither under
``/root/reference`` nor installed; its published algorithm is restated here and
anchored on the reference's call sites.

Pinning status
--------------
The reference holds no tests, golden vectors or fixtures.  Each function is
therefore pinned by what mathematics and PyTorch's own library routines fix
(see ``tests/test_oracle_*.py``):

* ``linear``            -- ``torch.nn.functional.linear``, identity / one-hot KATs
* ``layer_norm``        -- ``F.layer_norm``; zero-mean / unit-variance invariant
* ``rms_norm``          -- ``F.rms_norm``; scale invariance
* ``gelu_tanh``         -- ``F.gelu(approximate="tanh")``; values at 0, +-1, large |x|
* ``gelu_erf``          -- ``F.gelu``, ``math.erf`` point by point, the identity gelu(x) - gelu(-x) = x;
                           ``feed_forward`` with "gelu" / "geglu" / "linear-silu" against a chain of
                           ``F.linear`` / ``F.gelu`` / ``F.silu`` with mutations (swapped halves, tanh for erf)
* ``silu``              -- ``F.silu``
* ``attention``         -- ``F.scaled_dot_product_attention`` (math backend), numpy
                           brute force, rows-sum-to-one, constant-V, KV permutation
                           invariance, query-row independence
* ``apply_rotary_emb``  -- complex-multiplication form, norm preservation,
                           position-0 identity, relative-position property
* ``flux_rope_table`` / ``cogvideox_rope_table`` -- closed-form angle checks
* stale KV buffer       -- brute-force concatenation of fresh and stale slices
* block wiring (``sd3_joint_block`` with and without ``context_pre_only``,
  ``flux_double_block``, ``flux_single_block``, ``cogvideox_block``, and the
  attention functions inside them): every block is assembled a second time in
  ``tests/test_oracle_wiring.py`` from PyTorch's library modules
  (``nn.LayerNorm``, ``nn.Linear``, ``F.silu``, ``F.gelu(approximate="tanh")``,
  ``F.rms_norm``, ``F.scaled_dot_product_attention``, complex multiplication for
  the rotary embedding) in the order of the published diffusers ``forward`` of
  ``JointTransformerBlock``, ``FluxTransformerBlock``,
  ``FluxSingleTransformerBlock``, ``CogVideoXBlock``, ``AdaLayerNormZero``,
  ``AdaLayerNormZeroSingle``, ``AdaLayerNormContinuous``,
  ``CogVideoXLayerNormZero`` and of the reference's processors; the two agree
  to fp32 round-off, and each of some thirty plausible wiring mistakes (shift
  and scale swapped, gate chunks swapped, eps 1e-5 <-> 1e-6, scale-first <->
  shift-first, affine dropped, joint order flipped, text bias kept, wrong norm
  weights, rotation missing or on the wrong rows) breaks the agreement.  Also
  pinned: the adaLN-"Zero" identity (zero modulation weights => block is the
  identity on the residual stream), return orders and split points fixed by
  the reference's call sites, patch mode with a fresh buffer = rows of the full
  pass (``tests/test_oracle_blocks.py``).  What no test here can confirm is
  that the published diffusers modules are what the package a deployment
  installs really computes: diffusers (``setup.py:27``, ``>=0.31``, no upper
  pin) is neither under ``/root/reference`` nor installed, and the reference
  holds no golden vectors.
* head and tail of a step (``oracle/step.py``): patch embedding -- ``F.conv2d``;
  unpatchify -- ``F.fold`` and index checks; timestep projection and the 2-D
  sin-cos table -- closed forms; conditioning embedders and ``norm_out`` +
  ``proj_out`` -- ``torch.nn`` modules; guidance + Euler update -- fp64
  identities.  The layout conventions of diffusers' position table, timestep
  projection and sigma schedule are **parity unpinned** (see that file's header).
"""

from .ops import (  # noqa: F401
    silu,
    gelu_erf,
    gelu_tanh,
    linear,
    layer_norm,
    rms_norm,
    attention,
    apply_rotary_emb,
    flux_rope_table,
    cogvideox_rope_table,
    adaln_modulation,
    modulate,
)
from .blocks import (  # noqa: F401
    sd3_joint_block,
    flux_double_block,
    flux_single_block,
    cogvideox_block,
    feed_forward,
)
from .kv_cache import StaleKVBuffer  # noqa: F401
from . import step  # noqa: F401

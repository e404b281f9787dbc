"""CPU oracle for the transformer-layer hot path.

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain
CPU torch, the arithmetic of the reference's `torch` masked-softmax kernel path
(attention core, dense mask construction, rotary, RMSNorm / LayerNorm, SwiGLU /
GELU MLP, pre-norm transformer layer, KV-cache decode) so that the HIP kernels
can be checked against it.  Only the test-suite, the smoke check and the
`cpu_baseline` leg of the benchmark may import it; the product package
(`scaling_amd`) never does and fails loudly when its HIP library is missing.

Every function cites the reference file:line it follows (paths relative to the
reference checkout's `src/scaling/`).  The functions run in the dtype of their
inputs, reproducing the reference's rounding points (scores rounded to the
input dtype before the softmax, probabilities rounded to the value dtype before
PV, cos/sin tables rounded to the module dtype, RMSNorm arithmetic in the input
dtype).  Feeding fp32 / fp64 tensors yields the high-precision truth that the
parity tests compare the kernels against.

Pinning status (what fixes each function independently of this file):
  data_utils.*                      reference known answers (tests/golden/known_answers.py)
  dense mask, get_max_seq_length    reference known-answer matrices + per-element brute force
  masked_softmax                    torch.softmax closed form + row-sum / exact-zero invariants
  multi_head_attention (fwd, bwd)   F.scaled_dot_product_attention, triple-loop brute force,
                                    fp64 gradcheck, and the reference-held layer golden
                                    (tests/golden/backward_compatibility/*.pt)
  rotary / rotary_complex           textbook closed form, reference invariants, relative-position
                                    property, orthogonality; the layer golden
  rms_norm                          F.rms_norm; closed form
  layer_norm, gelu mlp              F.layer_norm / F.gelu; the layer golden
  swiglu (+ closed-form gradient)   F.silu; autograd vs closed form
  transformer layer, final norm     the layer golden (all 8 intermediate activations)
  cached decode                     cached == uncached invariant
  token_losses, cross_entropy_loss  F.cross_entropy (library routine), closed forms (uniform logits -> log V,
                                    gradient = softmax - onehot, rows of the gradient sum to 0), fp64 gradcheck
No function is "parity unpinned".
"""

from .data_utils import (  # noqa: F401
    add_cumulative_seq_lengths_padding,
    get_cumulative_seq_lengths,
    get_position_ids,
    remove_cumulative_seq_lengths_padding,
)
from .attention import (  # noqa: F401
    cumulative_seq_lengths_to_dense_attention_mask,
    get_max_seq_length,
    masked_softmax,
    multi_head_attention,
    repeat_kv,
)
from .rotary import RotaryTables, apply_rotary, apply_rotary_complex, rotary_tables  # noqa: F401
from .norm import layer_norm, rms_norm  # noqa: F401
from .loss import cross_entropy_loss, lm_head, token_losses  # noqa: F401
from .mlp import gelu_mlp, swiglu, swiglu_grad, swiglu_mlp  # noqa: F401
from .layer import (  # noqa: F401
    LayerSpec,
    attention_block,
    final_norm,
    generate_cached,
    generate_uncached,
    mlp_block,
    self_attention,
    transformer_layer,
)

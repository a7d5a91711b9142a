"""CPU oracle for the fused attention forward path.  TEST INFRASTRUCTURE, NOT PRODUCT CODE.

This package restates, in plain eager PyTorch (fp32 unless the caller passes another dtype), what the reference's
attention_variants/*.py compute.  It is the checker for the HIP kernels: only tests/, __graft_entry__.smoke() and
the `cpu_baseline` leg of bench.py may import it.  flashlight_amd/ never does.

How each function is pinned (tests/test_oracle_pinned.py) without running the reference:
  vanilla / GQA      torch.nn.functional.scaled_dot_product_attention; pure-Python triple loop at S <= 12
  causal             SDPA is_causal=True; row 0 equals value[0]
  sliding window     SDPA with a loop-built boolean mask; W >= S-1 == causal; W == 0 returns value
  prefix-LM          SDPA with a loop-built mask; P <= 1 == causal; P >= S == vanilla
  document mask      SDPA with a loop-built mask; equals independent attention per document
  ALiBi              SDPA with a loop-built float mask; zero slopes == vanilla
  softcap            pure-Python loop with math.tanh; cap -> inf == vanilla
  diff-attn          difference of two SDPA calls; lambda = 0 == branch 0; equal branches == (1 - lambda) * SDPA
  Evoformer          SDPA on transposed inputs with the summed bias as float mask; zero bias == vanilla
  gate               elementwise sigmoid written with math.exp in a loop
  dense score_mod    SDPA with the callable's tensor as float mask (with and without GQA)
  IPA                pure-Python loops over queries, keys and points with math.exp at N <= 6; zero points == SDPA with
                     the pair bias as float mask; a common translation of query and key points changes nothing;
                     two keys at distances d1, d2 get weights in the ratio exp(w (d1^2 - d2^2))
  dropout            (oracle/dropout.py; the reference ignores dropout_p) all kept == SDPA; the 1 / (1 - p) factor against
                     torch.nn.functional.dropout; mean over 400 seeds approaches the undropped result; the keep decisions
                     against a second restatement in plain Python integers, frozen values and correlation statistics;
                     gradients by central differences (tests/test_dropout.py)
The committed fixtures under tests/golden/ were produced by tests/golden/make_golden.py from those library
routines (never from this package), so they pin it from outside as well.
"""
from .attention import (  # noqa: F401
    alibi_slopes,
    attention_alibi,
    attention_causal,
    attention_document_mask,
    attention_evoformer,
    attention_prefix_lm,
    attention_sliding_window,
    attention_softcapped,
    attention_vanilla,
    attention_vanilla_nogqa,
    diff_attention,
    invariant_point_attention,
    tanh_softcap,
)
from .masks import (  # noqa: F401
    attend_matrix,
    attended_pairs,
    document_lengths_cfg3,
    document_ids_from_lengths,
)

"""How each golden case is evaluated by (a) the oracle and (b) the HIP front-end.  Shared by CPU and GPU tests."""
from __future__ import annotations


def oracle_call(name: str, t: dict, meta: dict):
    import oracle as O
    q, k, v = t["q"], t["k"], t["v"]
    if name == "vanilla_gqa":
        return O.attention_vanilla(q, k, v, enable_gqa=True)
    if name == "causal":
        return O.attention_causal(q, k, v)
    if name == "sliding":
        return O.attention_sliding_window(q, k, v, window_size=int(meta["window"]))
    if name == "prefix_lm":
        return O.attention_prefix_lm(q, k, v, prefix_lengths=int(meta["prefix"]))
    if name.startswith("document_causal"):
        return O.attention_document_mask(q, k, v, t["document_id"], is_causal=True)
    if name.startswith("document"):
        return O.attention_document_mask(q, k, v, t["document_id"])
    if name == "alibi_gqa":
        return O.attention_alibi(q, k, v, score_mod=q.size(1), enable_gqa=True).flatten(1, 2)
    if name == "softcap":
        return O.attention_softcapped(q, k, v, score_mod=meta["cap"], scale=meta["scale"])
    if name == "alibi_softcap_causal_gqa":
        return O.attention_alibi(q, k, v, score_mod=q.size(1), is_causal=True, honor_causal=True, enable_gqa=True,
                                 softcap=meta["cap"]).flatten(1, 2)
    if name == "diff_attn":
        return O.diff_attention(q, k, v, lambda_full=meta["lambda_full"])
    if name == "diff_attn_causal":
        return O.diff_attention(q, k, v, lambda_full=meta["lambda_full"], is_causal=True)
    if name == "evoformer":
        return O.attention_evoformer(q, k, v, [t["bias1"], t["bias2"]])
    if name == "evoformer_gate":
        return O.attention_evoformer(q, k, v, [t["bias1"], t["bias2"]], gate=t["gate"])
    raise KeyError(name)


def hip_call(name: str, t: dict, meta: dict):
    import flashlight_amd.attention_variants as A
    q, k, v = t["q"], t["k"], t["v"]
    if name == "vanilla_gqa":
        return A.attention_pytorch(q, k, v, enable_gqa=True)
    if name == "causal":
        return A.attention_pytorch_causal(q, k, v)
    if name == "sliding":
        return A.attention_pytorch_sliding_window(q, k, v, window_size=int(meta["window"]))
    if name == "prefix_lm":
        return A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=int(meta["prefix"]))
    if name.startswith("document_causal"):
        return A.attention_pytorch_document_mask(q, k, v, t["document_id"], is_causal=True)
    if name.startswith("document"):
        return A.attention_pytorch_document_mask(q, k, v, t["document_id"])
    if name == "alibi_gqa":
        return A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(q.size(1)),
                                         enable_gqa=True).flatten(1, 2)
    if name == "softcap":
        return A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(meta["cap"]), scale=meta["scale"])
    if name == "alibi_softcap_causal_gqa":
        return A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(q.size(1)), is_causal=True,
                                         enable_gqa=True, softcap=meta["cap"]).flatten(1, 2)
    if name == "diff_attn":
        return A.diffattn(q, k, v, lambda_full=meta["lambda_full"])
    if name == "diff_attn_causal":
        return A.diffattn(q, k, v, lambda_full=meta["lambda_full"], is_causal=True)
    if name == "evoformer":
        return A.attention_reference(q, k, v, [t["bias1"], t["bias2"]])
    if name == "evoformer_gate":
        return A.attention_reference(q, k, v, [t["bias1"], t["bias2"]], gate=t["gate"])
    raise KeyError(name)


GOLDEN_NAMES = ["vanilla_gqa", "causal", "sliding", "prefix_lm", "document_sorted", "document_causal_sorted",
                "document_mixed", "document_causal_mixed", "alibi_gqa", "softcap", "alibi_softcap_causal_gqa",
                "diff_attn", "diff_attn_causal", "evoformer", "evoformer_gate"]

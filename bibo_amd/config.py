"""MoE-relevant configuration fields, with the reference's names, defaults and derivations
(src/configuration_bibo.py:39-61,103-137,165-181).  Any object carrying these attributes, the
reference's own BiBoConfig included, can be handed to the modules in bibo_amd.moe instead."""
from __future__ import annotations

NORM_TOPK_MODES = ("sum", "softmax")


class BiBoMoEConfig:
    def __init__(self, hidden_size=768, intermediate_size=2304, moe_intermediate_size=None, num_experts_per_tok=6,
                 num_routed_experts=6, special_expert_pairs=1, pos_identity_expert=True, neg_identity_expert=True,
                 num_pos_identity_experts=None, num_neg_identity_experts=None, use_shared_expert=False,
                 shared_expert_type="mlp", num_shared_experts=1, norm_topk_prob="sum", bias_update_factor=None,
                 bias_update_threshold=8000, initializer_range=0.02, hidden_act="silu", kernel_size=3,
                 radial_p="sigmoid", expert_act="radial", **unused):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.num_experts_per_tok = num_experts_per_tok
        self.num_routed_experts = num_routed_experts
        self.special_expert_pairs = special_expert_pairs
        self.pos_identity_expert = pos_identity_expert
        self.neg_identity_expert = neg_identity_expert
        # per-sign counts default to the pair count when that sign is enabled (configuration_bibo.py:109-114)
        self.num_pos_identity_experts = (int(num_pos_identity_experts) if num_pos_identity_experts is not None
                                         else (special_expert_pairs if pos_identity_expert else 0))
        self.num_neg_identity_experts = (int(num_neg_identity_experts) if num_neg_identity_experts is not None
                                         else (special_expert_pairs if neg_identity_expert else 0))
        if self.num_pos_identity_experts < 0 or self.num_neg_identity_experts < 0:
            raise ValueError("identity expert counts must be >= 0")
        self.num_glu_experts = num_routed_experts - self.num_pos_identity_experts - self.num_neg_identity_experts
        self.use_shared_expert = use_shared_expert
        self.shared_expert_type = shared_expert_type
        self.num_shared_experts = num_shared_experts
        self.norm_topk_prob = "sum" if norm_topk_prob is True else norm_topk_prob      # configuration_bibo.py:126
        self.moe_intermediate_size = (moe_intermediate_size if moe_intermediate_size is not None
                                      else intermediate_size // num_experts_per_tok)    # configuration_bibo.py:130-133
        self.bias_update_factor = 0.4 if bias_update_factor is None else bias_update_factor
        self.bias_update_threshold = 8000 if bias_update_threshold is None else bias_update_threshold
        self.initializer_range = initializer_range
        self.hidden_act = hidden_act
        self.kernel_size = kernel_size          # causal Conv1d of the conv shared expert (configuration_bibo.py:56,124)
        # not fields of the reference's config: its harness keeps them in two module globals
        # (RADIAL_P / EXPERT_ACT, ablate/common/patches.py:53-69)
        self.radial_p = radial_p
        self.expert_act = expert_act
        if not 1 <= num_experts_per_tok <= num_routed_experts:
            raise ValueError(f"num_experts_per_tok ({num_experts_per_tok}) must be in "
                             f"[1, num_routed_experts={num_routed_experts}]")
        if self.num_glu_experts < 1:
            raise ValueError(f"num_routed_experts={num_routed_experts} leaves {self.num_glu_experts} GLU experts "
                             "after the +/-Identity specials; need at least 1")
        if self.norm_topk_prob and self.norm_topk_prob not in NORM_TOPK_MODES:
            raise ValueError(f"norm_topk_prob must be one of {NORM_TOPK_MODES} (or False), got {self.norm_topk_prob!r}")

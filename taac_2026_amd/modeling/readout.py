"""Readout modules of the token backbone (experiments/symbiosis/pooling.py:16-32, experiments/symbiosis/model.py:
215-222, 316-321), served by one kernel."""

from __future__ import annotations

import torch
from torch import nn

from taac_2026_amd.accelerators.readout import candidate_readout
from taac_2026_amd.modeling.normalization import RMSNorm


class CandidateClsPooler(nn.Module):
    """cls token | candidate token (or zeros) | masked mean of all tokens, then ``RMSNorm(3 * d_model)``.

    ``forward(tokens, batch)`` takes the reference's batch object (attributes ``cls_index``, ``candidate_index``,
    ``padding_mask``); ``token_norm`` optionally fuses the model's ``final_norm`` over the tokens in front."""

    def __init__(self, d_model: int, *, use_candidate_readout: bool) -> None:
        super().__init__()
        self.d_model = int(d_model)
        self.use_candidate_readout = bool(use_candidate_readout)
        self.output_dim = self.d_model * 3
        self.norm = RMSNorm(self.output_dim)

    def forward(self, tokens: torch.Tensor, batch, *, token_norm: RMSNorm | None = None) -> torch.Tensor:
        return candidate_readout(
            tokens, cls_index=int(batch.cls_index),
            candidate_index=int(batch.candidate_index) if self.use_candidate_readout else None,
            padding_mask=batch.padding_mask, token_norm_weight=None if token_norm is None else token_norm.weight,
            pool_norm_weight=self.norm.weight, eps=self.norm.eps)


class CandidateReadoutHead(nn.Module):
    """``final_norm`` + :class:`CandidateClsPooler` + ``Linear(3D, D) -> SiLU -> Linear(D, action_num)`` of
    ``PCVRSymbiosis`` as one module and one kernel launch. ``forward`` returns the logits, ``predict`` the pair
    ``(logits, embedding)`` like the model's methods of the same names."""

    def __init__(self, d_model: int, action_num: int = 1, *, use_candidate_readout: bool = True) -> None:
        super().__init__()
        self.final_norm = RMSNorm(d_model)
        self.pooler = CandidateClsPooler(d_model, use_candidate_readout=use_candidate_readout)
        self.classifier = nn.Sequential(nn.Linear(self.pooler.output_dim, d_model), nn.SiLU(), nn.Dropout(0.0),
                                        nn.Linear(d_model, action_num))

    def _run(self, tokens: torch.Tensor, batch, *, return_embedding: bool, sigmoid: bool = False):
        fc1, fc2 = self.classifier[0], self.classifier[3]
        return candidate_readout(
            tokens, cls_index=int(batch.cls_index),
            candidate_index=int(batch.candidate_index) if self.pooler.use_candidate_readout else None,
            padding_mask=batch.padding_mask, token_norm_weight=self.final_norm.weight,
            pool_norm_weight=self.pooler.norm.weight, eps=self.pooler.norm.eps, fc1_weight=fc1.weight, fc1_bias=fc1.bias,
            fc2_weight=fc2.weight, fc2_bias=fc2.bias, sigmoid=sigmoid, return_embedding=return_embedding)

    def forward(self, tokens: torch.Tensor, batch) -> torch.Tensor:
        return self._run(tokens, batch, return_embedding=False)

    def predict(self, tokens: torch.Tensor, batch) -> tuple[torch.Tensor, torch.Tensor]:
        return self._run(tokens, batch, return_embedding=True)


__all__ = ["CandidateClsPooler", "CandidateReadoutHead"]

"""The reference's own PyTorch fallbacks for the speculator operators, restated for the CPU baseline.

Test / measurement infrastructure like the rest of this package: nothing in the product imports it.  These are the
code paths the reference runs when its compiled operators are absent (USE_CUSTOM_OP false), in the tensors' own
16-bit type, as the reference would run them:

  speculator_ln_fallback   arctic_inference/vllm/spec_dec/arctic_speculator.py:92-99   (MLPSpeculatorLayerNorm.forward_fallback)
  sum_lstm_fallback        arctic_inference/vllm/spec_dec/arctic_speculator.py:784-806 (the LSTM branch of one speculator step)

They are pinned by tests/test_oracle_speculator.py against the C oracle (same formula, fp32 arithmetic) within the
path's tolerance; they are not bit-comparable to it because every intermediate here is rounded to bf16.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch


def speculator_ln_fallback(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                           eps: float) -> torch.Tensor:
    xf = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)      # :94
    out = xf.type_as(x)                                              # :95
    if weight is not None:                                           # :96-98 (scale then shift)
        out = weight * out
        out = out + bias
    return out


def sum_lstm_fallback(states_4d: torch.Tensor, z4_4d: torch.Tensor, prev_cell: torch.Tensor,
                      w_cell: Optional[torch.Tensor], b_cell: Optional[torch.Tensor], w_state: Optional[torch.Tensor],
                      b_state: Optional[torch.Tensor], alpha: float, eps_cell: float, eps_state: float,
                      use_fast_gelu: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    D = prev_cell.size(-1)
    act = torch.nn.GELU(approximate="tanh" if use_fast_gelu else "none")
    added = torch.add(states_4d, z4_4d, alpha=alpha)                                       # :785-787
    forget_input_output, cell_candidate = added.split([3 * D, D], dim=-1)                  # :789-790
    forget_gate, input_gate, output_gate = torch.sigmoid(forget_input_output).split([D, D, D], dim=-1)   # :791-794
    cell_candidate = act(speculator_ln_fallback(cell_candidate, w_cell, b_cell, eps_cell))   # :796-797
    cell_candidate = cell_candidate * input_gate                                           # :798
    cell = prev_cell * forget_gate                                                         # :800
    cell = cell + cell_candidate                                                           # :801
    state = act(speculator_ln_fallback(cell, w_state, b_state, eps_state)) * output_gate   # :803-805
    return state, cell

"""The description of one step's batch, on the host and on the device."""
from dataclasses import dataclass, field

import torch


@dataclass(frozen=True)
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""
    request: object
    tokens: tuple
    want: tuple = ()


@dataclass
class StepContext:
    """What parts see of a step.  Device tensors are int32.

    Rows are the step's tokens, packed request after request in entry order;
    ``cu_seqlens[s] .. cu_seqlens[s + 1]`` are the rows of sequence s.
    """
    n_tokens: int
    n_seqs: int
    n_logit_rows: int
    token_ids: torch.Tensor        # [N]
    positions: torch.Tensor        # [N] absolute position of each row
    row_seq: torch.Tensor          # [N] sequence index of each row
    cu_seqlens: torch.Tensor       # [S + 1]
    seq_starts: torch.Tensor       # [S] position of each sequence's first row (cached length before the step)
    seq_slots: torch.Tensor        # [S] state slot of each sequence's request
    logit_rows: torch.Tensor       # [M] rows whose logits are wanted
    single_rows: torch.Tensor      # rows that are alone in their sequence; None if every row is (max_query == 1)
    max_query: int                 # most rows of one sequence
    max_context: int               # largest position + 1
    host_cu_seqlens: list = field(default_factory=list)
    host_starts: list = field(default_factory=list)
    host_slots: list = field(default_factory=list)
    requests: list = field(default_factory=list)

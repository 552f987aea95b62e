"""Oracle for the vocab-parallel embedding, one rank's vocabulary slice. Test
infrastructure only (see oracle/__init__.py).

Reference statements followed (cubework/module/parallel_1d/module.py, VocabParallelEmbedding1D.forward;
parallel_2d/module.py:345-353 and parallel_3d/module.py:455-466 are the same statements):
  :443      input_mask = (input_ < vocab_start) | (input_ >= vocab_end)
  :445-446  masked_input = input_ - vocab_start; masked_input[input_mask] = 0
  :448-449  output_parallel = F.embedding(masked_input, weight, padding_idx)
  :452      output_parallel[input_mask, :] = 0
The reduce / reduce-scatter that follows (:454) sums the ranks' outputs. F.embedding is handed the
SHIFTED indices together with the UNSHIFTED padding_idx, so the row of the slice that gets no
gradient is `padding_idx` counted inside the slice; the restatement keeps that.
"""
import torch


def vocab_embedding_fwd(ids: torch.Tensor, weight: torch.Tensor, vocab_start: int) -> torch.Tensor:
    ids = ids.detach().to("cpu").to(torch.int64)
    w = weight.detach().to("cpu")
    vocab_end = vocab_start + w.shape[0]
    mask = (ids < vocab_start) | (ids >= vocab_end)
    masked = ids.clone() - vocab_start
    masked[mask] = 0
    out = w[masked].clone()
    out[mask, :] = 0
    return out


def vocab_embedding_bwd(ids: torch.Tensor, d_out: torch.Tensor, num_rows: int, vocab_start: int,
                        padding_idx=None) -> torch.Tensor:
    """fp32 gradient of the slice: scatter-add of the unmasked tokens' rows of d_out; masked tokens were
    overwritten with zeros after the lookup (:452), so nothing flows back through them."""
    ids = ids.detach().to("cpu").to(torch.int64).reshape(-1)
    g = d_out.detach().to("cpu").to(torch.float32).reshape(ids.numel(), -1)
    local = ids - vocab_start
    live = (local >= 0) & (local < num_rows)
    if padding_idx is not None:
        live &= local != padding_idx
    dw = torch.zeros((num_rows, g.shape[1]), dtype=torch.float32)
    dw.index_add_(0, local[live], g[live])
    return dw

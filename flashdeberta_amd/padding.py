"""Mask bookkeeping around the fused attention.

Counterpart of the reference's src/flashdeberta/padding.py (`_get_unpad_data` :79-88, `_upad_input`
:113-166, `pad_input` :30-44).  The reference gathers the real tokens into a packed [T, H, D]
tensor (with `.item()` host syncs) and scatters the result back.  Here the kernel reads the padded
[B, L, H, D] layout in place, given each row's first real token and its count, so nothing is
gathered, scattered or synchronised.  Callers that already hold packed [T, H, D] tensors pass
cu_seqlens to the operator instead.
"""
import torch


def key_padding_mask(attention_mask):
    """Reduce the masks DeBERTa passes around to a [B, L] bool key-validity mask.
    Accepts [B, L]; the encoder's outer-product mask [B, 1, L, L] (its diagonal is the token
    validity, transformers modeling_deberta_v2.py:601-608); or [B, L, L]."""
    m = attention_mask
    if m.dim() == 4:
        m = m[:, 0]
    if m.dim() == 3:
        m = m.diagonal(dim1=-2, dim2=-1)
    if m.dim() != 2:
        raise ValueError("attention_mask must be [B, L], [B, L, L] or [B, 1, L, L]; got %s" % (tuple(attention_mask.shape),))
    return m.bool()


def seq_bounds(mask2d):
    """[B, L] bool -> (seq_start int32 [B], seq_len int32 [B], holes bool [B]) on the mask's device, no
    host sync.  The kernels take the real tokens of a row as one contiguous run (left or right padding).
    A row whose ones are not contiguous is flagged in `holes` and given seq_len -1, the kernels' mark for
    "write NaN": nothing is computed from a mask they cannot honour, and nothing passes for a result."""
    m = mask2d.to(torch.int32)
    L = m.shape[-1]
    count = m.sum(dim=-1, dtype=torch.int32)
    first = torch.argmax(m, dim=-1).to(torch.int32)  # first 1; 0 for an all-padding row
    last = (L - 1 - torch.argmax(m.flip(-1), dim=-1)).to(torch.int32)
    holes = (count > 0) & (last - first + 1 != count)
    return first, torch.where(holes, torch.full_like(count, -1), count), holes


def assert_contiguous_mask(attention_mask):
    """Raise ValueError if any row of the mask has masked tokens between real ones (one host sync);
    for callers that prefer an error to the NaN rows the module writes for such a mask."""
    _, _, holes = seq_bounds(key_padding_mask(attention_mask))
    if bool(holes.any()):
        raise ValueError("attention_mask rows %s have masked tokens between real ones; the fused attention takes "
                         "the real tokens of a row as one contiguous run" % holes.nonzero().flatten().tolist())

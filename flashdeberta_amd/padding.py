"""Mask bookkeeping around the fused attention.

Counterpart of the reference's src/flashdeberta/padding.py (`_get_unpad_data` :79-88, `_upad_input`
:113-166, `pad_input` :30-44).  The reference gathers the real tokens into a packed [T, H, D]
tensor (with `.item()` host syncs) and scatters the result back.  Here the kernel reads the padded
[B, L, H, D] layout in place, given each row's first real token and its count, so nothing is
gathered, scattered or synchronised; the packed helpers remain for callers that already hold
packed tensors.
"""
import torch
import torch.nn.functional as F


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
    A row whose ones are not contiguous is flagged in `holes` and given seq_len 0, so that nothing is
    computed from a mask the kernels cannot honour."""
    m = mask2d.to(torch.int32)
    L = m.shape[-1]
    count = m.sum(dim=-1, dtype=torch.int32)
    first = torch.argmax(m, dim=-1).to(torch.int32)  # first 1; 0 for an all-padding row
    last = (L - 1 - torch.argmax(m.flip(-1), dim=-1)).to(torch.int32)
    holes = (count > 0) & (last - first + 1 != count)
    return first, torch.where(holes, torch.zeros_like(count), count), holes


def assert_contiguous_mask(attention_mask):
    """Raise ValueError if any row of the mask has masked tokens between real ones (one host sync);
    for callers that prefer an error to the NaN rows the module writes for such a mask."""
    _, _, holes = seq_bounds(key_padding_mask(attention_mask))
    if bool(holes.any()):
        raise ValueError("attention_mask rows %s have masked tokens between real ones; the fused attention takes "
                         "the real tokens of a row as one contiguous run" % holes.nonzero().flatten().tolist())


def get_unpad_data(mask2d):
    """(indices of real tokens in the flattened [B*L] batch, cu_seqlens int32 [B+1], longest length).
    The longest length is returned as a 0-d tensor: turning it into a python int is the caller's
    choice (it is the only step that would synchronise)."""
    seqlens = mask2d.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(mask2d.flatten(), as_tuple=False).flatten()
    cu_seqlens = F.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))
    return indices, cu_seqlens, seqlens.max()


def unpad_input(x, indices):
    """x [B, L, ...] -> [T, ...] rows of the real tokens."""
    return x.reshape(-1, *x.shape[2:]).index_select(0, indices)


def pad_input(x, indices, batch, seqlen):
    """x [T, ...] -> [B, L, ...] with zeros in the padded rows."""
    out = torch.zeros((batch * seqlen,) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
    out.index_copy_(0, indices, x)
    return out.view(batch, seqlen, *x.shape[1:])

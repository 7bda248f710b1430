"""Host side of tk_get_fused_mapping; signature and return tuple follow
tile_kernels/moe/get_fused_mapping_kernel.py:166-250."""
import torch

from .. import _ffi


def get_fused_mapping(topk_idx: torch.Tensor, num_experts: int, num_expanded_tokens: int, alignment: int,
                      force_no_sync: bool = False):
    """Mappings between the (token, k) routing list and the expert-major expanded layout.

    ``num_expanded_tokens == 0`` (without ``force_no_sync``) sizes the buffers for the worst case, then
    trims them to the real padded length, which needs a host synchronisation.

    Returns ``(pos_to_expert, pos_to_token, pos_to_token_topk, token_topk_to_pos, expert_start, expert_end,
    num_tokens_per_expert, num_tokens_per_expert_list)``; the list is empty unless a sync happened.
    """
    num_tokens, num_topk = topk_idx.shape
    assert topk_idx.is_contiguous() and topk_idx.dtype == torch.int64
    dev = _ffi.require_gpu(topk_idx)
    lib = _ffi.load()

    should_sync = False
    if num_expanded_tokens == 0 and not force_no_sync:
        should_sync = True
        num_expanded_tokens = (num_tokens * num_topk + (alignment - 1) * num_experts) // alignment * alignment

    i32 = dict(dtype=torch.int32, device=dev)
    pos_to_expert = torch.empty((num_expanded_tokens,), **i32)
    pos_to_token = torch.empty((num_expanded_tokens,), **i32)
    pos_to_token_topk = torch.empty((num_expanded_tokens,), **i32)
    token_topk_to_pos = torch.empty((num_tokens, num_topk), **i32)
    expert_start = torch.empty((num_experts,), **i32)
    expert_end = torch.empty((num_experts,), **i32)
    num_tokens_per_expert = torch.empty((num_experts,), **i32)
    ws_bytes = lib.tk_fused_mapping_workspace_bytes(num_tokens, num_topk, num_experts)
    workspace = torch.empty((max(ws_bytes, 4) // 4,), **i32)

    with _ffi.on_device(dev):
        rc = lib.tk_get_fused_mapping(
            topk_idx.data_ptr(), num_tokens, num_topk, num_experts, alignment, num_expanded_tokens,
            pos_to_expert.data_ptr(), pos_to_token.data_ptr(), pos_to_token_topk.data_ptr(), token_topk_to_pos.data_ptr(),
            expert_start.data_ptr(), expert_end.data_ptr(), num_tokens_per_expert.data_ptr(),
            workspace.data_ptr(), workspace.numel() * 4, _ffi.current_stream(dev))
    _ffi.check(rc, 'tk_get_fused_mapping')

    num_tokens_per_expert_list = []
    if should_sync:
        num_tokens_per_expert_list = num_tokens_per_expert.tolist()
        n = sum(num_tokens_per_expert_list)
        pos_to_expert, pos_to_token, pos_to_token_topk = pos_to_expert[:n], pos_to_token[:n], pos_to_token_topk[:n]
    return (pos_to_expert, pos_to_token, pos_to_token_topk, token_topk_to_pos, expert_start, expert_end,
            num_tokens_per_expert, num_tokens_per_expert_list)

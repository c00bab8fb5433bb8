"""The allocation-free sparse map (`fm_sparse_map_static`) against `fm_sparse_map`, both through the C ABI: same
bits, on two calls in a row (the second on a smaller input, so that stale scratch content would show), and the
refusal of inputs whose scratch does not fit the fixed array."""

import pytest
import torch

from fast_llm_amd import _lib
from oracle import moe_oracle

pytestmark = pytest.mark.gpu


def _maps(library, device, top_experts: torch.Tensor, num_experts: int, static: bool):
    tokens, k = top_experts.shape
    rows = (tokens * k + num_experts * 128) // 128 * 128
    index_dtype = torch.int16 if rows < 32768 else torch.int32
    # Outputs pre-filled so that an entry the kernels fail to write cannot pass by accident.
    sparse_rows = torch.full((tokens, k), -7, dtype=index_dtype, device=device)
    expert_ends = torch.full((num_experts,), -7, dtype=index_dtype, device=device)
    expert_pad_begins = torch.full((num_experts,), -7, dtype=index_dtype, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    common = (top_experts.data_ptr(), tokens, k, num_experts, 128, _lib.index_tag(index_dtype), sparse_rows.data_ptr(),
              expert_ends.data_ptr(), expert_pad_begins.data_ptr())  # fmt: skip
    if static:
        status = library.fm_sparse_map_static(*common, stream)
    else:
        size = library.fm_sparse_map_workspace_size(tokens, k, num_experts)
        workspace = torch.empty(size, dtype=torch.uint8, device=device)
        status = library.fm_sparse_map(*common, workspace.data_ptr(), size, stream)
    _lib.check(status)
    torch.cuda.synchronize(device)
    return sparse_rows, expert_ends, expert_pad_begins


def test_static_sparse_map_matches_the_workspace_entry_point(library, device):
    generator = torch.Generator().manual_seed(3)
    # The wide benchmark shape first, then a much smaller input with other expert and slot counts.
    for tokens, num_experts, k in ((16384, 128, 8), (777, 6, 2)):
        logits = torch.randn(tokens, num_experts, generator=generator)
        top_experts = torch.topk(logits, k, dim=-1).indices.to(device)
        expected = _maps(library, device, top_experts, num_experts, static=False)
        results = _maps(library, device, top_experts, num_experts, static=True)
        for ours, theirs in zip(results, expected):
            assert ours.dtype == theirs.dtype and torch.equal(ours, theirs)
        oracle_map = moe_oracle.sparse_map(top_experts.cpu(), num_experts)
        assert torch.equal(results[0].cpu().long(), oracle_map.sparse_rows)
        assert torch.equal(results[1].cpu().long(), oracle_map.expert_ends)
        assert torch.equal(results[2].cpu().long(), oracle_map.expert_pad_begins)

    # Free device memory as the driver sees it does not move over a call (outputs allocated beforehand).
    tokens, k = top_experts.shape
    outputs = [torch.empty(n, dtype=torch.int16, device=device) for n in (tokens * k, num_experts, num_experts)]
    torch.cuda.synchronize(device)
    free_before = torch.cuda.mem_get_info(device)[0]
    status = library.fm_sparse_map_static(
        top_experts.data_ptr(), tokens, k, num_experts, 128, _lib.index_tag(torch.int16), *(t.data_ptr() for t in outputs),
        torch.cuda.current_stream(device).cuda_stream,
    )  # fmt: skip
    _lib.check(status)
    torch.cuda.synchronize(device)
    assert torch.cuda.mem_get_info(device)[0] == free_before
    assert torch.equal(outputs[0].view(tokens, k), results[0])


def test_static_sparse_map_refuses_what_does_not_fit(library, device):
    assert library.fm_sparse_map_static_scratch_size() == 1 << 20
    tokens, k, num_experts = 1 << 18, 8, 1024  # 2048 workgroups x 1024 experts x 4 bytes = 8 MiB of counts
    assert library.fm_sparse_map_workspace_size(tokens, k, num_experts) > library.fm_sparse_map_static_scratch_size()
    fake = 256  # non-null pointers that must never be dereferenced
    status = library.fm_sparse_map_static(fake, tokens, k, num_experts, 128, 1, fake, fake, fake, None)
    assert status == _lib.FM_ERR_UNSUPPORTED
    message = library.fm_last_error().decode()
    assert "scratch" in message and "fm_sparse_map" in message
    with pytest.raises(NotImplementedError):
        _lib.check(status)

"""gmm_moe_route_noalloc (the routing entry point that allocates nothing: its histogram table is a static
device array) against gmm_moe_route with a caller workspace, through the C ABI: two calls in a row, the
second on a smaller problem, every output bit for bit; sizes beyond the built-in table are refused."""
import pytest
import torch

from grouped_mm_bf16_amd import _lib
from oracle import moe_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def route(entry: str, logits: torch.Tensor, k: int, renorm: int):
    lib = _lib.load()
    T, E = logits.shape
    S = T * k
    outs = [torch.full((E,), -7, device=DEV, dtype=torch.int32), torch.full((S,), -7, device=DEV, dtype=torch.int32),
            torch.full((S,), -7.0, device=DEV, dtype=torch.float32), torch.full((S,), -7, device=DEV, dtype=torch.int32),
            torch.full((S,), -7, device=DEV, dtype=torch.int32)]
    head = [logits.data_ptr(), logits.stride(0), _lib.DT_F32, T, E, k, renorm] + [o.data_ptr() for o in outs]
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "workspace":
        need = lib.gmm_moe_route_workspace_bytes(T, E, k)
        ws = torch.empty(max(need, 4) // 4, device=DEV, dtype=torch.int32)
        rc = lib.gmm_moe_route(*head, ws.data_ptr(), need, stream)
    else:
        rc = lib.gmm_moe_route_noalloc(*head, stream)
    torch.cuda.synchronize()
    return rc, outs


def test_two_calls_in_a_row_match_the_workspace_entry_point():
    gen = torch.Generator().manual_seed(123)
    # first a problem that fills most of the table (200 workgroups x 256 experts), then a smaller one with
    # other sizes: what the first call left in the table must not show in the second
    for T, E, k, renorm in [(25600, 256, 8, 1), (1500, 37, 3, 0)]:
        logits = torch.randn(T, E, generator=gen).to(DEV)
        rc_w, want = route("workspace", logits, k, renorm)
        rc_n, got = route("noalloc", logits, k, renorm)
        assert rc_w == 0 and rc_n == 0
        for name, g, w in zip(("offs", "slot_expert", "slot_weight", "row_token", "token_rows"), got, want):
            assert torch.equal(g, w), name
        assert int(got[0][-1]) == T * k and sorted(got[4].tolist()) == list(range(T * k))
        # and against the oracle, so that a mistake both entry points share does not pass
        ref = moe_oracle.route(logits.cpu(), k, bool(renorm))
        assert torch.equal(got[0].cpu(), ref.offs) and torch.equal(got[1].cpu(), ref.slot_expert)
        assert torch.equal(got[3].cpu(), ref.row_token) and torch.equal(got[4].cpu(), ref.token_rows)
        torch.testing.assert_close(got[2].cpu(), ref.slot_weight, rtol=2e-5, atol=1e-7)


def test_sizes_beyond_the_built_in_table_are_refused():
    lib = _lib.load()
    T, E, k = 20000, 1023, 8                      # 157 workgroups x 1023 experts x 4 bytes > 256 KiB
    assert lib.gmm_moe_route_workspace_bytes(T, E, k) > 262144
    logits = torch.zeros(T, E, device=DEV)
    rc, outs = route("noalloc", logits, k, 1)
    assert rc == 4 and b"workspace" in lib.gmm_status_string(rc)
    assert all((o == -7).all() for o in outs), "a refused call must not write"
    rc, _ = route("workspace", logits, k, 1)      # the same problem with a workspace is fine
    assert rc == 0

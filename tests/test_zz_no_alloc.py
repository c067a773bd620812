"""The allocation-free greedy-sampling entry point, tllm_unembedding_argmax_noalloc_bf16, against the entry point it is a
variant of (tllm_unembedding_argmax_bf16 with a caller's workspace): same token ids, bit for bit, on two calls in a row --
the second with a smaller input, so that whatever the first call left in the library-owned scratch array must not leak
into it -- and no device memory taken from PyTorch's allocator by the call. Raw C ABI throughout."""
import pytest
import torch

from oracle import layers as O
from tritonllm_amd import _lib

pytestmark = pytest.mark.gpu


def _argmax_pair(gpu, rows, vocab, hidden, seed, fp8=False):
    L = _lib.lib()
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, hidden, generator=g).bfloat16().to(gpu)
    w = (0.02 * torch.randn(vocab, hidden, generator=g)).bfloat16()
    if fp8:
        w8, ws = O.quantize_fp8_rows_ref(w)
        wd, wsd = w8.to(gpu), ws.to(gpu)
        logits_ref = O.linear_ref(x.cpu(), O.dequant_fp8_ref(w8, ws).bfloat16(), None)
    else:
        wd, wsd = w.to(gpu), None
        logits_ref = O.linear_ref(x.cpu(), w, None)
    stream = torch.cuda.current_stream().cuda_stream
    wsp = wsd.data_ptr() if wsd is not None else None
    # the existing entry point, with a caller-provided workspace
    nbytes = L.tllm_unembedding_argmax_workspace_bytes(rows)
    work = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
    ids_ws = torch.full((rows,), -1, dtype=torch.int32, device=gpu)
    rc = L.tllm_unembedding_argmax_bf16(x.data_ptr(), wd.data_ptr(), wsp, work.data_ptr(), nbytes, ids_ws.data_ptr(), rows, hidden, vocab, stream)
    assert rc == 0, L.tllm_last_error()
    # the allocation-free one: outputs exist before the call, nothing may be allocated during it
    ids_na = torch.full((rows,), -1, dtype=torch.int32, device=gpu)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(gpu)["allocation.all.allocated"], torch.cuda.memory_reserved(gpu)
    rc = L.tllm_unembedding_argmax_noalloc_bf16(x.data_ptr(), wd.data_ptr(), wsp, ids_na.data_ptr(), rows, hidden, vocab, stream)
    assert rc == 0, L.tllm_last_error()
    torch.cuda.synchronize()
    after = torch.cuda.memory_stats(gpu)["allocation.all.allocated"], torch.cuda.memory_reserved(gpu)
    assert before == after, "the allocation-free entry point went through PyTorch's allocator"
    assert torch.equal(ids_na, ids_ws), (ids_na.tolist(), ids_ws.tolist())
    # and both name a maximum of the oracle's logits (a rival within rounding distance of the best is also right)
    ids = ids_na.cpu().long()
    assert ((ids >= 0) & (ids < vocab)).all()
    best = logits_ref.max(dim=1).values
    got = logits_ref.gather(1, ids[:, None])[:, 0]
    assert (best - got <= 1e-3 * best.abs().clamp(min=1.0)).all(), (best, got)
    return ids_na


def test_noalloc_argmax_matches_workspace_form_twice_in_a_row(gpu):
    L = _lib.lib()
    assert L.tllm_unembedding_argmax_noalloc_max_rows() == 16
    _argmax_pair(gpu, rows=16, vocab=20000, hidden=2880, seed=1)      # fills the scratch for 16 rows
    _argmax_pair(gpu, rows=3, vocab=3001, hidden=2880, seed=2)        # smaller input, ragged last tile: stale candidates must not win
    _argmax_pair(gpu, rows=8, vocab=5000, hidden=2880, seed=3, fp8=True)
    _argmax_pair(gpu, rows=1, vocab=4097, hidden=512, seed=4)


def test_noalloc_argmax_full_vocabulary_and_limits(gpu):
    L = _lib.lib()
    vocab, hidden, rows = O.VOCAB, O.HIDDEN, 8
    gg = torch.Generator(device=gpu).manual_seed(5)
    w = torch.empty(vocab, hidden, dtype=torch.bfloat16, device=gpu).normal_(0, 0.02, generator=gg)
    x = torch.empty(rows, hidden, dtype=torch.bfloat16, device=gpu).normal_(0, 1, generator=gg)
    plant = [0, 31, 4097, 100000, 150001, 201087, 77, 201056]
    for r, v in enumerate(plant):
        w[v] = (x[r].float() * 0.05).bfloat16()                          # a clear winner per row
    stream = torch.cuda.current_stream().cuda_stream
    ids = torch.full((rows,), -1, dtype=torch.int32, device=gpu)
    rc = L.tllm_unembedding_argmax_noalloc_bf16(x.data_ptr(), w.data_ptr(), None, ids.data_ptr(), rows, hidden, vocab, stream)
    assert rc == 0, L.tllm_last_error()
    assert ids.tolist() == plant
    nbytes = L.tllm_unembedding_argmax_workspace_bytes(rows)
    work = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
    ids2 = torch.full((rows,), -1, dtype=torch.int32, device=gpu)
    rc = L.tllm_unembedding_argmax_bf16(x.data_ptr(), w.data_ptr(), None, work.data_ptr(), nbytes, ids2.data_ptr(), rows, hidden, vocab, stream)
    assert rc == 0 and torch.equal(ids, ids2)
    # a smaller call right after the full-vocabulary one
    ids3 = torch.full((2,), -1, dtype=torch.int32, device=gpu)
    rc = L.tllm_unembedding_argmax_noalloc_bf16(x.data_ptr(), w.data_ptr(), None, ids3.data_ptr(), 2, hidden, 4096, stream)
    assert rc == 0
    want = O.linear_ref(x[:2].cpu(), w[:4096].cpu(), None).argmax(dim=1)
    assert ids3.cpu().long().tolist() == want.tolist()
    # beyond the scratch: refused with a message, nothing launched
    big = torch.zeros(17, hidden, dtype=torch.bfloat16, device=gpu)
    ids17 = torch.zeros(17, dtype=torch.int32, device=gpu)
    rc = L.tllm_unembedding_argmax_noalloc_bf16(big.data_ptr(), w.data_ptr(), None, ids17.data_ptr(), 17, hidden, vocab, stream)
    assert rc == -2 and b"at most 16 rows" in L.tllm_last_error()
    assert L.tllm_unembedding_argmax_noalloc_bf16(x.data_ptr(), w.data_ptr(), None, None, rows, hidden, vocab, stream) == -1
    assert L.tllm_unembedding_argmax_noalloc_bf16(None, None, None, None, 0, hidden, vocab, stream) == 0


def test_noalloc_argmax_replays_in_a_captured_graph(gpu):
    """The use the entry point is for: after the per-device set-up call, the launch is captured in a HIP graph and
    replayed with new activations; every replay must give the token ids of the workspace form on the same input."""
    L = _lib.lib()
    assert L.tllm_unembedding_argmax_noalloc_init() == 0, L.tllm_last_error()
    rows, vocab, hidden = 8, 6001, O.HIDDEN
    g = torch.Generator().manual_seed(11)
    w = (0.02 * torch.randn(vocab, hidden, generator=g)).bfloat16().to(gpu)
    xs = [torch.randn(rows, hidden, generator=g).bfloat16().to(gpu) for _ in range(3)]
    x = xs[0].clone()
    ids = torch.full((rows,), -1, dtype=torch.int32, device=gpu)
    nbytes = L.tllm_unembedding_argmax_workspace_bytes(rows)
    work = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
    ids_ws = torch.full((rows,), -1, dtype=torch.int32, device=gpu)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = L.tllm_unembedding_argmax_noalloc_bf16(x.data_ptr(), w.data_ptr(), None, ids.data_ptr(), rows, hidden, vocab,
                                                        torch.cuda.current_stream().cuda_stream)
    assert rc == 0, L.tllm_last_error()
    torch.cuda.current_stream().wait_stream(side)
    for xi in xs[1:] + xs[:1]:
        x.copy_(xi)
        ids.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        rc = L.tllm_unembedding_argmax_bf16(xi.data_ptr(), w.data_ptr(), None, work.data_ptr(), nbytes, ids_ws.data_ptr(), rows, hidden, vocab,
                                            torch.cuda.current_stream().cuda_stream)
        assert rc == 0, L.tllm_last_error()
        torch.cuda.synchronize()
        assert torch.equal(ids, ids_ws), (ids.tolist(), ids_ws.tolist())
        want = O.linear_ref(xi.cpu(), w.cpu(), None)
        got = want.gather(1, ids.cpu().long()[:, None])[:, 0]
        assert (want.max(dim=1).values - got <= 1e-3).all()

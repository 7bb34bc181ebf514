"""Weights kept in tiles for the products of few rows: the layout itself, the embedding lookup from it,
what is refused, and whole tiny models whose every matrix is packed against the plain implementation.
(The products on packed weights are tested next to the others in test_kernels_gpu.py.)"""
import pytest
import torch

from conftest import TINY, WHOLE_ROTATION, make_folder
from helpers import assert_logits, first_bad_position, run_batched, run_tail_decoded, run_whole, token_ids
import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from xeno_rt_amd.ops import load_ops
    return load_ops()


def matrix(rows, cols, seed):
    return torch.randn(rows, cols, generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16).to(DEV)


def place(row, k, cols):
    """Element offset of (packed row, column k): groups of 16 rows, tiles of 32 columns one after another along k,
    inside a tile the pieces of 8 columns of one row at place row % 16 + 16 * (k % 32 // 8)."""
    return ((row // 16) * (cols // 32) + k // 32) * 512 + ((k % 32 // 8) * 16 + row % 16) * 8 + k % 8


@pytest.mark.parametrize("rows,cols", [(16, 32), (50, 96), (384, 256), (129, 64)])
def test_layout_of_plain_tiles(ops, rows, cols):
    w = matrix(rows, cols, rows)
    packed = ops.pack(w, "tiles")
    assert packed.shape == (rows, cols) and packed.data.numel() == (rows + 15) // 16 * 16 * cols
    flat = packed.data.cpu()
    for row, k in ((0, 0), (rows - 1, cols - 1), (rows // 2, 9), (7, 31), (15, cols - 8), (rows - 1, 0)):
        assert flat[place(row, k, cols)] == w[row, k].cpu(), (row, k)
    padded = (rows + 15) // 16 * 16
    for row in range(rows, padded):                       # rows beyond the matrix hold zeros
        assert float(flat[place(row, 5, cols)]) == 0.0
    assert torch.equal(packed.unpacked(), w)


def test_layout_pairs_gate_with_up_rows_and_the_halves_of_rotated_heads(ops):
    n, cols = 40, 64
    w = matrix(2 * n, cols, 1)
    packed = ops.pack(w, "gated", gated_n=n)
    flat = packed.data.cpu()
    for j in (0, 7, 8, 23, 39):                            # output j: gate row j, up row n + j, eight places apart in one group
        assert flat[place(j // 8 * 16 + j % 8, 3, cols)] == w[j, 3].cpu()
        assert flat[place(j // 8 * 16 + 8 + j % 8, 3, cols)] == w[n + j, 3].cpu()
    assert torch.equal(packed.unpacked(), w)
    heads, rotated, hd = 5, 3, 48                          # three rotated heads, two that keep their order
    w = matrix(heads * hd, cols, 2)
    packed = ops.pack(w, "rotary", head_dim=hd, rotated_heads=rotated)
    flat = packed.data.cpu()
    for head, d in ((0, 0), (1, 7), (2, 8), (2, 23), (0, 24), (1, 31), (2, 47)):
        half, within = d // (hd // 2), d % (hd // 2)
        row = head * hd + within // 8 * 16 + half * 8 + within % 8
        assert flat[place(row, 40, cols)] == w[head * hd + d, 40].cpu(), (head, d)
    for head, d in ((3, 0), (3, 30), (4, 47)):
        assert flat[place(head * hd + d, 40, cols)] == w[head * hd + d, 40].cpu()
    assert torch.equal(packed.unpacked(), w)


def test_embedding_lookup_from_a_packed_table(ops):
    table = matrix(777, 96, 3)
    ids = torch.tensor([0, 776, 5, 5, 123, 16, 15], dtype=torch.int32, device=DEV)
    out = torch.empty(7, 96, device=DEV)
    ops.embed(ops.pack(table, "tiles"), ids, out)
    assert torch.equal(out, table[ids.long()].float())


def test_what_does_not_fit_is_refused(ops):
    from xeno_rt_amd.ops.hip import KernelError
    with pytest.raises(KernelError, match="multiple of 32"):
        ops.pack(matrix(32, 40, 1), "tiles")
    with pytest.raises(KernelError, match="multiple of 8"):
        ops.pack(matrix(2 * 12, 64, 1), "gated", gated_n=12)
    with pytest.raises(KernelError, match="heads"):
        ops.pack(matrix(100, 64, 1), "rotary", head_dim=48, rotated_heads=1)
    a = matrix(4, 64, 2)
    gated = ops.pack(matrix(2 * 16, 64, 1), "gated", gated_n=16)
    with pytest.raises(KernelError, match="gated product"):
        ops.linear(a, gated, torch.empty(4, 32, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError, match="gated product"):
        ops.linear_glu(a, ops.pack(matrix(2 * 16, 64, 1), "tiles"), torch.empty(4, 16, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError):                       # an embedding table with its rows regrouped
        ops.embed(gated, torch.zeros(1, dtype=torch.int32, device=DEV), torch.empty(1, 64, device=DEV))
    # the library's own advice: whole rounds over the compute units or many of them, and small matrices
    assert ops.packing_suits(4096, 4096) and ops.packing_suits(28672, 4096) and ops.packing_suits(128256, 4096)
    assert ops.packing_suits(6144, 4096) and ops.packing_suits(64, 64)
    assert not ops.packing_suits(5120, 5120) and not ops.packing_suits(2048, 4096) and not ops.packing_suits(4096, 100)


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """Tiny models whose widths are multiples of 32, so that every matrix can be packed: name -> (folder, plain model)."""
    out = {}
    for name, changes in (("llama", dict(intermediate_size=160, head_dim=32)), ("qwen3", dict(WHOLE_ROTATION))):
        raw = dict(TINY[name], **changes)
        folder = make_folder(raw, tmp_path_factory.mktemp(f"packed_{name}"), seed=61 if name == "llama" else 67, std=0.2)
        out[name] = (folder, P.PlainModel(folder))
    return out


@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_models_with_every_matrix_packed(name, models):
    """Whole, with the last tokens one by one, and in unequal batches through reused slots: the logits of a
    model whose matrices are all packed against the plain model, and next to those of the same model unpacked."""
    from xeno_rt_amd.engine import Engine
    folder, plain = models[name]
    packed = Engine.load(folder, dtype="bfloat16", max_tokens=64 * 8, max_slots=3, pack_weights="always")
    rows_along_k = Engine.load(folder, dtype="bfloat16", max_tokens=64 * 8, max_slots=3, pack_weights=False)
    layer = packed.model.spec.layers[-1]
    for weight in (layer.mixer.w_qkv, layer.mixer.w_o, layer.feed_forward.w_gate_up, layer.feed_forward.w_down,
                   packed.model.spec.head.weight):
        assert hasattr(weight, "unpacked")
    assert not hasattr(rows_along_k.model.spec.layers[-1].mixer.w_qkv, "unpacked")
    if plain.config.tied:
        assert packed.model.spec.embedding.table is packed.model.spec.head.weight
    vocab = plain.config.vocab_size
    requests = [token_ids(vocab, n, seed=n) for n in (1, 9, 64, 65, 100, 17)]
    wants = [plain.logits(ids) for ids in requests]
    for ids, want in zip(requests, wants):
        for what, run in (("whole", run_whole), ("tail decoded", run_tail_decoded)):
            got = run(packed, ids)
            assert_logits(got, want, "bfloat16", f"{name} packed, {what}, {len(ids)} tokens, first bad row {first_bad_position(got, want, 'bfloat16')}")
            assert_logits(got, run(rows_along_k, ids), "bfloat16", f"{name} packed against unpacked, {what}")
    for batch in ([0, 1, 2], [3, 4, 5], [2, 5, 0]):
        got = run_batched(packed, [requests[i] for i in batch], [max(1, len(requests[i]) - 2 - 3 * j) for j, i in enumerate(batch)])
        for i, logits in zip(batch, got):
            assert_logits(logits, wants[i], "bfloat16", f"{name} packed, batch {batch}, request {i}")
        packed.cache.check()
        assert packed.cache.slots.n_held == 0 and packed.cache.held_blocks() == 0

"""Synthetic token batches (reference src/olmax/data/utils.py:12-66): the device generator must be
bit-exact against the oracle's integer closed form, including the label == V quirk, and the
loader must honour the benchmark's (key, batches_processed, epoch) state protocol
(src/integration_tests/train_transformer.py:50-99; shapes as src/test/data/utils_test.py:7-22)."""
import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu


def test_sequential_tokens_bit_exact_and_label_quirk():
    from olmax_amd import data
    V, S = 1000, 257
    off = torch.tensor([0, 1, 998, 742, 999 - 256, 500], dtype=torch.int32)
    inp, tgt = data.sequential_tokens(off.cuda(), S, V)
    winp, wtgt = ref.sequential_tokens(off, S, V)
    assert inp.dtype == torch.int32 and torch.equal(inp.cpu(), winp) and torch.equal(tgt.cpu(), wtgt)
    # a target equals V exactly where the input is V - 1, and nowhere else leaves [1, V]
    assert torch.equal(tgt.cpu() == V, inp.cpu() == V - 1) and int(tgt.min()) >= 1 and int(tgt.max()) <= V
    assert (inp.cpu() == V - 1).any()


def test_full_size_batch_properties():
    from olmax_amd import data
    V, S, B = 100352, 4096, 2
    off = data.start_offsets(0, 0, 0, 0, B, V)
    assert off.shape == (B,) and int(off.min()) >= 0 and int(off.max()) < V - 1
    inp, tgt = data.sequential_tokens(off.cuda(), S, V)
    assert inp.shape == (B, S)
    d = (inp[:, 1:] - inp[:, :-1]).cpu()
    assert ((d == 1) | (d == 1 - V)).all() and torch.equal(inp[:, 0].cpu(), off)
    assert torch.equal(tgt, inp + 1)


def test_loader_shapes_state_and_resume():
    from olmax_amd import data
    kw = dict(vocab_size=128, sequence_length=16, global_batch_size_instances=8, total_batches=4, num_microbatches=2)
    dl = data.DataLoader(7, **kw)
    batches = list(dl)
    assert len(batches) == 4 and all(len(b) == 2 for b in batches)
    assert all(x.shape == (4, 16) and y.shape == (4, 16) for b in batches for x, y in b)
    assert dl.get_state() == (7, 0, 1)  # one epoch consumed
    # resume in the middle of an epoch reproduces the remaining batches exactly
    dl2 = data.DataLoader(7, **kw)
    it = iter(dl2)
    next(it); next(it)
    state = dl2.get_state()
    assert state == (7, 2, 0)
    dl3 = data.DataLoader(0, **kw)
    dl3.load_state(state)
    rest = list(dl3)
    assert len(rest) == 2
    for got, want in zip(rest, batches[2:]):
        for (gx, gy), (wx, wy) in zip(got, want):
            assert torch.equal(gx, wx) and torch.equal(gy, wy)
    with pytest.raises(ValueError):
        next(data.generate_batches_of_sequential_tokens(0, vocab_size=8, sequence_length=4, global_batch_size_instances=3,
                                                        total_batches=1, num_microbatches=2))

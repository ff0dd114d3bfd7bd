"""The index-yielding loader (behaviour of actnn/actnn/dataloader.py:385-390: `index, data`)."""
import pytest
import torch
from torch.utils.data import IterableDataset, TensorDataset

from actnn_amd.dataloader import DataLoader


def _dataset(n=23):
    x = torch.arange(n, dtype=torch.float32).view(n, 1) * 10
    y = torch.arange(n)
    return TensorDataset(x, y)


def test_sequential_batches_carry_their_indices():
    batches = list(DataLoader(_dataset(), batch_size=5))
    assert [idx for idx, _ in batches] == [list(range(i, min(i + 5, 23))) for i in range(0, 23, 5)]
    for idx, (x, y) in batches:
        assert y.tolist() == idx and x.view(-1).tolist() == [10.0 * i for i in idx]


@pytest.mark.parametrize("workers", [0, 2])
def test_shuffled_batches_with_and_without_workers(workers):
    gen = torch.Generator().manual_seed(3)
    loader = DataLoader(_dataset(), batch_size=4, shuffle=True, drop_last=True, num_workers=workers,
                        generator=gen)
    assert len(loader) == 5
    seen = []
    for idx, (x, y) in loader:
        assert len(idx) == 4 and y.tolist() == idx
        seen += idx
    assert len(set(seen)) == 20 and seen != sorted(seen)


def test_custom_collate_batch_sampler_and_unbatched():
    ds = _dataset(6)
    loader = DataLoader(ds, batch_sampler=[[4, 1], [0, 5, 2]], collate_fn=lambda s: len(s))
    assert list(loader) == [([4, 1], 2), ([0, 5, 2], 3)]
    single = list(DataLoader(ds, batch_size=None))
    assert [i for i, _ in single] == list(range(6)) and single[3][1][1].item() == 3
    assert DataLoader(ds, 2).dataset.tensors[1].tolist() == list(range(6))      # attributes pass through


def test_iterable_datasets_are_refused():
    class Stream(IterableDataset):
        def __iter__(self):
            return iter(range(3))
    with pytest.raises(TypeError):
        DataLoader(Stream())

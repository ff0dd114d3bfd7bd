"""A data loader that also yields the dataset indices of every batch.

Per-sample gradient statistics (config.use_gradient) are kept per dataset entry, so the training
loop has to tell the policy which entries a batch holds: ``QScheme.batch = indices``
(mem_speed_benchmark/train.py:358).  The reference ships a fork of torch's loader whose iterators
return ``index, data`` (actnn/actnn/dataloader.py:385-390, 998-1000).  Here the stock loader is
kept and the index travels with the sample instead: the dataset is wrapped so that entry ``i``
comes back as ``(i, dataset[i])`` and the collate step splits the two again.  That works unchanged
with worker processes, pinned memory, samplers and batch samplers.
"""
from torch.utils.data import DataLoader as _TorchDataLoader
from torch.utils.data import IterableDataset
from torch.utils.data.dataloader import default_collate


class _WithIndex:
    """Map-style view of a dataset whose entries carry their own index."""

    def __init__(self, dataset):
        self.dataset = dataset

    def __len__(self):
        return len(self.dataset)

    def __getitem__(self, i):
        return i, self.dataset[i]

    def __getattr__(self, name):                    # classes, transforms, ... of the wrapped dataset
        if name == "dataset":
            raise AttributeError(name)
        return getattr(self.dataset, name)


class _SplitIndices:
    """Collate function: [(i, sample), ...] -> ([i, ...], collate([sample, ...]))."""

    def __init__(self, collate_fn):
        self.collate_fn = collate_fn

    def __call__(self, entries):
        return [int(i) for i, _ in entries], self.collate_fn([sample for _, sample in entries])


class DataLoader(_TorchDataLoader):
    """torch.utils.data.DataLoader whose iterator yields ``(indices, batch)``: `indices` is the
    list of dataset indices in the order of the batch's samples (an int when automatic batching
    is off, i.e. ``batch_size=None``)."""

    def __init__(self, dataset, *args, **kwargs):
        if isinstance(dataset, IterableDataset):
            raise TypeError("an iterable-style dataset has no indices to yield")
        names = ("batch_size", "shuffle", "sampler", "batch_sampler", "num_workers", "collate_fn")
        kwargs.update(zip(names, args))
        if len(args) > len(names):
            raise TypeError("pass DataLoader arguments after collate_fn by keyword")
        batched = kwargs.get("batch_size", 1) is not None or kwargs.get("batch_sampler") is not None
        if batched:
            kwargs["collate_fn"] = _SplitIndices(kwargs.get("collate_fn") or default_collate)
        elif kwargs.get("collate_fn") is not None:
            inner = kwargs["collate_fn"]
            kwargs["collate_fn"] = lambda entry: (entry[0], inner(entry[1]))
        super().__init__(_WithIndex(dataset), **kwargs)

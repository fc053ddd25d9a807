from abc import ABC


class BaseIndexer(ABC):
    """Surface of the reference's indexer/base.py:5-10."""

    def build(self, keys, values):
        raise NotImplementedError

    def update(self, new_keys, values):
        raise NotImplementedError

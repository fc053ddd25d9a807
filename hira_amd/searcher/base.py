from abc import ABC


class BaseSearcher(ABC):
    """Surface of the reference's searcher/base.py:4-6."""

    def search(self, query, threshold, indexer, scaling=None):
        raise NotImplementedError

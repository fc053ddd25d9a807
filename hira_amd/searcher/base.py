"""The searcher contract of this path (the reference declares it in searcher/base.py:4-6).

``search`` answers a halfspace range query per query head: which indexed keys score at least
``threshold`` against the head's query.  What it returns is the reference's dense form: a
(H_q, N) tensor holding ``score * scaling`` at the selected keys and a fill value elsewhere.
"""
import abc


class BaseSearcher(abc.ABC):
    @abc.abstractmethod
    def search(self, query, threshold, indexer, scaling=None):
        """``query`` (H_q, D) or (B, H_q, 1, D); ``threshold`` scalar or (H_q,); ``indexer`` a
        built index; ``scaling`` None or (H_q,) factors applied to the returned scores."""

"""The indexer contract of this path (the reference declares it in indexer/base.py:5-10).

An indexer owns one ball tree per (sequence, KV head).  ``build`` takes the keys (and values)
of a prompt, ``update`` appends keys in the order given; both return the indexer itself so
that calls chain, as the reference's implementations do (indexer/cpu.py:122, 190).
"""
import abc


class BaseIndexer(abc.ABC):
    #: keys handed to the index so far, per tree
    num_keys: int = 0

    @abc.abstractmethod
    def build(self, keys, values=None):
        """Index ``keys`` (B, H_kv, L, D); ``values`` (B, H_kv, L, Dv) ride along with their
        keys when given.  Returns ``self``."""

    @abc.abstractmethod
    def update(self, new_keys, values=None):
        """Append ``new_keys`` (B, H_kv, m, D) (and their values) to a built index, in order.
        Returns ``self``."""

"""TEST INFRASTRUCTURE: CPU restatements of the reference's algorithms for the hot path.
Importable only from tests, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU baseline."""

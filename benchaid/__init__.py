"""Measurement aids of ``bench.py``: the gather probe (a kernel that only fetches the rows a
batch looks up), the copy kernel that calibrates memory counters, and the record of
counter-measured memory traffic per prebuilt library.  Nothing in ``recflex_amd`` imports this
package; only ``bench.py``, ``__graft_entry__.build()`` and the tests of these aids do."""

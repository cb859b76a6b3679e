"""CPU oracle for the compressed-BF16 linear path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this directory: it is the checker used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``.  Everything here is plain numpy restating either

* the reference's own algorithm and data layout (``planes``, ``ref_tables``,
  ``ref_layout``: files ``utils.py``, ``huffman.py``, ``ans.py``,
  ``functional.py`` and ``src/kernel.cu`` of lszxb/bf16_huffman_infer), or
* the wave64 stream format the HIP kernels of this repository consume
  (``wave64``), written as an executable specification.

How each function is pinned is stated in the header of its module.
"""

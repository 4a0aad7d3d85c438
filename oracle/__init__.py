"""CPU oracle for the LL128 + ring collective data path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: it is the checker used by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``.  It restates, on the CPU with
numpy / torch-CPU, the semantics of the reference's device path:

* ``ll128.py``    - the LL128 line format (reference ``protocol.py:42-100``,
                    ``2_sendrecv_indirect.py:61-93``) in the reference's
                    8-lane "pair" layout and in the 64-lane "wave64" layout the
                    HIP kernels put on the wire.
* ``ring.py``     - element arithmetic (``primitive.py:232-247``) and the ring
                    collectives' results in the reference's fold order
                    (``4_broadcast.py:61-72``, ``5_reduce.py:70-89``,
                    ``6_allgather.py:56-74``, ``7_reducescatter.py:54-73``).
* ``flowmodel.py``- an explicit-state model of the slot / credit flow control
                    that replaces ``protocol.py:161-189``.
* ``topology.py`` - ring / route search (``topology.py:23-93``).
* ``ll128_ref.c`` - an integer-only C restatement of the codec and of the
                    fp16 / bf16 add, used to cross-check the numpy code.

Pinning status of every function is stated in its module docstring.
"""

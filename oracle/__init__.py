"""CPU checkers for the darknet forward path (test infrastructure, never shipped).

``oracle.cpu``   ctypes bindings to this repository's own C restatement (``liboracle.so``).
``oracle.cfg``   restatement of the reference's cfg grammar and layer geometry rules.
``oracle.net``   a forward_network loop over a parsed layer table, built on ``oracle.cpu``.
``oracle.ref``   bindings to the *compiled reference* under ``oracle/_ref`` (optional).

Only tests/, ``__graft_entry__.smoke()`` and bench.py's ``cpu_baseline`` leg import this package.
"""

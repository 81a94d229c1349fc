"""CPU oracle for the ReBeL search hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package (``poker2_amd``)
may import, call or link anything in this directory.  The only permitted users
are ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py``, and there only as the checker or as the timed CPU baseline,
never as a compute path that ships.

Every function restates, in numpy (plus a small C file for the integer
ranker), what the reference computes, and cites the reference file:line it
follows.  How each function is pinned (reference-held vectors, golden fixtures
written by running the reference's own ``rules.py`` / ``hunl_tensor_env.py`` /
``sparse_cfr_evaluator.py`` in the build container, closed forms, brute force) is
listed per module.

Parity status
-------------
* cards, ranker, unblocked mass, showdown, betting tree: pinned (see modules).
* cfr, warm start, best response / exploitability: pinned by vectors written from the
  reference's own evaluator (``tests/golden/cfr_golden.npz``) and by an explicit hand-pair
  game (see ``oracle/cfr.py``, ``oracle/best_response.py``).
* chance nodes (one card, flop): pinned by vectors written from the reference's own helper
  (``tests/golden/chance_golden.npz``, ``flop_chance_golden.npz``), per-sample loops and closed
  forms (``oracle/chance.py``).
* feature encoding and training targets: pinned by vectors written from the reference's own
  evaluator, encoder and chance helper (``tests/golden/training_data_golden.npz``; ``oracle/datagen.py``).
"""

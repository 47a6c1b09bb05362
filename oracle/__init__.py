"""TEST INFRASTRUCTURE ONLY: CPU checkers for the RNN-T mutual-information path.

``oracle.mi``   - C restatement (and, where built, the compiled reference) of the MI recursion.
``oracle.rnnt`` - numpy restatement of the surrounding rnnt_loss.py op chains.

The product package never imports this; only tests, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do.
"""

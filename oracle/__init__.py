"""CPU restatement of DeltaCNN's sparse delta-propagation path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory; it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported baseline.

``delta_ops``    functional restatement of every operator on the path
``delta_layers`` stateful layer protocol (first frame, caches, thresholds)
"""

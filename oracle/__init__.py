"""CPU oracle for ragged paged attention -- TEST INFRASTRUCTURE ONLY.

Nothing under this directory is part of the product path.  It may be imported
only by the test-suite, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``; the shipped operators never call it and
raise when the HIP library is missing.
"""

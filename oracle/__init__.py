"""TEST INFRASTRUCTURE ONLY: CPU oracles for the projection and scoring paths.

Nothing under trak_amd/ imports this package.  tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py are its only users.
"""

"""CPU checker for the elementwise and reduction path.  Test infrastructure
only: imported by tests/, by __graft_entry__.smoke() and by the CPU leg of
bench.py, never by the library."""

"""CPU oracle for the NativeLstm2 forward op -- test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package.  Nothing under returnn_amd/ does.
"""

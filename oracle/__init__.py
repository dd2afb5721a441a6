"""CPU oracle for the LSTM forward/backward path -- test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this package; the product (fastlstm_amd/) never does.
"""

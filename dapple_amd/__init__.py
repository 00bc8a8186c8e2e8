"""MI355X-native DAPPLE pipeline-stage runtime (one stage, one GPU).

Host code is Python; all compute goes through the C-ABI of
``csrc/libdapple_hip.so`` (declared in include/dapple_stage.h).
"""
__version__ = "0.1.0"

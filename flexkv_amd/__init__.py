"""flexkv_amd — GPU<->CPU KV-cache block transfer for AMD Instinct MI355X.

``flexkv_amd.c_ext`` carries the operator names of FlexKV's ``flexkv.c_ext`` for
this path; ``flexkv_amd.layout`` the layout/stride arithmetic its workers use;
``flexkv_amd.host_buffer`` the pinned host-pool helpers.  Importing ``c_ext`` or
``host_buffer`` loads ``libfkv_hip.so`` and fails if it has not been built.
"""
__version__ = "0.1.0"

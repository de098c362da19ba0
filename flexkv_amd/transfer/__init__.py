"""Worker-process harness around the GPU<->CPU transfer operators.

Host-side mirror of the part of FlexKV's ``flexkv/transfer`` and
``flexkv/common`` packages that sits directly on this path: the transfer-op
records, the shared block-id buffer, the worker processes with their completion
reports and trace lines, and the handles that carry an engine's KV tensors into
a worker process.
"""

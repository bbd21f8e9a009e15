"""Declaration and agreement layer: registry, arch tag, contract build, handshake, install fingerprint.

Mirrors the reference's ``isoexec/core`` surface for the accelerated path (core/registry.py,
core/arch.py, core/contract_build.py, core/process_contract.py, core/fingerprint.py,
core/enforce.py). Everything here runs on the host and imports no kernel code.
"""

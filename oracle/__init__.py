# SPDX-License-Identifier: Apache-2.0
"""TEST INFRASTRUCTURE: the CPU oracle of the load path.

``st_oracle`` restates the reference's header rules, slice algebra, rank blocks and
nogds reader in numpy / C so that the GPU path can be checked byte for byte.  Only
``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU baseline may import it;
nothing under ``fastsafetensors_amd/`` does.
"""

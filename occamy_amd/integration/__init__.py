"""Retargeting a checkout of the reference compiler at this runtime (see retarget.py)."""

"""Script-form tests in the reference's style: `python -m operators_amd.tests.<op> --amd`.

Counterparts of the reference's operatorspy/tests/{add,rms_norm,rotary_embedding,swiglu}.py:
the same case tables, the same torch formulas as the second opinion, the same
tolerances, run against the amd-gpu device through the C ABI.  They need a GPU
and print one line per case, as the reference's scripts do.
"""

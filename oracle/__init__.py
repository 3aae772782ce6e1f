"""CPU oracle for the SNN-TC ops: test infrastructure, never part of the shipped path.

Only the test-suite, the smoke check and the benchmark's ``cpu_baseline`` leg may import this
package.  ``oracle.capi`` binds the C restatement (``snntc_oracle.c``); ``oracle.closed_form``
holds independent numpy statements used to pin the C restatement.
"""

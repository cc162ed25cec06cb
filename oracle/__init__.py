"""CPU oracle for the PAM arithmetic path -- test infrastructure only.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this
package; the shipped library never does.
"""

"""CPU oracle for the approximate-multiplier hot path (TEST INFRASTRUCTURE).

Only tests/, the smoke check and the bench's cpu_baseline leg may import this
package.  The shipped library never does.
"""

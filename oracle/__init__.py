"""CPU oracle for the HiP attention hot path -- test infrastructure only, never shipped."""

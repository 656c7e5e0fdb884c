"""CPU oracle for the Q8_0 x Q8_1 linear path.  Test infrastructure only."""

"""CPU oracle for the pcieThrough data-movement path. Test infrastructure only."""

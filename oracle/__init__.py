"""CPU oracle for the BTP hot path. Test infrastructure: never imported by the shipped package."""

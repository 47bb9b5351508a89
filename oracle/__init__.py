"""CPU oracle for the bidirectional SSD path.  Test infrastructure only: nothing that ships imports it."""

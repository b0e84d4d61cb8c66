"""CPU oracle for the attention path. Test infrastructure only; never imported by axlearn_amd."""

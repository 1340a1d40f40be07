"""CPU oracle of the block-sparse compute path.  Test infrastructure only: nothing under
``blksprs_amd/`` imports it."""

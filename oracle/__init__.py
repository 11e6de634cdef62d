"""TEST INFRASTRUCTURE: CPU oracle for the grouped attention path. Not product code."""

"""TEST INFRASTRUCTURE: CPU oracle for the lego_hip hot path.  Never imported by lego_amd."""

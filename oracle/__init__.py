"""TEST INFRASTRUCTURE: CPU oracle for the MI355X backend. Never imported by tensorfrost_amd."""

"""Test-only CPU oracle for the DAX W8A8 linear.  Never imported by dax_amd."""

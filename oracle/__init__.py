"""Test infrastructure: CPU restatements of the reference's forward path.  Never imported by the product package."""

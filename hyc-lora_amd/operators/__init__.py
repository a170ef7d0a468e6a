"""host-side mirror of the reference operator API (filled in below)"""

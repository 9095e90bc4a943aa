"""Graph inputs: COO to canonical CSR on the device (``csr``), the Planetoid-format
dataset wrapper (``dataset``) and the seeded synthetic generators (``graphgen``)."""

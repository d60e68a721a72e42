"""Chunk-64 prefill of the gated delta rule (``pla.prefill`` drop-in): ``flashqla`` (GDN) and
``flashkdapro`` (KDA)."""

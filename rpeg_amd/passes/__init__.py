"""Graph passes under the reference's names (RPEG/passes): `unroll.unroll`, `lower.lower`."""

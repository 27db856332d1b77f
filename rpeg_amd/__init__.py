"""rpeg_amd: batched RPEG plan evaluation on AMD MI355X (gfx950)."""

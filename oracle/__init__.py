"""TEST INFRASTRUCTURE: CPU oracle for the gfx950 Thrust device system (never imported by the product)."""

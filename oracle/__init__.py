"""CPU oracle of the FlashGS forward path: test infrastructure, never imported by the product."""

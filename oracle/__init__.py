"""CPU oracle of the Plexus GCN hot path -- test infrastructure, never imported by the product."""

"""Host-side mirror of the reference's runtime/ package: operator layer and the HIP backends behind it."""

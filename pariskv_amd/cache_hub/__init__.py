"""Mirror of the reference's ``cache_hub`` package for the retrieval path."""

"""Test and benchmark support: seeded synthetic weights and models, a GGUF writer.  Nothing here is on the decode path."""

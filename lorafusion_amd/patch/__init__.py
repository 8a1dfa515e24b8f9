"""Mirror of ``lorafusion.patch``."""

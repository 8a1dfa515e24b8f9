"""Mirror of the part of ``lorafusion.utils`` that touches the hot path's neighbours."""

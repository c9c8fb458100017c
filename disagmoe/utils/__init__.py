"""Constants of the reference's ``disagmoe.utils`` that the expert path reads."""

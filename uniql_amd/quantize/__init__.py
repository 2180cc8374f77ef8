"""Drop-in counterparts of the reference's quantize/ layer modules."""

"""CPU oracle for the paged-KV operators. Test infrastructure: never imported by the product."""

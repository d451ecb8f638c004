"""CPU oracle for the SVDQuant kernel path: test infrastructure, never imported by the product package."""

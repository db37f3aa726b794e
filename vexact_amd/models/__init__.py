"""Model patch points of the reference's ``vexact.models`` package that sit on the hot path."""

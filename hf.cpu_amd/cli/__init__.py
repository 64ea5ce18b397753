"""The command line in the reference's manner: option table, wire protocol, operations."""

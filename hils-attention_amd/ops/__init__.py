"""Drop-in operator modules: same module and function names as the reference's ``ops`` package."""

"""`import shared` for code written against epfml/pam (shared/modules/factories.py): see shared.modules."""

"""TEST INFRASTRUCTURE — CPU oracle of the reference's operators.  Not imported by the product."""

"""TEST INFRASTRUCTURE -- CPU oracle for the DAG operators; never imported by the shipped package."""
